"""Builds the HIP library for gfx950 with hipcc, in-tree (linrec_amd/lib/liblinrec_hip.so).

Role of linrec/impl/cuda/build.py:56-80 in the reference (JIT build of the extension); here the
library is a torch-free shared object compiled directly by hipcc, so no torch build helper and no
source translation step is involved.  The kernels are compiled as several translation units side by
side (csrc/kernels_*.hip, one object each) and linked with the C ABI (csrc/linrec_capi.hip).

    python linrec_amd/build.py [-v] [--asm] [--incremental] [-j N]

Run it as a file (not with -m): importing the package itself requires the built library.
"""
import argparse
import concurrent.futures
import os
import re
import shutil
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIBNAME = "liblinrec_hip.so"
DRIVER = "linrec_driver"
SOURCES = ["linrec_capi.hip", "kernels_f32_rows.hip", "kernels_f32_teams.hip", "kernels_f32_walk.hip", "kernels_f32_cols.hip",
           "kernels_f16_rows.hip", "kernels_f16_cols.hip", "kernels_bf16_rows.hip", "kernels_bf16_cols.hip",
           "launch_model.hip", "linrec_host.cpp"]
ARCH = "gfx950"

FLAGS = [
    "-O3", "-std=c++20", "-fPIC", f"--offload-arch={ARCH}",
    "-fno-gpu-rdc", "-ffp-contract=off", "-Wall", "-Wno-unused-function", "-pthread",
    # packed fp32 VALU forms are switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the library can only be built on a ROCm image")
    return exe


def lib_path():
    return os.path.join(LIBDIR, LIBNAME)


def _local_includes(path, seen=None):
    """`path` and every file it includes with #include "..." (recursively), as absolute paths."""
    seen = set() if seen is None else seen
    path = os.path.normpath(path)
    if path in seen or not os.path.exists(path):
        return seen
    seen.add(path)
    with open(path) as f:
        for inc in re.findall(r'^\s*#\s*include\s+"([^"]+)"', f.read(), flags=re.M):
            _local_includes(os.path.join(os.path.dirname(path), inc), seen)
    return seen


def _stale(obj, src):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(dep) > t for dep in _local_includes(src) | {os.path.abspath(__file__)})


def build(verbose=False, save_asm=False, incremental=False, jobs=None):
    """Compile every kernel for gfx950 and link the shared library.  Returns its path.
    `incremental`: objects newer than their source and everything it includes are kept."""
    os.makedirs(OBJDIR, exist_ok=True)
    include = os.path.join(os.path.dirname(HERE), "include")
    t0 = time.time()

    def compile_one(src):
        path = os.path.join(CSRC, src)
        obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
        if incremental and not _stale(obj, path):
            return src, 0, "", 0.0
        cmd = [hipcc(), *FLAGS, "-I", include, "-c", path, "-o", obj]
        if save_asm:
            cmd += ["-save-temps=obj"]
        if verbose:
            cmd += ["-Rpass-analysis=kernel-resource-usage"]
        t = time.time()
        proc = subprocess.run(cmd, cwd=OBJDIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        return src, proc.returncode, proc.stdout, time.time() - t

    workers = jobs or min(len(SOURCES), max(1, min(16, os.cpu_count() or 1)))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        results = list(pool.map(compile_one, SOURCES))
    for src, rc, out, secs in results:
        if rc != 0:
            sys.stderr.write(out)
            raise RuntimeError(f"hipcc failed on {src} with exit code {rc}")
        if verbose:
            print(f"== {src}: {secs:.1f} s")
            print(out)
    out_path = lib_path()
    tmp = out_path + ".tmp"
    objs = [os.path.join(OBJDIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    link = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-pthread", "-o", tmp, *objs]
    proc = subprocess.run(link, cwd=LIBDIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError(f"hipcc failed to link with exit code {proc.returncode}")
    os.replace(tmp, out_path)
    # standalone driver for profilers (no Python in the process)
    drv = [hipcc(), "-O2", "-std=c++17", "-I", include,
           os.path.join(CSRC, "linrec_driver.cpp"), "-L", LIBDIR, "-llinrec_hip", "-Wl,-rpath,$ORIGIN",
           "-o", os.path.join(LIBDIR, DRIVER)]
    proc = subprocess.run(drv, cwd=LIBDIR, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError(f"hipcc failed on the driver with exit code {proc.returncode}")
    if verbose:
        print(f"built {out_path} and {DRIVER} in {time.time() - t0:.1f} s")
    return out_path


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("--asm", action="store_true", help="keep the gfx950 assembly next to the objects")
    ap.add_argument("--incremental", action="store_true", help="recompile only what changed")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    a = ap.parse_args()
    print(build(verbose=a.verbose, save_asm=a.asm, incremental=a.incremental, jobs=a.jobs))
