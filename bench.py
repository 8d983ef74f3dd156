#!/usr/bin/env python3
"""Benchmark of the linear-recurrence scan on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--no-cpu]

One step = one forward + one backward pass of linrec over one batch of synthetic fp32 inputs that
already live in HBM (configuration C2 of the baseline: shape (512, 65536), inputs ~ N(0,1),
coeffs ~ U[0,1), output gradient ~ N(0,1), reverse=False).  The step runs the library's two
kernels through its C ABI, exactly what the registered operator and its autograd rule launch.

Prints ONE JSON line.  `value` is the achieved bandwidth of the step in algorithmic bytes
(forward 12 B/element: read inputs and coeffs, write outputs; backward 20 B/element: read
d_outputs, coeffs, outputs, write d_inputs, d_coeffs), i.e. 32 * elements / time per step.
`roofline` prices the dominant kernel (backward) against the 8 TB/s HBM peak with its duration
measured by HIP events on the launch stream; `roofline_fwd` does the same for the forward kernel.
`cpu_baseline` times the CPU checker's restatement of the reference's eager-torch host loop on this
box's cores, with a numpy and a multi-threaded C line beside it (reported baselines, not targets).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each scaled by
# what the same counter reads for the library's copy kernel of known size in the same run: x1.998 to x2.000 and
# x0.9989 to x0.9994), keyed
# by (configuration, kernel); a kernel the planner no longer picks for a configuration reports null.
MEASURED_TRAFFIC_BYTES = {
    ("C1", "tile_w8_s2_v4_MODE_FWD_0_0"): 3.195e6,
    ("C1", "tile_w8_s2_v4_MODE_BWD_1_0"): 5.362e6,
    ("C2", "drift_w8_s4_MODE_FWD_0"): 403.83e6,
    ("C2", "drift_w16_s2_MODE_FWD_0"): 403.61e6,
    ("C2", "drift_w8_s2_MODE_BWD_1"): 674.74e6,
    ("C2", "drift_w16_s1_MODE_BWD_1"): 675.45e6,
    ("C2", "stream_w8_s4_MODE_FWD_0"): 402.71e6,
    ("C2", "stream_w8_s4_MODE_BWD_1"): 671.42e6,
    ("C2", "sweep_w8_s4_MODE_BWD_1"): 673.19e6,
    ("C3", "tile_w4_s2_v4_MODE_FWD_1_0"): 402.58e6,
    ("C3", "tile_w4_s2_v4_MODE_BWD_0_0"): 676.67e6,
    ("C4", "drift_w8_s4_MODE_FWD_0"): 202.30e6,
    ("C4", "sweep_w8_s4_MODE_FWD_0"): 202.13e6,
    ("C4", "sweep_w8_s8_MODE_BWD_1"): 336.69e6,
    ("C4", "drift_w16_s1_MODE_BWD_1"): 338.40e6,
    ("C5", "column_v2_u8_MODE_FWD_0"): 805.12e6,
    ("C5", "column_v2_u8_MODE_BWD_1"): 1340.78e6,
    ("C2", "bf16_stream_w8_s2_MODE_FWD_0"): 201.40e6,
    ("C2", "bf16_stream_w8_s2_MODE_BWD_1"): 335.63e6,
    ("C2", "bf16_drift_w16_s2_MODE_FWD_0"): 202.14e6,
    ("C2", "bf16_drift_w16_s1_MODE_BWD_1"): 337.22e6,
    ("C4", "bf16_drift_w16_s2_MODE_FWD_0"): 101.29e6,
    ("C4", "bf16_drift_w16_s1_MODE_BWD_1"): 169.01e6,
    # the three launches of a segmented scan together (reduce + carry + apply): the inputs are read twice
    ("T1", "segment_apply_v2_u8_MODE_FWD_0"): 1352.9e6,
    ("T1", "colblock_v1_u8_g2_MODE_FWD_0"): 805.16e6,
    # column drift kernels: the steps' maps that team mates exchange add 5.5 % forward, 3.3 % backward
    ("T1", "coldrift_w16_v1_u8_MODE_FWD_0"): 849.78e6,
    ("T1", "coldrift_w8_v1_u16_MODE_BWD_1"): 1387.0e6,
    ("T2", "colblock_v2_u8_g2_MODE_FWD_1"): 402.70e6,
    ("T2", "colblock_v2_u4_g2_MODE_BWD_0"): 670.96e6,
    ("T1", "segment_apply_v2_u8_MODE_BWD_1"): 1889.5e6,
}
FWD_BYTES_PER_ELEM = 12
BWD_BYTES_PER_ELEM = 20

CONFIGS = {
    "C1": dict(shape=(64, 4096), coeffs="uniform", reverse=False, transposed=False),
    "C2": dict(shape=(512, 65536), coeffs="uniform", reverse=False, transposed=False),
    "C3": dict(shape=(16384, 2048), coeffs="sigmoid", reverse=True, transposed=False),
    "C4": dict(shape=(16, 1048576), coeffs="near1", reverse=False, transposed=False),
    "C5": dict(shape=(262144, 256), coeffs="uniform", reverse=False, transposed=True),
    # not one of the reference's configurations: time-major data (16384 timesteps x 4096 channels seen
    # as 4096 rows), which the column drift kernels serve
    "T1": dict(shape=(4096, 16384), coeffs="uniform", reverse=False, transposed=True),
    # C3's tensor kept time-major (2048 timesteps x 16384 channels seen as 16384 rows): the column block kernels
    "T2": dict(shape=(16384, 2048), coeffs="sigmoid", reverse=True, transposed=True),
}


def make_set(torch, cfg, seed, dev):
    """x, c, dy drawn on the CPU from a seeded generator (so a CPU run sees the same bits), moved
    to the device, plus result buffers of the same layout."""
    g = torch.Generator().manual_seed(seed)
    shape = cfg["shape"]
    base = tuple(reversed(shape)) if cfg["transposed"] else shape
    x = torch.randn(base, generator=g)
    if cfg["coeffs"] == "uniform":
        c = torch.rand(base, generator=g)
    elif cfg["coeffs"] == "near1":
        c = 0.9 + 0.1 * torch.rand(base, generator=g)
    else:
        c = torch.sigmoid(torch.randn(base, generator=g) + 2.0)
    dy = torch.randn(base, generator=g)
    host = [t.t() if cfg["transposed"] else t for t in (x, c, dy)]
    devt = [t.to(dev) for t in host]
    devt = [t if t.stride() == h.stride() else torch.empty_strided(h.size(), h.stride(), device=dev).copy_(h)
            for t, h in zip(devt, host)]
    outs = [torch.empty_strided(devt[0].size(), devt[0].stride(), device=dev) for _ in range(3)]
    return host, devt, outs


def event_time_ms(torch, fn, iters):
    """Average duration of fn() over `iters` back-to-back calls, by HIP events on the current stream."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def event_series_ms(torch, fn, iters):
    """Durations of `iters` back-to-back calls of fn(), one HIP event between every two of them."""
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(iters):
        fn(i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    return sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(iters))


def cpu_baseline(cfg, host, budget_s=20.0):
    """The reference's host path on this box's cores, restated by the CPU checker and timed on a bounded
    sample of the same workload (a reported baseline, not a target): the eager-torch loop as the
    reference writes it (one multiply-add over all rows per timestep, linrec/impl/python/ops.py:16-18
    and :32-40), with torch's thread count; the same loop in numpy; and a plain C loop per row with the
    rows spread over OpenMP threads."""
    import numpy as np
    import torch
    from oracle import oracle
    xt, ct, dyt = host
    n, L = xt.shape
    # bound the sample: one probe of a few hundred timesteps, then as many timesteps as fit the budget
    probe = min(L, 512)
    t0 = time.perf_counter()
    oracle.fwd_torch(xt[:, :probe], ct[:, :probe], cfg["reverse"])
    per_step = (time.perf_counter() - t0) / probe
    L_s = L if per_step * L * 2.6 <= budget_s else max(1, int(budget_s / (per_step * 2.6)))
    xs, cs, dys = xt[:, :L_s], ct[:, :L_s], dyt[:, :L_s]
    elems = n * L_s
    gb = (FWD_BYTES_PER_ELEM + BWD_BYTES_PER_ELEM) * elems / 1e9
    sample = f"fwd+bwd of all {n} rows, timesteps[:{L_s}] of the same inputs"

    def timed(fn, at_least_s):
        """Average time of one pass; passes are repeated until `at_least_s` seconds have gone by."""
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            spent = time.perf_counter() - t0
            if spent >= at_least_s:
                return spent / reps, reps

    def torch_pass():
        y = oracle.fwd_torch(xs, cs, cfg["reverse"])
        oracle.bwd_torch(dys, cs, y, cfg["reverse"])

    xn, cn, dyn = (t.numpy() for t in (xs, cs, dys))

    def numpy_pass():
        yn = oracle.fwd_numpy(xn, cn, cfg["reverse"], dtype=np.float32)
        oracle.bwd_numpy(dyn, cn, yn, cfg["reverse"], dtype=np.float32)

    def c_pass():
        yc = oracle.fwd(xn, cn, cfg["reverse"], dtype=np.float32)
        oracle.bwd(dyn, cn, yc, cfg["reverse"], dtype=np.float32)

    t_torch, r_torch = timed(torch_pass, 0.35 * budget_s)
    t_np, r_np = timed(numpy_pass, 0.2 * budget_s)
    threads = oracle.threads()
    c_pass()  # (the threads start up outside the timed passes)
    t_c, r_c = timed(c_pass, 0.15 * budget_s)
    cpus = os.cpu_count()
    return ({"value": gb / t_torch, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
             "sample": f"{sample}, eager-torch loop over timesteps (the reference's host path), {r_torch} passes of "
                       f"{t_torch:.2f} s, torch.get_num_threads() = {torch.get_num_threads()}, host has {cpus} cpus"},
            {"value": gb / t_np, "unit": "GB/s", "cores": 1, "kind": "port",
             "sample": f"same sample, the same loop in numpy, {r_np} passes of {t_np:.2f} s"},
            {"value": gb / t_c, "unit": "GB/s", "cores": threads, "kind": "port",
             "sample": f"same sample, sequential C loop per row, rows over {threads} OpenMP threads "
                       f"(includes the wrapper's allocation of the results), {r_c} passes of {t_c:.3f} s"})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--config", default="C2", choices=sorted(CONFIGS))
    ap.add_argument("--sets", type=int, default=3, help="distinct buffer sets rotated through (defeats the last-level cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"],
                    help="storage type of the tensors (arithmetic is fp32); the headline workload is f32")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build targets one GPU per process and measures one GPU; run with --gpus 1 "
                 "(rows shard across GPUs without communication, so N GPUs run N copies of this workload)")

    import torch
    import __graft_entry__
    __graft_entry__.ensure_built()  # loads what is built; builds only a tree in which nothing is
    import linrec_amd
    from linrec_amd import _native

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = CONFIGS[a.config]
    rev = cfg["reverse"]
    elems = cfg["shape"][0] * cfg["shape"][1]

    tdtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[a.dtype]
    esize = 4 if a.dtype == "f32" else 2
    fwd_bpe, bwd_bpe = 3 * esize, 5 * esize  # algorithmic bytes per element
    sets = [make_set(torch, cfg, seed, dev) for seed in range(a.sets)]
    if a.dtype != "f32":
        sets = [(h, [t.to(tdtype) for t in d], [t.to(tdtype) for t in o]) for h, d, o in sets]
        for _, d, o in sets:
            assert all(t.stride() == d[0].stride() for t in d + o)
    host0 = sets[0][0]

    def fwd(i):
        _, (x, c, dy), (y, dx, dc) = sets[i % len(sets)]
        _native.fwd(x, c, rev, out=y)

    def bwd(i):
        _, (x, c, dy), (y, dx, dc) = sets[i % len(sets)]
        _native.bwd(dy, c, y, rev, out=(dx, dc))

    def step(i):
        fwd(i)
        bwd(i)

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / a.steps
    value = (fwd_bpe + bwd_bpe) * elems / (ms_per_step * 1e-3) / 1e9

    # per-kernel durations by HIP events on the launch stream
    k_iters = max(20, a.steps)
    fwd_ms = event_time_ms(torch, fwd, k_iters)
    bwd_ms = event_time_ms(torch, bwd, k_iters)
    fwd_gbps = fwd_bpe * elems / (fwd_ms * 1e-3) / 1e9
    bwd_gbps = bwd_bpe * elems / (bwd_ms * 1e-3) / 1e9
    # spread of the step: the same loop once more with an event after every step
    series = event_series_ms(torch, step, k_iters)

    # the operator path a user takes: linrec_amd.linrec + autograd (allocates its results)
    xg = [s[1][0].detach().requires_grad_() for s in sets]
    cg = [s[1][1].detach().requires_grad_() for s in sets]

    def op_step(i):
        k = i % len(sets)
        y = linrec_amd.linrec(xg[k], cg[k], rev)
        torch.autograd.grad(y, (xg[k], cg[k]), sets[k][1][2])

    # (the first dozens of calls through autograd are slower than the steady state: its device thread, the
    # allocator's pools and the binding's repeat-call tables warm up)
    for i in range(60):
        op_step(i)
    op_ms = event_time_ms(torch, op_step, max(100, a.steps))

    # what the same step costs with an operator of torch's own in the place of the scan (an elementwise product):
    # the floor that autograd's bookkeeping and its device thread set for any two-launch step
    def floor_step(i):
        k = i % len(sets)
        y = xg[k] * cg[k]
        torch.autograd.grad(y, (xg[k], cg[k]), sets[k][1][2])

    for i in range(60):
        floor_step(i)
    floor_ms = event_time_ms(torch, floor_step, max(100, a.steps))

    # measured ceilings: streaming kernels without a scan, same access pattern, fp32 streams of the
    # tensors' byte size: a plain copy, and the forward's (2 in, 1 out) and backward's (3 in, 2 out) mixes
    copy_gbps = mix_fwd_gbps = mix_bwd_gbps = None
    if sets[0][1][0].is_contiguous():
        nflt = elems * esize // 4
        srcs = [[torch.randn(nflt, device=dev) for _ in range(3)] for _ in sets]
        dsts = [[torch.empty(nflt, device=dev) for _ in range(2)] for _ in sets]
        ns = len(sets)
        for i in range(5):
            _native.copy(srcs[i % ns][0], dsts[i % ns][0])
        cp_ms = event_time_ms(torch, lambda i: _native.copy(srcs[i % ns][0], dsts[i % ns][0]), k_iters)
        copy_gbps = 8 * nflt / (cp_ms * 1e-3) / 1e9
        mf_ms = event_time_ms(torch, lambda i: _native.stream_mix(srcs[i % ns][:2], dsts[i % ns][:1]), k_iters)
        mb_ms = event_time_ms(torch, lambda i: _native.stream_mix(srcs[i % ns], dsts[i % ns]), k_iters)
        mix_fwd_gbps = 12 * nflt / (mf_ms * 1e-3) / 1e9
        mix_bwd_gbps = 20 * nflt / (mb_ms * 1e-3) / 1e9
        del srcs, dsts

    plan_f = _native.plan(sets[0][1][0], rev, False)
    plan_b = _native.plan(sets[0][1][0], rev, True)
    names = _native.kernel_table()

    out = {
        "metric": "linrec fwd+bwd achieved HBM GB/s (algorithmic bytes), %s %dx%d" % (
            {"f32": "fp32", "f16": "fp16", "bf16": "bf16"}[a.dtype], *cfg["shape"]),
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "ms_per_step_median": round(series[len(series) // 2], 5),
        "ms_per_step_min": round(series[0], 5),
        "ms_per_step_max": round(series[-1], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": a.dtype,
        "data": "synthetic",
        "config": {"workload": f"{a.config}: linrec forward+backward, {a.dtype} {cfg['shape']}, coeffs {cfg['coeffs']}, "
                               f"reverse={rev}, {'transposed view' if cfg['transposed'] else 'contiguous'}; "
                               f"{a.sets} rotating buffer sets", "elements": elems},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "elements_per_s": round(elems / (ms_per_step * 1e-3), 1),
        "roofline": {"bound": "hbm", "kernel": names[plan_b["kernel_id"]], "achieved": round(bwd_gbps, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(bwd_gbps / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get((a.config, names[plan_b["kernel_id"]])),
                     "avg_kernel_ms": round(bwd_ms, 5),
                     "algorithmic_bytes_per_launch": bwd_bpe * elems},
        "roofline_fwd": {"bound": "hbm", "kernel": names[plan_f["kernel_id"]], "achieved": round(fwd_gbps, 1),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(fwd_gbps / HBM_PEAK_GBPS, 4),
                         "traffic": MEASURED_TRAFFIC_BYTES.get((a.config, names[plan_f["kernel_id"]])),
                         "avg_kernel_ms": round(fwd_ms, 5),
                         "algorithmic_bytes_per_launch": fwd_bpe * elems},
        "operator_path": {"ms_per_step": round(op_ms, 5),
                          "GBps": round((fwd_bpe + bwd_bpe) * elems / (op_ms * 1e-3) / 1e9, 1),
                          "what": "linrec_amd.linrec + torch.autograd.grad, results allocated per call",
                          "same_step_with_torch_mul_ms": round(floor_ms, 5)},
        "copy_ceiling_GBps": None if copy_gbps is None else round(copy_gbps, 1),
        "stream_mix_ceiling_GBps": None if mix_fwd_gbps is None else {
            "fwd_2_in_1_out": round(mix_fwd_gbps, 1), "bwd_3_in_2_out": round(mix_bwd_gbps, 1),
            "what": "streaming kernel with the pass's mix of read and write streams and no scan"},
        "plan_fwd": plan_f, "plan_bwd": plan_b,
        "device": torch.cuda.get_device_name(0),
    }
    if not a.no_cpu and a.dtype == "f32":
        lines = cpu_baseline(cfg, host0)
        for key, line in zip(("cpu_baseline", "cpu_baseline_numpy", "cpu_baseline_c_loop"), lines):
            out[key] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in line.items()}
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
