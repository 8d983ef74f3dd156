"""Python face of the CPU checker (test infrastructure, never on the product path).

Two independent restatements of the reference's recurrence live here:

* ``fwd`` / ``bwd``: ctypes calls into ``liblinrec_oracle.so`` (``linrec_oracle.c``), the
  element-by-element loop of linrec/impl/cuda/linrec_ref.cuh:53-94.
* ``fwd_numpy`` / ``bwd_numpy``: the per-timestep, all-rows-at-once loop of
  linrec/impl/python/ops.py:8-40 (``prev*c[i] + x[i]``, ``shift`` with fill 0), in numpy.

They are pinned against each other and against closed forms in tests/test_oracle_pins.py.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblinrec_oracle.so")
_lib = None


def build(force=False):
    """Compile linrec_oracle.c with gcc (a second or so)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liblinrec_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        i64, p, i = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        for sfx in ("f64", "f32"):
            getattr(lib, f"oracle_linrec_fwd_{sfx}").argtypes = [p, p, p, i64, i64, i64, i64, i]
            getattr(lib, f"oracle_linrec_fwd_{sfx}").restype = None
            getattr(lib, f"oracle_linrec_bwd_{sfx}").argtypes = [p, p, p, p, p, i64, i64, i64, i64, i]
            getattr(lib, f"oracle_linrec_bwd_{sfx}").restype = None
        lib.oracle_max_threads.restype = i
        lib.oracle_set_threads.argtypes = [i]
        _lib = lib
    return _lib


def threads(n=None):
    """Threads the C loops run rows on (OpenMP); `n` sets it.  Returns the number in force."""
    lib = _load()
    if n is not None:
        lib.oracle_set_threads(int(n))
    return int(lib.oracle_max_threads())


def _canon(*arrays, dtype):
    """Dense (numseq, L) copies in `dtype`; the scan runs over the last axis."""
    shape = arrays[0].shape
    out = []
    for a in arrays:
        a = np.asarray(a)
        assert a.shape == shape, (a.shape, shape)
        out.append(np.ascontiguousarray(a.reshape(-1, shape[-1]) if a.ndim else a.reshape(1, 1), dtype=dtype))
    return shape, out


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64"
    if dtype == np.float32:
        return "f32"
    raise TypeError(dtype)


def fwd(x, c, reverse=False, dtype=np.float64):
    """y[first] = x[first]; y[l] = y[l -/+ 1] * c[l] + x[l]; arithmetic in `dtype`."""
    shape, (x2, c2) = _canon(x, c, dtype=dtype)
    y2 = np.empty_like(x2)
    n, L = x2.shape
    if x2.size:
        getattr(_load(), f"oracle_linrec_fwd_{_sfx(dtype)}")(
            x2.ctypes.data, c2.ctypes.data, y2.ctypes.data, n, L, L, 1, int(bool(reverse)))
    return y2.reshape(shape)


def bwd(dy, c, y, reverse=False, dtype=np.float64):
    """(d_inputs, d_coeffs) of `fwd` given the output gradient, coeffs and saved outputs."""
    shape, (dy2, c2, y2) = _canon(dy, c, y, dtype=dtype)
    dx2, dc2 = np.empty_like(dy2), np.empty_like(dy2)
    n, L = dy2.shape
    if dy2.size:
        getattr(_load(), f"oracle_linrec_bwd_{_sfx(dtype)}")(
            dy2.ctypes.data, c2.ctypes.data, y2.ctypes.data, dx2.ctypes.data, dc2.ctypes.data,
            n, L, L, 1, int(bool(reverse)))
    return dx2.reshape(shape), dc2.reshape(shape)


def shift_numpy(a, shift, fill=0.0):
    """Roll along the last axis without wrap-around (linrec/impl/python/ops.py:22-30)."""
    out = np.full_like(a, fill)
    L = a.shape[-1]
    if shift > 0:
        out[..., shift:] = a[..., :L - shift]
    elif shift < 0:
        out[..., :L + shift] = a[..., -shift:]
    else:
        out[...] = a
    return out


def fwd_numpy(x, c, reverse=False, dtype=np.float64):
    """All rows per timestep, `prev = 0` start (linrec/impl/python/ops.py:8-20)."""
    x = np.asarray(x, dtype=dtype)
    c = np.asarray(c, dtype=dtype)
    y = np.zeros_like(x)
    prev = np.zeros(x.shape[:-1], dtype=dtype)
    order = range(x.shape[-1])
    for i in (reversed(order) if reverse else order):
        prev = prev * c[..., i] + x[..., i]
        y[..., i] = prev
    return y


def bwd_numpy(dy, c, y, reverse=False, dtype=np.float64):
    """shift + opposite-direction scan + multiply (linrec/impl/python/ops.py:32-40)."""
    dy = np.asarray(dy, dtype=dtype)
    c = np.asarray(c, dtype=dtype)
    y = np.asarray(y, dtype=dtype)
    cs = shift_numpy(c, -1 if not reverse else 1, 0.0)
    dx = fwd_numpy(dy, cs, reverse=not reverse, dtype=dtype)
    dc = dx * shift_numpy(y, 1 if not reverse else -1, 0.0)
    return dx, dc


def fwd_torch(x, c, reverse=False):
    """The reference's host path as it is written, in eager torch: one multiply-add over all rows per
    timestep and a column store (linrec/impl/python/ops.py:8-20).  `x`, `c`: CPU torch tensors."""
    import torch
    y = torch.empty_like(x)
    prev = torch.zeros_like(x[..., 0])
    order = range(x.shape[-1])
    for i in (reversed(order) if reverse else order):
        prev = prev * c[..., i] + x[..., i]
        y[..., i] = prev
    return y


def bwd_torch(dy, c, y, reverse=False):
    """shift, opposite-direction loop, multiply, in eager torch (linrec/impl/python/ops.py:22-40)."""
    import torch

    def shift(a, k):  # roll without wrap-around, fill 0
        out = torch.zeros_like(a)
        if k > 0:
            out[..., k:] = a[..., :-k]
        elif k < 0:
            out[..., :k] = a[..., -k:]
        return out

    dx = fwd_torch(dy, shift(c, -1 if not reverse else 1), reverse=not reverse)
    return dx, dx * shift(y, 1 if not reverse else -1)


def running_error_scale(x, c, reverse=False):
    """S = linrec(|x|, |c|) in float64: the magnitude the rounding errors of any evaluation
    order of the recurrence are proportional to (error <= k * 2^-24 * S for fp32)."""
    return fwd(np.abs(np.asarray(x, dtype=np.float64)), np.abs(np.asarray(c, dtype=np.float64)),
               reverse=reverse, dtype=np.float64)


def error_report(got, want64, scale=None, mixed_rtol=1e-5, mixed_atol=1e-5):
    """Error figures used by the parity tests; `got` fp32, `want64` float64 ground truth.

    normwise  = max|got - want| / max|want|          (headline bar: <= 1e-5)
    mixed     = share of elements with |got - want| <= rtol * |want| + atol * rms(want), rtol = atol = 1e-5
                (an elementwise bar: small values next to large ones cannot hide behind max|want|)
    maxabs    = max|got - want|                      (the reference's own figure, eval/test.py:24)
    reassoc   = max(|got - want| / (2^-24 * scale))  (in units of fp32 roundoff of the running bound)
    """
    got = np.asarray(got, dtype=np.float64)
    want64 = np.asarray(want64, dtype=np.float64)
    if got.size == 0:
        return {"normwise": 0.0, "maxabs": 0.0, "reassoc": 0.0, "mixed": 1.0}
    diff = np.abs(got - want64)
    denom = np.max(np.abs(want64))
    rms = float(np.sqrt(np.mean(want64 * want64)))
    rep = {"maxabs": float(diff.max()),
           "normwise": float(diff.max() / denom) if denom > 0 else float(diff.max()),
           "mixed": float(np.mean(diff <= mixed_rtol * np.abs(want64) + mixed_atol * rms))}
    if scale is not None:
        s = np.asarray(scale, dtype=np.float64)
        ok = s > 0
        rep["reassoc"] = float(np.max(diff[ok] / (2.0 ** -24 * s[ok]))) if ok.any() else 0.0
    return rep
