"""Shared helpers of the test-suite: seeded inputs of the five benchmark configurations and
the error figures the parity bar is written in."""
import numpy as np
import torch

from oracle import oracle

TOL_NORMWISE = 1e-5  # max|got - truth| / max|truth| against the float64 recurrence (fp32 kernels)


def make_inputs(shape, coeff_kind="uniform", seed=0, transposed=False):
    """x, c, dy as fp32 CPU tensors, drawn in this order from one seeded generator.
    coeff_kind: 'uniform' U[0,1) | 'near1' U[0.9,1) | 'sigmoid' sigmoid(N(2,1)) | 'signed' U(-1,1)."""
    g = torch.Generator().manual_seed(seed)
    base = tuple(reversed(shape)) if transposed else tuple(shape)

    def fin(t):
        return t.t() if transposed else t

    x = torch.randn(base, generator=g)
    if coeff_kind == "uniform":
        c = torch.rand(base, generator=g)
    elif coeff_kind == "near1":
        c = 0.9 + 0.1 * torch.rand(base, generator=g)
    elif coeff_kind == "sigmoid":
        c = torch.sigmoid(torch.randn(base, generator=g) + 2.0)
    elif coeff_kind == "signed":
        c = torch.rand(base, generator=g) * 2.0 - 1.0
    else:
        raise ValueError(coeff_kind)
    dy = torch.randn(base, generator=g)
    return fin(x), fin(c), fin(dy)


def truth(x, c, dy, reverse):
    """float64 sequential recurrence on the fp32 data: y, dx, dc (numpy float64)."""
    xn, cn, dyn = (t.detach().cpu().numpy() for t in (x, c, dy))
    y = oracle.fwd(xn, cn, reverse, dtype=np.float64)
    dx, dc = oracle.bwd(dyn, cn, y, reverse, dtype=np.float64)
    return y, dx, dc


TOL_MIXED_SHARE = 0.999  # share of elements within |d| <= 1e-5 |t| + 1e-5 rms(t) of the float64 recurrence


def check_close(got, want64, what, tol=TOL_NORMWISE, mixed_share=TOL_MIXED_SHARE):
    """The parity bar: the normwise figure (max|got - truth| / max|truth| <= tol), and next to it the
    elementwise mixed tolerance |d| <= 1e-5 |t| + 1e-5 rms(t), which all but a sliver of the elements
    must meet (a reassociated fp32 scan is a few roundoffs of the running bound off, which can exceed
    1e-5 of an element that happens to be tiny).  16-bit storage is held to the normwise bar alone:
    its rounding unit is far above 1e-5."""
    got = got.detach().double().cpu().numpy()
    assert got.shape == want64.shape, (what, got.shape, want64.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values in the result"
    rep = oracle.error_report(got, want64)
    assert rep["normwise"] <= tol, f"{what}: {rep}"
    if tol <= TOL_NORMWISE:
        assert rep["mixed"] >= mixed_share, f"{what}: {rep}"
    return rep
