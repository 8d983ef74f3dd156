"""Pins the CPU checker (oracle/) before anything is compared against it.

The reference holds no golden vectors for this path, so the checker is pinned by
(1) hand-computed known answers (tests/golden/known_answers.json),
(2) closed forms that reduce to library routines (cumsum, cumprod, an IIR filter),
(3) invariants (linearity, flip equivalence, chunk composition, row independence),
(4) for the backward: autograd through an explicit O(L^2) sum that shares no code or
    formula with the scan, and central finite differences.
Each check is chosen so that a dropped term, an off-by-one shift or a swapped direction fails it.
"""
import json
import os

import numpy as np
import pytest
import scipy.signal
import torch

from oracle import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")


def _fwd_torch(x, c, reverse=False, dtype=np.float64):
    t = [torch.from_numpy(np.ascontiguousarray(a, dtype=dtype)) for a in (x, c)]
    return oracle.fwd_torch(*t, reverse=reverse).numpy()


def _bwd_torch(dy, c, y, reverse=False, dtype=np.float64):
    t = [torch.from_numpy(np.ascontiguousarray(a, dtype=dtype)) for a in (dy, c, y)]
    return tuple(r.numpy() for r in oracle.bwd_torch(*t, reverse=reverse))


IMPLS = [("c", oracle.fwd, oracle.bwd), ("numpy", oracle.fwd_numpy, oracle.bwd_numpy),
         ("torch", _fwd_torch, _bwd_torch)]


def _cases():
    with open(GOLDEN) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("impl", IMPLS, ids=lambda t: t[0])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_known_answers(impl, case, dtype):
    _, fwd, bwd = impl
    x, c = np.array(case["x"], dtype=dtype), np.array(case["c"], dtype=dtype)
    y = fwd(x, c, reverse=case["reverse"], dtype=dtype)
    np.testing.assert_array_equal(y, np.array(case["y"], dtype=dtype))
    if "dy" in case:
        dx, dc = bwd(np.array(case["dy"], dtype=dtype), c, y, reverse=case["reverse"], dtype=dtype)
        np.testing.assert_array_equal(dx, np.array(case["dx"], dtype=dtype))
        np.testing.assert_array_equal(dc, np.array(case["dc"], dtype=dtype))


def _rand(shape, seed, lo=0.0, hi=1.0):
    rng = np.random.default_rng(seed)
    return rng.standard_normal(shape), rng.uniform(lo, hi, shape)


@pytest.mark.parametrize("impl", IMPLS, ids=lambda t: t[0])
@pytest.mark.parametrize("reverse", [False, True])
class TestClosedForms:
    def test_zero_coeffs_is_identity(self, impl, reverse):
        x, _ = _rand((3, 37), 1)
        np.testing.assert_array_equal(impl[1](x, np.zeros_like(x), reverse=reverse), x)

    def test_unit_coeffs_is_cumsum(self, impl, reverse):
        x, _ = _rand((4, 129), 2)
        want = np.flip(np.cumsum(np.flip(x, -1), -1), -1) if reverse else np.cumsum(x, -1)
        np.testing.assert_allclose(impl[1](x, np.ones_like(x), reverse=reverse), want, rtol=1e-12, atol=1e-12)

    @pytest.mark.parametrize("r", [0.5, -0.9, 1.1])
    def test_constant_coeff_is_one_pole_filter(self, impl, reverse, r):
        x, _ = _rand((2, 200), 3)
        xin = np.flip(x, -1) if reverse else x
        want = scipy.signal.lfilter([1.0], [1.0, -r], xin, axis=-1)
        want = np.flip(want, -1) if reverse else want
        np.testing.assert_allclose(impl[1](x, np.full_like(x, r), reverse=reverse), want, rtol=1e-10, atol=1e-10)

    def test_impulse_gives_cumprod_of_later_coeffs(self, impl, reverse):
        _, c = _rand((3, 50), 4, 0.5, 1.5)
        x = np.zeros_like(c)
        if reverse:
            x[:, -1] = 1.0
            cc = np.flip(c, -1).copy()
        else:
            x[:, 0] = 1.0
            cc = c.copy()
        cc[:, 0] = 1.0  # the first coefficient in scan order takes no part
        want = np.cumprod(cc, -1)
        want = np.flip(want, -1) if reverse else want
        np.testing.assert_allclose(impl[1](x, c, reverse=reverse), want, rtol=1e-12)

    def test_zero_input_gives_zero(self, impl, reverse):
        _, c = _rand((2, 33), 5)
        assert not impl[1](np.zeros_like(c), c, reverse=reverse).any()


@pytest.mark.parametrize("impl", IMPLS, ids=lambda t: t[0])
@pytest.mark.parametrize("reverse", [False, True])
class TestInvariants:
    def test_linearity_in_inputs(self, impl, reverse):
        x1, c = _rand((3, 70), 6)
        x2, _ = _rand((3, 70), 7)
        lhs = impl[1](2.5 * x1 - 0.75 * x2, c, reverse=reverse)
        rhs = 2.5 * impl[1](x1, c, reverse=reverse) - 0.75 * impl[1](x2, c, reverse=reverse)
        np.testing.assert_allclose(lhs, rhs, rtol=1e-11, atol=1e-11)

    def test_reverse_is_flip_forward_flip(self, impl, reverse):
        x, c = _rand((3, 41), 8)
        a = impl[1](x, c, reverse=True)
        b = np.flip(impl[1](np.flip(x, -1), np.flip(c, -1), reverse=False), -1)
        np.testing.assert_array_equal(a, b)

    @pytest.mark.parametrize("k", [1, 2, 17, 63, 64])
    def test_chunk_composition(self, impl, reverse, k):
        # scanning a prefix, then restarting with the carry folded into the next input,
        # equals the full scan: pins every tile/carry scheme built on top of it
        x, c = _rand((2, 65), 9)
        if reverse:
            x, c = np.flip(x, -1), np.flip(c, -1)
        full = impl[1](x, c, reverse=False)
        head = impl[1](x[:, :k], c[:, :k], reverse=False)
        x_tail = x[:, k:].copy()
        x_tail[:, 0] += head[:, -1] * c[:, k]
        tail = impl[1](x_tail, c[:, k:], reverse=False)
        np.testing.assert_allclose(np.concatenate([head, tail], -1), full, rtol=1e-12, atol=1e-12)

    def test_rows_are_independent_and_first_coeff_unused(self, impl, reverse):
        x, c = _rand((4, 30), 10)
        base = impl[1](x, c, reverse=reverse)
        x2, c2 = x.copy(), c.copy()
        x2[1] = np.nan
        # the element loop never reads the first coefficient (linrec_ref.cuh:63); the per-timestep
        # loop multiplies it by prev = 0 (python/ops.py:11,17), so only finite values drop out there
        c2[2, -1 if reverse else 0] = np.inf if impl[0] == "c" else 12345.0
        got = impl[1](x2, c2, reverse=reverse)
        np.testing.assert_array_equal(got[[0, 2, 3]], base[[0, 2, 3]])
        assert np.isnan(got[1]).all()

    def test_nd_and_1d_shapes(self, impl, reverse):
        x, c = _rand((2, 3, 19), 11)
        y = impl[1](x, c, reverse=reverse)
        assert y.shape == x.shape
        np.testing.assert_array_equal(y[1, 2], impl[1](x[1, 2], c[1, 2], reverse=reverse))


def test_the_three_restatements_agree():
    for seed, shape in enumerate([(1, 1), (5, 2), (3, 257), (2, 4, 33)]):
        x, c = _rand(shape, 100 + seed, -1.2, 1.2)
        dy, _ = _rand(shape, 200 + seed)
        for reverse in (False, True):
            for dt in (np.float32, np.float64):
                y = oracle.fwd(x, c, reverse, dtype=dt)
                dx, dc = oracle.bwd(dy, c, y, reverse, dtype=dt)
                for _, fwd, bwd in IMPLS[1:]:
                    np.testing.assert_array_equal(y, fwd(x, c, reverse, dtype=dt))
                    dx2, dc2 = bwd(dy, c, y, reverse, dtype=dt)
                    np.testing.assert_array_equal(dx, dx2)
                    np.testing.assert_array_equal(dc, dc2)


def test_rows_on_several_threads_give_the_same_bits():
    """The C loops run rows on OpenMP threads; a row's arithmetic never crosses threads."""
    x, c = _rand((37, 501), 7, -1.1, 1.1)
    dy, _ = _rand((37, 501), 8)
    had = oracle.threads()
    try:
        oracle.threads(1)
        y1 = oracle.fwd(x, c, True, dtype=np.float32)
        b1 = oracle.bwd(dy, c, y1, True, dtype=np.float32)
        assert oracle.threads(4) == 4
        y4 = oracle.fwd(x, c, True, dtype=np.float32)
        b4 = oracle.bwd(dy, c, y4, True, dtype=np.float32)
    finally:
        oracle.threads(had)
    np.testing.assert_array_equal(y1, y4)
    np.testing.assert_array_equal(b1[0], b4[0])
    np.testing.assert_array_equal(b1[1], b4[1])


def _explicit_sum_torch(x, c, reverse):
    """y_l = sum_{k<=l} x_k * prod_{i=k+1..l} c_i, written as a double loop over torch scalars.
    Shares nothing with the scan (no running state, no shift)."""
    if reverse:
        x, c = x.flip(-1), c.flip(-1)
    L = x.shape[-1]
    cols = []
    for l in range(L):
        acc = torch.zeros_like(x[..., 0])
        for k in range(l + 1):
            term = x[..., k]
            for i in range(k + 1, l + 1):
                term = term * c[..., i]
            acc = acc + term
        cols.append(acc)
    y = torch.stack(cols, -1)
    return y.flip(-1) if reverse else y


@pytest.mark.parametrize("impl", IMPLS, ids=lambda t: t[0])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("L", [1, 2, 3, 9])
def test_backward_matches_autograd_of_explicit_sum(impl, reverse, L):
    g = torch.Generator().manual_seed(L)
    x = torch.randn(3, L, dtype=torch.float64, generator=g, requires_grad=True)
    c = (torch.rand(3, L, dtype=torch.float64, generator=g) * 2 - 1).requires_grad_()
    dy = torch.randn(3, L, dtype=torch.float64, generator=g)
    y = _explicit_sum_torch(x, c, reverse)
    np.testing.assert_allclose(impl[1](x.detach().numpy(), c.detach().numpy(), reverse=reverse),
                               y.detach().numpy(), rtol=1e-12, atol=1e-12)
    gx, gc = torch.autograd.grad(y, (x, c), dy, allow_unused=True)
    gc = torch.zeros_like(c) if gc is None else gc  # L == 1: no coefficient takes part
    dx, dc = impl[2](dy.numpy(), c.detach().numpy(), y.detach().numpy(), reverse=reverse)
    np.testing.assert_allclose(dx, gx.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(dc, gc.numpy(), rtol=1e-11, atol=1e-11)


@pytest.mark.parametrize("reverse", [False, True])
def test_backward_matches_finite_differences(reverse):
    x, c = _rand((2, 12), 12, -1.0, 1.0)
    dy, _ = _rand((2, 12), 13)
    y = oracle.fwd(x, c, reverse)
    dx, dc = oracle.bwd(dy, c, y, reverse)
    loss = lambda xx, cc: float((oracle.fwd(xx, cc, reverse) * dy).sum())
    eps = 1e-6
    for arr, grad, which in ((x, dx, 0), (c, dc, 1)):
        for idx in np.ndindex(arr.shape):
            up, dn = arr.copy(), arr.copy()
            up[idx] += eps
            dn[idx] -= eps
            num = (loss(up, c) - loss(dn, c)) if which == 0 else (loss(x, up) - loss(x, dn))
            assert abs(num / (2 * eps) - grad[idx]) < 1e-7, (which, idx)


def test_shift_is_roll_without_wraparound():
    a = np.arange(1.0, 7.0).reshape(1, 6)
    np.testing.assert_array_equal(oracle.shift_numpy(a, 1), [[0, 1, 2, 3, 4, 5]])
    np.testing.assert_array_equal(oracle.shift_numpy(a, -1), [[2, 3, 4, 5, 6, 0]])
    np.testing.assert_array_equal(oracle.shift_numpy(a, -2, fill=9), [[3, 4, 5, 6, 9, 9]])


def test_running_error_scale_bounds_fp32_sequential_error():
    # The fp32 sequential loop must sit within a few roundoffs of the float64 truth when
    # measured in units of S = linrec(|x|,|c|): this is the yardstick the GPU reports use.
    x, c = _rand((8, 4096), 14, 0.9, 1.0)
    x32, c32 = x.astype(np.float32), c.astype(np.float32)
    truth = oracle.fwd(x32, c32, dtype=np.float64)
    got = oracle.fwd(x32, c32, dtype=np.float32)
    rep = oracle.error_report(got, truth, oracle.running_error_scale(x32, c32))
    assert rep["reassoc"] < 4.0, rep
    assert rep["normwise"] < 1e-5, rep
