"""GPU tests through the public operator `linrec_amd.linrec` that follow the reference's own procedures:
its shape sweep (eval/test.py:10-30,40-57: tensors of shape (#SMs, 100, L) for L = 2^4 .. 2^10, both
directions, forward and `autograd.grad` with an explicit output gradient, maximum absolute difference to
the sequential recurrence), the `logc` option of its CPU entry point (linrec/impl/python/ops.py:8-14,
37-38) on device tensors, and what happens when a kernel's bounded wait for another workgroup runs out."""
import numpy as np
import pytest
import torch

import linrec_amd
from linrec_amd import _native as nat
from oracle import oracle

from .util import check_close

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("log2_len", range(4, 11))
def test_reference_shape_sweep(log2_len, reverse):
    L = 1 << log2_len
    shape = (256, 100, L)  # the reference takes the SM count for the first size; 256 CUs here
    g = torch.Generator().manual_seed(log2_len)
    x = torch.randn(shape, generator=g)
    c = torch.rand(shape, generator=g)
    dy = torch.randn(shape, generator=g)
    xd, cd = x.to(DEV).requires_grad_(), c.to(DEV).requires_grad_()
    y = linrec_amd.linrec(xd, cd, reverse)
    dx, dc = torch.autograd.grad(y, (xd, cd), dy.to(DEV))
    torch.cuda.synchronize()
    y_t = oracle.fwd(x.numpy(), c.numpy(), reverse, dtype=np.float64)
    dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y_t, reverse, dtype=np.float64)
    worst = 0.0
    for name, got, want in (("outputs", y, y_t), ("d_inputs", dx, dx_t), ("d_coeffs", dc, dc_t)):
        rep = check_close(got, want, f"(256, 100, {L}) reverse={reverse} {name}")
        worst = max(worst, rep["maxabs"])
    # the reference prints this figure (eval/test.py:24); for fp32 and these lengths it stays in the 1e-5 range
    print(f"L={L} reverse={reverse}: max abs difference {worst:.3e}", flush=True)
    assert worst < 1e-4
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("shape", [(64, 4096), (16, 131072), (5, 7, 300), (300, 20000)])
def test_coefficients_given_as_logarithms(shape, reverse):
    """linrec(x, log c, logc=True): the outputs of linrec(x, c), and the gradient with respect to the
    logarithms, d_coeffs * c.  The exponential runs on the device in fp32, so the coefficients the kernels
    see are the fp32 exponentials; the ground truth takes exactly those."""
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g)
    logc = torch.log(0.05 + 0.95 * torch.rand(shape, generator=g))
    dy = torch.randn(shape, generator=g)
    xd, ld = x.to(DEV).requires_grad_(), logc.to(DEV).requires_grad_()
    y = linrec_amd.linrec(xd, ld, reverse, logc=True)
    dx, dl = torch.autograd.grad(y, (xd, ld), dy.to(DEV))
    torch.cuda.synchronize()
    c_seen = torch.exp(logc.to(DEV)).cpu().numpy()
    y_t = oracle.fwd(x.numpy(), c_seen, reverse, dtype=np.float64)
    dx_t, dc_t = oracle.bwd(dy.numpy(), c_seen, y_t, reverse, dtype=np.float64)
    check_close(y, y_t, f"logc {shape} outputs")
    check_close(dx, dx_t, f"logc {shape} d_inputs")
    check_close(dl, dc_t * c_seen.astype(np.float64), f"logc {shape} gradient with respect to the logarithms")
    # and it is the same function as exponentiating by hand
    y2 = linrec_amd.linrec(x.to(DEV), torch.exp(logc.to(DEV)), reverse)
    assert torch.equal(y, y2)


def test_a_wait_that_runs_out_never_shows_in_the_results():
    """With a poll limit of one, every kernel family whose workgroups wait for each other is run through
    the public operator, forward and backward: the results must be as right as ever (a wave whose wait
    runs out computes what it needs from the row's own data), never NaN and never silently wrong."""
    lib = nat.lib()
    cases = [((16, 131072), False), ((512, 16384), False), ((3, 200000), True), ((8, 100004), False), ((40, 65536), True)]
    old = lib.linrec_set_spin_limit(1)
    try:
        for shape, reverse in cases:
            g = torch.Generator().manual_seed(shape[0])
            x = torch.randn(shape, generator=g)
            c = torch.rand(shape, generator=g)
            dy = torch.randn(shape, generator=g)
            fams = (nat.plan(x.to(DEV), reverse, False)["family"], nat.plan(x.to(DEV), reverse, True)["family"])
            print("poll limit 1:", shape, reverse, "families", fams, flush=True)
            xd, cd = x.to(DEV).requires_grad_(), c.to(DEV).requires_grad_()
            y = linrec_amd.linrec(xd, cd, reverse)
            dx, dc = torch.autograd.grad(y, (xd, cd), dy.to(DEV))
            torch.cuda.synchronize()
            y_t = oracle.fwd(x.numpy(), c.numpy(), reverse, dtype=np.float64)
            dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y_t, reverse, dtype=np.float64)
            check_close(y, y_t, f"{shape} outputs")
            check_close(dx, dx_t, f"{shape} d_inputs")
            check_close(dc, dc_t, f"{shape} d_coeffs")
    finally:
        lib.linrec_set_spin_limit(old)
    torch.cuda.synchronize()
    print("waits that ran out:", nat.gave_up_count(), flush=True)
    # the other tests take a count of zero as the sign that nobody ever had to fall back: start over
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0
    assert nat.gave_up_count() == 0
