"""Seeded random layouts through the public operator, forward and autograd backward, against the
float64 recurrence: rank 1-3, scan lengths from 1 to 70 000, dense / row-padded / offset /
transposed / broadcast-free strided views, both directions, the three storage types, `dim` other
than the last.  The cases are fixed by the seeds, so a failure names its case."""
import numpy as np
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
# one rounding to the storage type (half a unit in the last place of the largest element) plus fp32 noise
TOL = {torch.float32: 1e-5, torch.bfloat16: 1.05 * 2.0 ** -8, torch.float16: 1.05 * 2.0 ** -11}


def _random_case(rng):
    """A dict describing one case; every choice comes from `rng`."""
    rank = int(rng.integers(1, 4))
    if rng.integers(0, 4) == 0:
        # rows of a whole number of tiles, many of them: the kernels whose teams go from row to row
        L = 4096 * int(rng.integers(1, 18))
        rank = max(rank, 2)
        lead = [int(rng.integers(1, 25)) for _ in range(rank - 2)] + [int(rng.integers(4, 320))]
        cap = 6000000
    else:
        L = int(np.exp(rng.uniform(0, np.log(70000))))
        budget = 400000 // L + 1
        lead = [int(rng.integers(1, max(2, min(40, budget)))) for _ in range(rank - 1)]
        cap = 600000
    while int(np.prod(lead or [1])) * L > cap and lead:
        lead[int(np.argmax(lead))] = max(1, max(lead) // 2)
    layout = ["dense", "padded", "offset", "transposed", "dim"][int(rng.integers(0, 5))]
    if rank == 1 and layout in ("transposed", "dim", "padded"):
        layout = "offset"
    return dict(shape=tuple(lead) + (L,), layout=layout, reverse=bool(rng.integers(0, 2)),
                dtype=DTYPES[int(rng.integers(0, 3))], pad=int(rng.integers(1, 9)), offset=int(rng.integers(1, 9)),
                coeffs=["uniform", "signed", "near1"][int(rng.integers(0, 3))],
                # what autograd hands back for y.sum(): one value expanded with zero strides
                expanded_grad=bool(rng.integers(0, 4) == 0))


def _materialise(case, gen, dev):
    """x, c, dy on the device in the case's layout, and `dim`."""
    shape, dtype = case["shape"], case["dtype"]

    def values(kind):
        if kind == "normal":
            return torch.randn(shape, generator=gen)
        u = torch.rand(shape, generator=gen)
        return {"uniform": u, "signed": 2 * u - 1, "near1": 0.9 + 0.1 * u}[case["coeffs"]]

    def place(v):
        v = v.to(dtype)
        lay = case["layout"]
        if lay == "dense":
            return v.to(dev), -1
        if lay == "padded":  # rows of a wider tensor
            wide = torch.full(shape[:-1] + (shape[-1] + case["pad"],), float("nan"), dtype=dtype, device=dev)
            view = wide[..., :shape[-1]]
            view.copy_(v)
            return view, -1
        if lay == "offset":  # a view that starts a few elements into its buffer
            n = v.numel()
            buf = torch.full((n + 16,), float("nan"), dtype=dtype, device=dev)
            view = buf[case["offset"]:case["offset"] + n].view(shape)
            view.copy_(v)
            return view, -1
        if lay == "transposed":  # the scan axis is the strided one
            base = torch.empty(shape[:-2] + (shape[-1], shape[-2]), dtype=dtype, device=dev)
            view = base.transpose(-1, -2)
            view.copy_(v)
            return view, -1
        # "dim": the caller scans over dim -2 of a dense tensor
        t = v.transpose(-1, -2).contiguous().to(dev)
        return t, -2

    (x, dim), (c, _), (dy, _) = place(values("normal")), place(values("coeffs")), place(values("normal"))
    return x, c, dy, dim


@pytest.mark.parametrize("seed", range(300))
def test_random_layout(seed):
    import linrec_amd
    from linrec_amd import _native as nat
    rng = np.random.default_rng(1000 + seed)
    case = _random_case(rng)
    print(seed, case, flush=True)
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(seed)
    x, c, dy, dim = _materialise(case, gen, dev)
    if case["expanded_grad"]:
        dy = torch.full((), 0.5, dtype=case["dtype"], device=dev).expand(x.shape)
    xg, cg = x.detach().requires_grad_(), c.detach().requires_grad_()
    y = linrec_amd.linrec(xg, cg, case["reverse"], dim=dim)
    gx, gc = torch.autograd.grad(y, (xg, cg), dy)
    torch.cuda.synchronize()
    assert y.shape == x.shape and gx.shape == x.shape and gc.shape == x.shape
    assert nat.gave_up_count() == 0

    def scan_last(t):  # float64 numpy with the scan axis last
        t = t.detach().float().cpu()
        return (t.transpose(-1, -2) if dim == -2 else t).contiguous().numpy().astype(np.float64)

    xn, cn, dyn, yn = scan_last(x), scan_last(c), scan_last(dy), scan_last(y)
    y_t = oracle.fwd(xn, cn, case["reverse"])
    dx_t, dc_t = oracle.bwd(dyn, cn, yn, case["reverse"])  # from the outputs the forward stored
    tol = TOL[case["dtype"]]
    for got, want, what in ((yn, y_t, "outputs"), (scan_last(gx), dx_t, "d_inputs"), (scan_last(gc), dc_t, "d_coeffs")):
        assert np.isfinite(got).all(), (what, case)
        rep = oracle.error_report(got, want)
        assert rep["normwise"] <= tol, (what, case, rep)


@pytest.mark.parametrize("seed", range(4))
def test_random_long_and_short_rows_through_the_default_plan(seed):
    """Dense row-major tensors at the sizes where the planner's long-row kernels take over (up to 4e7 elements), 40
    seeded cases each: rows of whole tiles, rows of whole slots that end in a partial tile (few and many of them), one to
    five very long rows, arbitrary lengths, and short rows down to two elements.  Both passes through the C ABI with the
    default plan, result buffers poisoned, against the float64 recurrence; 16-bit results to half a unit in the last
    place."""
    from linrec_amd import _native as nat
    rng = np.random.default_rng(7000 + seed)
    dev = torch.device("cuda:0")
    names = nat.kernel_table()
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    for case in range(40):
        dtype = DTYPES[int(rng.integers(3))]
        fv = 4 if dtype == torch.float32 else 8
        kind = int(rng.integers(6))
        if kind == 0:    # short dense rows
            L, n = int(rng.integers(2, 70)), int(rng.integers(2, 5000))
        elif kind == 1:  # whole slots, a partial last tile
            tile = 8192 if dtype == torch.float32 else 16384
            L = int(rng.integers(2, 40)) * (tile // 2) + int(rng.integers(1, tile // fv)) * fv
            n = int(rng.choice([1, 2, 3, 5, 16, 33, 100, 257, 300, 600]))
        elif kind == 2:  # whole tiles
            L, n = int(rng.integers(1, 30)) * 8192, int(rng.choice([1, 2, 4, 16, 64, 130, 256, 300, 512]))
        elif kind == 3:  # arbitrary lengths
            L, n = int(rng.integers(100, 200000)), int(rng.integers(1, 400))
        elif kind == 4:  # a few thousand elements
            L, n = int(rng.integers(200, 9000)), int(rng.integers(1, 3000))
        else:            # a few very long rows
            L, n = int(rng.integers(200000, 3000000)), int(rng.integers(1, 6))
        if n * L > 40_000_000:
            n = max(1, 40_000_000 // L)
        reverse = bool(rng.integers(2))
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        x = torch.randn(n, L, generator=g).to(dtype)
        c = (torch.rand(n, L, generator=g) * (0.2 if L > 4000 else 1.8) + (0.8 if L > 4000 else -0.9)).to(dtype)
        dy = torch.randn(n, L, generator=g).to(dtype)
        xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
        kernels = [names[nat.plan(xd, reverse, b)["kernel_id"]] for b in (False, True)]
        what = (seed, case, str(dtype), (n, L), reverse, kernels)
        print(*what, flush=True)
        y = nat.fwd(xd, cd, reverse, None, out=torch.full_like(xd, float("nan")))
        dx, dc = nat.bwd(dyd, cd, y, reverse, None, out=(torch.full_like(xd, float("nan")), torch.full_like(xd, float("nan"))))
        torch.cuda.synchronize()
        y_t = oracle.fwd(f64(x), f64(c), reverse)
        dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y), reverse)  # from the outputs the forward stored
        for got, want, name in ((y, y_t, "outputs"), (dx, dx_t, "d_inputs"), (dc, dc_t, "d_coeffs")):
            got = f64(got)
            assert np.isfinite(got).all(), (name, what)
            if dtype == torch.float32:
                assert np.abs(got - want).max() <= 2e-5 * max(np.abs(want).max(), 1e-30), (name, what)
            else:
                unit = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 1e-30))) - (10 if dtype == torch.float16 else 7))
                assert (np.abs(got - want) <= 0.51 * unit + 1e-5 * np.abs(want).max()).all(), (name, what)
    assert nat.gave_up_count() == 0


def _view_of(t, ops):
    """`t` after a sequence of view-making operations (op, dim, argument); operations that do not apply
    to the tensor at hand are skipped."""
    for op, d, a in ops:
        if t.dim() == 0:
            break
        d = d % t.dim()
        if op == 0 and t.dim() > 1:
            t = t.transpose(d, a % t.dim())
        elif op == 1 and t.size(d) > 1:
            t = t.narrow(d, a % 2, t.size(d) - 1)
        elif op == 2 and t.size(d) > 2:
            t = t[(slice(None),) * d + (slice(None, None, 2),)]
        elif op == 3 and t.size(d) == 1:  # broadcast: a zero stride
            t = t.expand(*[(2 + a % 3) if i == d else -1 for i in range(t.dim())])
        elif op == 4 and t.dim() > 2:
            t = t.permute(*np.random.default_rng(a).permutation(t.dim()).tolist())
    return t


@pytest.mark.parametrize("chunk", range(8))
def test_random_views(chunk):
    """Views made by random transposes, slices, steps, broadcasts and permutations, scanned over a random
    dim, through the operator and autograd: whatever the layout, the values are those of the recurrence
    on the same numbers laid out densely."""
    import linrec_amd
    from linrec_amd import _native as nat
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5000 + chunk)
    for case in range(150):
        rank = int(rng.integers(1, 4))
        shape = [int(rng.integers(1, 9)) for _ in range(rank)]
        shape[int(rng.integers(0, rank))] = int(rng.integers(1, 3000 if rng.integers(0, 3) == 0 else 300))
        if rng.integers(0, 4) == 0:
            shape[int(rng.integers(0, rank))] = 1
        ops = [(int(rng.integers(0, 5)), int(rng.integers(0, 4)), int(rng.integers(0, 1000))) for _ in range(int(rng.integers(0, 4)))]
        dtype = DTYPES[int(rng.integers(0, 3))]
        g = torch.Generator().manual_seed(chunk * 1000 + case)
        x = _view_of(torch.randn(shape, generator=g).to(dtype).to(dev), ops)
        c = _view_of((torch.rand(shape, generator=g) * 1.6 - 0.8).to(dtype).to(dev), ops)
        if rng.integers(0, 3) == 0:
            c = c.contiguous()  # coefficients that lie differently in memory than the inputs
        if x.numel() == 0 or x.dim() == 0:
            continue
        dim = int(rng.integers(0, x.dim())) if rng.integers(0, 3) == 0 else -1
        reverse = bool(rng.integers(0, 2))
        dy = torch.randn(x.shape, generator=g).to(dtype).to(dev)
        what = (chunk, case, shape, ops, dtype, dim, reverse, tuple(x.shape), x.stride(), c.stride())
        xg, cg = x.detach().requires_grad_(), c.detach().requires_grad_()
        y = linrec_amd.linrec(xg, cg, reverse, dim=dim)
        gx, gc = torch.autograd.grad(y, (xg, cg), dy)
        torch.cuda.synchronize()
        scan_last = lambda t: t.detach().float().cpu().movedim(dim, -1).contiguous().numpy().astype(np.float64)
        y_t = oracle.fwd(scan_last(x), scan_last(c), reverse)
        dx_t, dc_t = oracle.bwd(scan_last(dy), scan_last(c), scan_last(y), reverse)
        for got, want, name in ((scan_last(y), y_t, "outputs"), (scan_last(gx), dx_t, "d_inputs"), (scan_last(gc), dc_t, "d_coeffs")):
            assert np.isfinite(got).all(), (name, what)
            rep = oracle.error_report(got, want)
            assert rep["normwise"] <= TOL[dtype], (name, what, rep)
    assert nat.gave_up_count() == 0
