"""fp16 and bf16 storage (fp32 arithmetic) against the float64 recurrence on the same 16-bit inputs.

Bar: every result element within 0.51 units in the last place of the 16-bit format around the float64
truth (plus 1e-5 of the row-set maximum for the fp32 accumulation), i.e. the kernels behave like an
exact computation followed by one rounding; normwise that is 2^-9 (bf16) and 2^-12 (fp16)."""
import numpy as np
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu

MANT = {torch.float16: 10, torch.bfloat16: 7}
MIN_EXP = {torch.float16: -14, torch.bfloat16: -126}


def _ulp(truth, dtype):
    a = np.abs(truth)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** MIN_EXP[dtype])))
    return 2.0 ** (e - MANT[dtype])


def _check(got, truth, dtype, what):
    g = got.detach().float().cpu().numpy().astype(np.float64)
    assert np.isfinite(g).all(), what
    err = np.abs(g - truth)
    bound = 0.51 * _ulp(truth, dtype) + 1e-5 * np.abs(truth).max()
    bad = err > bound
    assert not bad.any(), f"{what}: {bad.sum()} elements off, worst {np.max(err / bound):.2f} x bound"


def _inputs(shape, dtype, seed, transposed=False, coeffs="uniform"):
    g = torch.Generator().manual_seed(seed)
    base = tuple(reversed(shape)) if transposed else shape
    x = torch.randn(base, generator=g).to(dtype)
    c = torch.rand(base, generator=g)
    if coeffs == "near1":
        c = 0.9 + 0.1 * c
    c = c.to(dtype)
    dy = torch.randn(base, generator=g).to(dtype)
    return tuple(t.t() if transposed else t for t in (x, c, dy))


def _nan_like(t):
    return torch.empty_strided(t.size(), t.stride(), dtype=t.dtype, device=t.device).fill_(float("nan"))


def _run(nat, x, c, dy, reverse, tuning, label, backward_too=True):
    dev = torch.device("cuda:0")
    xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
    assert xd.stride() == x.stride()
    f64 = lambda t: t.float().numpy().astype(np.float64)
    y_t = oracle.fwd(f64(x), f64(c), reverse)
    y = nat.fwd(xd, cd, reverse, tuning, out=_nan_like(xd))
    torch.cuda.synchronize()
    _check(y, y_t, x.dtype, f"{label} outputs")
    if not backward_too:
        assert nat.gave_up_count() == 0
        return
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y.cpu()), reverse)  # from the 16-bit outputs that were saved
    dx, dc = nat.bwd(dyd, cd, y, reverse, tuning, out=(_nan_like(xd), _nan_like(xd)))
    torch.cuda.synchronize()
    _check(dx, dx_t, x.dtype, f"{label} d_inputs")
    _check(dc, dc_t, x.dtype, f"{label} d_coeffs")
    assert nat.gave_up_count() == 0


@pytest.fixture(scope="module")
def nat():
    import linrec_amd
    from linrec_amd import _native
    return _native


def _tunings(nat, L):
    out = [None]
    for waves, slots, carry in [(1, 1, 0), (2, 1, 0), (4, 1, 0), (4, 2, 0), (8, 2, 0), (16, 2, 0), (4, 2, 1), (8, 4, 1)]:
        tile = waves * slots * 512
        if carry == 0 and L + 7 > tile:
            continue
        if carry == 1 and (L + 7) // tile > 200:
            continue
        out.append(nat.Tuning(nat.FAMILY_TILE, waves, slots, carry))
    out.append(nat.Tuning(nat.FAMILY_STREAM, 8, 2))
    out.append(nat.Tuning(nat.FAMILY_TEAM, 8, 2, -1, 3))
    if L % 8192 == 0:  # rows of whole tiles: teams that go on from row to row
        out.append(nat.Tuning(nat.FAMILY_SWEEP, 8, 2))
        out.append(nat.Tuning(nat.FAMILY_SWEEP, 8, 2, 2, 1))
    if L % 8192 == 0:  # the same with tiles stored two steps late: 16 waves of one slot, both passes
        k = L // 8192
        out.append(nat.Tuning(nat.FAMILY_DRIFT, 16, 1))                     # team = tiles of a row
        out.append(nat.Tuning(nat.FAMILY_DRIFT, 16, 1, 3, 0))               # three teams share the rows
        out.append(nat.Tuning(nat.FAMILY_DRIFT, 16, 1, 1, 1))               # one walker takes whole rows
        if k % 2 == 0:
            out.append(nat.Tuning(nat.FAMILY_DRIFT, 16, 1, 2, k // 2))      # two tiles of a row per walker
    if L % 16384 == 0:  # forward only: tiles of 16384 elements, which wait in LDS as packed inputs and are scanned twice
        k = L // 16384
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 16, 2), False))
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 16, 2, 3, 0), False))
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 16, 2, 1, 1), False))
        if k % 2 == 0:
            out.append((nat.Tuning(nat.FAMILY_DRIFT, 16, 2, 2, k // 2), False))
    if L % 4096 == 0:  # tiles of 4096 elements in 8 waves (compiled for the forward only)
        k = L // 4096
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 8, 1), False))            # team = tiles of a row
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 8, 1, 3, 0), False))      # three teams share the rows
        out.append((nat.Tuning(nat.FAMILY_DRIFT, 8, 1, 1, 1), False))      # one walker takes whole rows
        if k % 2 == 0:
            out.append((nat.Tuning(nat.FAMILY_DRIFT, 8, 1, 2, k // 2), False))  # two tiles of a row per walker
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("L", [1, 7, 8, 9, 511, 512, 513, 1000, 4096, 4099, 8192, 16384, 16385, 40000, 65536, 131073])
def test_seqlen_sweep(nat, L, reverse, dtype):
    numseq = 5 if L > 8192 else 33
    x, c, dy = _inputs((numseq, L), dtype, seed=L)
    for tuning in _tunings(nat, L):
        backward_too = True
        if isinstance(tuning, tuple):
            tuning, backward_too = tuning
        label = f"{dtype} L={L} rev={reverse} tune={None if tuning is None else (tuning.family, tuning.waves, tuning.slots, tuning.carry, tuning.tasks)}"
        print(label, flush=True)
        _run(nat, x, c, dy, reverse, tuning, label, backward_too)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_layouts(nat, reverse, dtype):
    dev = torch.device("cuda:0")
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    # padded rows with an odd width: rows start at varying phases of a 16-byte slot; padding must survive
    L, width, n = 3001, 3005, 7
    xw, cw, dyw = _inputs((n, width), dtype, seed=1)
    xd, cd = xw.to(dev)[:, :L], cw.to(dev)[:, :L]
    ybuf = torch.full((n, width), float("nan"), dtype=dtype, device=dev)
    y = nat.fwd(xd, cd, reverse, out=ybuf[:, :L])
    torch.cuda.synchronize()
    _check(y, oracle.fwd(f64(xw[:, :L]), f64(cw[:, :L]), reverse), dtype, "padded rows")
    assert torch.isnan(ybuf[:, L:]).all()
    # all bases shifted by k elements; then only one of them (element-sized accesses)
    for off in (1, 3, 7):
        x, c, dy = _inputs((4, 2000), dtype, seed=off)

        def shifted(t, o):
            buf = torch.full((t.numel() + 16,), float("nan"), dtype=dtype, device=dev)
            v = buf[o:o + t.numel()].view(t.shape)
            v.copy_(t)
            return v
        y = nat.fwd(shifted(x, off), shifted(c, off), reverse, out=shifted(torch.full(x.shape, float("nan")), off))
        torch.cuda.synchronize()
        _check(y, oracle.fwd(f64(x), f64(c), reverse), dtype, f"bases shifted by {off}")
        lib = nat.lib()
        xs, cs, ys = shifted(x, off), c.to(dev), torch.full(x.shape, float("nan"), dtype=dtype, device=dev)
        ws = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
        rc = lib.linrec_fwd(nat.DTYPES[dtype], xs.data_ptr(), cs.data_ptr(), ys.data_ptr(), 4, 2000, 2000, 1,
                            int(reverse), ws.data_ptr(), ws.numel(), None, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        _check(ys, oracle.fwd(f64(x), f64(c), reverse), dtype, f"one base shifted by {off}")
    # transposed views: eight rows per lane, and the element-wise kernel when the row count is odd
    # and the segmented launches for scan axes of 256 elements and more
    for shape in [(2048, 100), (1001, 33), (520, 700), (77, 3000)]:
        x, c, dy = _inputs(shape, dtype, seed=shape[0], transposed=True)
        family = nat.FAMILY_COLUMN if shape[0] % 8 == 0 else nat.FAMILY_NAIVE
        assert nat.plan(x.to("cuda:0"), reverse)["family"] == (nat.FAMILY_SEGMENT if shape[1] >= 256 else nat.FAMILY_COLUMN)
        for tuning in (None, nat.Tuning(family, 0, 0, -1), nat.Tuning(nat.FAMILY_SEGMENT, 0, 8, -1, 5),
                       nat.Tuning(nat.FAMILY_SEGMENT, 1, 8, -1, 3)):
            _run(nat, x, c, dy, reverse, tuning, f"transposed {shape} tuning={None if tuning is None else (tuning.family, tuning.waves, tuning.tasks)}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("name,shape,coeffs,reverse,transposed", [
    ("C2", (512, 65536), "uniform", False, False), ("C3", (16384, 2048), "uniform", True, False),
    ("C4", (16, 1048576), "near1", False, False), ("C5", (262144, 256), "uniform", False, True)])
def test_config_shapes_through_autograd(name, shape, coeffs, reverse, transposed, dtype):
    import linrec_amd
    x, c, dy = _inputs(shape, dtype, seed=0, transposed=transposed, coeffs=coeffs)
    dev = torch.device("cuda:0")
    xd, cd = x.to(dev).requires_grad_(), c.to(dev).requires_grad_()
    y = linrec_amd.linrec(xd, cd, reverse)
    assert y.dtype == dtype and y.stride() == x.stride()
    gx, gc = torch.autograd.grad(y, (xd, cd), dy.to(dev))
    torch.cuda.synchronize()
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    y_t = oracle.fwd(f64(x), f64(c), reverse)
    _check(y, y_t, dtype, f"{name} outputs")
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y), reverse)
    _check(gx, dx_t, dtype, f"{name} d_inputs")
    _check(gc, dc_t, dtype, f"{name} d_coeffs")
    from linrec_amd import _native
    assert _native.gave_up_count() == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_a_few_very_long_rows(nat, reverse, dtype):
    """One or two very long rows run in teams that fill the launch (four and two collecting waves), both passes where
    the rows are whole tiles of 8192 elements; where they are whole tiles of 4096 only, the forward in those and the
    backward in tiles of 8192 of which the last is half full; three to
    five rows with less than four tiles for every compute unit, or ragged ones, run forward in teams of up to 64 and
    backward in look-back tiles.  Also with a poll limit of one: every wait of the team members for each other's maps
    may run out, and the results are the same."""
    dev = torch.device("cuda:0")
    D, TM, TL = nat.FAMILY_DRIFT, nat.FAMILY_TEAM, nat.FAMILY_TILE
    for shape, fwd, bwd in [((1, 8192 * 512), (D, 16, 1, 256), (D, 16, 1, 256)), ((2, 8192 * 300), (D, 16, 1, 100), (D, 16, 1, 100)),
                            ((2, 4096 * 605), (D, 8, 1, 121), (D, 8, 2, 101)),
                            ((4, 16384 * 512), (D, 16, 2, 256), (D, 16, 1, 256)), ((5, 16384 * 231), (D, 16, 2, 231), (D, 16, 1, 231)),
                            ((3, 4096 * 300), (TM, 8, 4, 64), (TL, 8, 4, 1)), ((5, 4096 * 150 + 24), (TM, 8, 4, 38), (TL, 8, 4, 1))]:
        x, c, dy = _inputs(shape, dtype, seed=shape[0], coeffs="near1")
        plan = nat.plan(x.to(dev), reverse)
        assert (plan["family"], plan["waves"], plan["slots"], plan["tasks"]) == fwd, plan
        plan = nat.plan(x.to(dev), reverse, True)
        assert (plan["family"], plan["waves"], plan["slots"], plan["tasks"]) == bwd, plan
        _run(nat, x, c, dy, reverse, None, f"{dtype} {shape} rev={reverse}")
    # (the last: forward in tiles of 16384 elements, backward in tiles of 8192)
    for shape in ((1, 4096 * 1024), (8, 16384 * 128)):
        _poll_limit_one(nat, shape, dtype, reverse)


def _poll_limit_one(nat, shape, dtype, reverse):
    dev = torch.device("cuda:0")
    x, c, dy = _inputs(shape, dtype, seed=7)
    y_kept = nat.fwd(x.to(dev), c.to(dev), reverse)
    old = nat.lib().linrec_set_spin_limit(1)
    try:
        y = nat.fwd(x.to(dev), c.to(dev), reverse)
        dx, dc = nat.bwd(dy.to(dev), c.to(dev), y_kept, reverse)
        torch.cuda.synchronize()
    finally:
        nat.lib().linrec_set_spin_limit(old)
    print("16-bit drift, poll limit 1: waits that ran out:", nat.gave_up_count(), flush=True)
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0  # (the other tests take a count of zero as the sign that nobody had to fall back)
    f64 = lambda t: t.float().numpy().astype(np.float64)
    _check(y, oracle.fwd(f64(x), f64(c), reverse), dtype, "with a poll limit of one")
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y_kept.cpu()), reverse)
    _check(dx, dx_t, dtype, "d_inputs with a poll limit of one")
    _check(dc, dc_t, dtype, "d_coeffs with a poll limit of one")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_column_drift_kernels_two_rows_per_lane(nat, reverse, dtype):
    """Scan axis strided, 16-bit storage: blocks of 128 rows (two to a lane, kept packed from a step's loads to its
    stores) in teams along the scan axis.  Every compiled geometry is forced with team sizes from 1 to 8 on row lengths
    around whole steps, on fewer steps than team members allow and on row counts that leave lanes without rows; then
    the planner's own choice, a batch of time-major matrices, and a poll limit of one."""
    D = nat.FAMILY_COLDRIFT
    dev = torch.device("cuda:0")
    f64 = lambda t: t.float().numpy().astype(np.float64)
    for n, L in [(128, 256), (2, 129), (130, 257), (66, 1000), (1000, 1290), (190, 2048), (4100, 700)]:
        x, c, dy = _inputs((n, L), dtype, n + L, transposed=True)
        y_kept = None
        for waves, run, passes in [(16, 8, "f"), (8, 16, "fb"), (16, 4, "b")]:
            steps, blocks = -(-L // (waves * run)), -(-(n // 2) // 64)
            for team in sorted({1, 2, 3, min(waves, steps), min(8, steps)}):
                if team > steps or blocks * team > 256:
                    continue
                tuning = nat.Tuning(D, waves, run, 2, team)
                label = f"{dtype} rev={reverse} {n} x {L} waves={waves} run={run} team={team}"
                plan = nat.plan(x.to(dev), reverse, passes == "b", tuning)
                assert (plan["family"], plan["vec"], plan["block"], plan["tasks"], plan["grid"], plan["tiles_per_row"]) == (
                    D, 2, 64 * waves, team, blocks * team, steps), plan
                if passes != "b":
                    _run(nat, x, c, dy, reverse, tuning, label, backward_too=passes == "fb")
                else:
                    if y_kept is None:
                        y_kept = nat.fwd(x.to(dev), c.to(dev), reverse)
                    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y_kept.cpu()), reverse)
                    dx, dc = nat.bwd(dy.to(dev), c.to(dev), y_kept, reverse, tuning, out=(_nan_like(y_kept), _nan_like(y_kept)))
                    torch.cuda.synchronize()
                    _check(dx, dx_t, dtype, label + " d_inputs")
                    _check(dc, dc_t, dtype, label + " d_coeffs")
                    assert nat.gave_up_count() == 0
    # the planner's own choice, both passes: teams of 8 on 4096 rows
    x, c, dy = _inputs((4096, 2100), dtype, 5, transposed=True, coeffs="near1")
    for is_bwd in (False, True):
        plan = nat.plan(x.to(dev), reverse, is_bwd)
        assert (plan["family"], plan["vec"], plan["tasks"], plan["grid"]) == (D, 2, 8, 256), plan
    _run(nat, x, c, dy, reverse, None, f"{dtype} transposed 4096 x 2100")
    # a batch of time-major matrices: 3 x (2100 timesteps x 2688 channels) scanned over time
    g = torch.Generator().manual_seed(11)
    xb, cb, dyb = (f((3, 2100, 2688), generator=g).to(dtype) for f in (torch.randn, torch.rand, torch.randn))
    xv, cv, dyv = (t.to(dev).transpose(1, 2) for t in (xb, cb, dyb))
    plan = nat.plan(xv, reverse, False)
    assert plan["family"] == D and plan["grid"] == 63 * plan["tasks"], plan
    y = nat.fwd(xv, cv, reverse)
    dx, dc = nat.bwd(dyv, cv, y, reverse)
    torch.cuda.synchronize()
    xt, ct, dyt = (t.transpose(1, 2) for t in (xb, cb, dyb))
    _check(y, oracle.fwd(f64(xt), f64(ct), reverse), dtype, "batched outputs")
    dx_t, dc_t = oracle.bwd(f64(dyt), f64(ct), f64(y.cpu()), reverse)
    _check(dx, dx_t, dtype, "batched d_inputs")
    _check(dc, dc_t, dtype, "batched d_coeffs")
    # a poll limit of one: waits run out, the value entering a step comes from the rows' own data instead
    x, c, dy = _inputs((700, 6000), dtype, 3, transposed=True)
    y_kept = nat.fwd(x.to(dev), c.to(dev), reverse)
    old = nat.lib().linrec_set_spin_limit(1)
    try:
        y = nat.fwd(x.to(dev), c.to(dev), reverse, nat.Tuning(D, 16, 8, 2, 8))
        dx, dc = nat.bwd(dy.to(dev), c.to(dev), y_kept, reverse, nat.Tuning(D, 8, 16, 2, 8))
        torch.cuda.synchronize()
    finally:
        nat.lib().linrec_set_spin_limit(old)
    print("16-bit column drift, poll limit 1: waits that ran out:", nat.gave_up_count(), flush=True)
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0  # (the other tests take a count of zero as the sign that nobody had to fall back)
    _check(y, oracle.fwd(f64(x), f64(c), reverse), dtype, "poll limit 1 outputs")
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y_kept.cpu()), reverse)
    _check(dx, dx_t, dtype, "poll limit 1 d_inputs")
    _check(dc, dc_t, dtype, "poll limit 1 d_coeffs")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_rows_with_a_partial_last_tile_run_in_drift_teams(nat, reverse, dtype):
    """16-bit rows of whole slots of eight elements whose length is not a whole number of tiles: the drift kernels'
    last tile of a row is a partial one (every slot lies in the row or beyond its end), the teams need not divide the
    tiles of a row.  The forward in tiles of 16384 elements, the backward in tiles of 8192 in 8 waves of two slots.
    Forced team sizes, the planner's own choice, and a poll limit of one."""
    D = nat.FAMILY_DRIFT
    dev = torch.device("cuda:0")
    names = nat.kernel_table()
    f64 = lambda t: t.float().numpy().astype(np.float64)

    def backward(x, c, dy, tuning, label):
        y = nat.fwd(x.to(dev), c.to(dev), reverse)
        dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y.cpu()), reverse)
        dx, dc = nat.bwd(dy.to(dev), c.to(dev), y, reverse, tuning, out=(_nan_like(y), _nan_like(y)))
        torch.cuda.synchronize()
        _check(dx, dx_t, dtype, label + " d_inputs")
        _check(dc, dc_t, dtype, label + " d_coeffs")

    for shape, teams in [((3, 16384 * 2 + 8), (0, 2, 3)), ((5, 16384 * 3 + 8192), (0, 3)), ((7, 16384 * 5 - 8), (0, 4)),
                         ((33, 16384 * 4 + 1000), (0, 5)), ((2, 16384 * 13 + 16376), (0, 9)), ((1, 16384 * 40 + 24), (0, 7))]:
        x, c, dy = _inputs(shape, dtype, shape[0] + shape[1], coeffs="near1")
        for team in teams:
            tf = nat.Tuning(D, 16, 2, -1, team)
            kb = -(-shape[1] // 8192)
            team_b = min(2 * team, kb)
            if team_b and shape[1] % 8192 == 0 and kb % team_b:
                team_b = kb  # (rows of whole such tiles take the kernel for them, whose teams divide the tiles of a row)
            tb = nat.Tuning(D, 8, 2, -1, team_b) if shape[1] % 8192 else nat.Tuning(D, 16, 1, -1, team_b)
            pf, pb = nat.plan(x.to(dev), reverse, False, tf), nat.plan(x.to(dev), reverse, True, tb)
            assert "drift_ragged_w16_s2" in names[pf["kernel_id"]] and pf["tiles_per_row"] == -(-shape[1] // 16384), pf
            assert ("drift_ragged_w8_s2" in names[pb["kernel_id"]]) == (shape[1] % 8192 != 0) and pb["tiles_per_row"] == kb, pb
            label = f"{dtype} {shape} rev={reverse} forward team {pf['tasks']}, backward team {pb['tasks']}"
            _run(nat, x, c, dy, reverse, tf, label, backward_too=False)
            backward(x, c, dy, tb, label)
            assert nat.gave_up_count() == 0
    # the planner's own choice
    for shape in [(335, 100000), (16, 1000000), (100, 250000)]:
        x, c, dy = _inputs(shape, dtype, shape[0], coeffs="near1")
        for is_bwd, geometry in ((False, (16, 2)), (True, (8, 2))):
            plan = nat.plan(x.to(dev), reverse, is_bwd)
            assert plan["family"] == D and "ragged" in names[plan["kernel_id"]] and (plan["waves"], plan["slots"]) == geometry, plan
            assert plan["grid"] <= 256 and plan["grid"] % plan["tasks"] == 0, plan
        _run(nat, x, c, dy, reverse, None, f"{dtype} {shape} rev={reverse}, default plan")
    # a poll limit of one: waits run out, the value entering a tile comes from the row's own data instead
    x, c, dy = _inputs((6, 16384 * 50 + 5000), dtype, 4, coeffs="near1")
    y_kept = nat.fwd(x.to(dev), c.to(dev), reverse)
    old = nat.lib().linrec_set_spin_limit(1)
    try:
        y = nat.fwd(x.to(dev), c.to(dev), reverse, nat.Tuning(D, 16, 2, -1, 17))
        dx, dc = nat.bwd(dy.to(dev), c.to(dev), y_kept, reverse, nat.Tuning(D, 8, 2, -1, 33))
        torch.cuda.synchronize()
    finally:
        nat.lib().linrec_set_spin_limit(old)
    print("16-bit drift with partial tiles, poll limit 1: waits that ran out:", nat.gave_up_count(), flush=True)
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0  # (the other tests take a count of zero as the sign that nobody had to fall back)
    _check(y, oracle.fwd(f64(x), f64(c), reverse), dtype, "poll limit 1 outputs")
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y_kept.cpu()), reverse)
    _check(dx, dx_t, dtype, "poll limit 1 d_inputs")
    _check(dc, dc_t, dtype, "poll limit 1 d_coeffs")
