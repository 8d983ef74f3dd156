"""Parity of the HIP kernels with the CPU checker, through the C ABI (ctypes) and through the
registered operators.  Bar: normwise relative error <= 1e-5 against the float64 sequential
recurrence on identical seeded fp32 inputs, for outputs, d_inputs and d_coeffs.

Every result buffer is pre-filled with NaN, so an element the kernel failed to write, or padding
it wrote by mistake, is caught."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle
from tests.util import TOL_NORMWISE, check_close, make_inputs, truth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def nat():
    import linrec_amd
    from linrec_amd import _native
    return _native


def _nan_like(t):
    out = torch.empty_strided(t.size(), t.stride(), dtype=t.dtype, device=t.device)
    out.fill_(float("nan"))
    return out


def _run_both(nat, x, c, dy, reverse, tuning, label):
    """fwd + bwd on the GPU with poisoned result buffers; compares with the float64 truth."""
    dev = torch.device("cuda:0")
    xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
    assert xd.stride() == x.stride()
    y_t, dx_t, dc_t = truth(x, c, dy, reverse)
    y = nat.fwd(xd, cd, reverse, tuning, out=_nan_like(xd))
    torch.cuda.synchronize()
    check_close(y, y_t, f"{label} outputs")
    # backward from the float32 outputs the forward produced (what autograd saves)
    dx, dc = nat.bwd(dyd, cd, y, reverse, tuning, out=(_nan_like(xd), _nan_like(xd)))
    torch.cuda.synchronize()
    check_close(dx, dx_t, f"{label} d_inputs")
    check_close(dc, dc_t, f"{label} d_coeffs")
    assert nat.gave_up_count() == 0


def _run_forward(nat, x, c, reverse, tuning, label, check_gave_up=True):
    """The forward pass alone (geometries that are compiled for the forward only); returns the device's outputs."""
    y_t = truth(x, c, torch.zeros_like(x), reverse)[0]
    dev = torch.device("cuda:0")
    xd, cd = x.to(dev), c.to(dev)
    y = nat.fwd(xd, cd, reverse, tuning, out=_nan_like(xd))
    torch.cuda.synchronize()
    check_close(y, y_t, f"{label} outputs")
    assert not check_gave_up or nat.gave_up_count() == 0
    return y


def _run_backward(nat, dy, c, y, reverse, tuning, label, check_gave_up=True):
    """The backward pass alone, from outputs `y` that a forward left on the device."""
    dev = torch.device("cuda:0")
    dx_t, dc_t = oracle.bwd(dy.numpy().astype(np.float64), c.numpy().astype(np.float64),
                            y.cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
    dx, dc = nat.bwd(dy.to(dev), c.to(dev), y, reverse, tuning, out=(_nan_like(y), _nan_like(y)))
    torch.cuda.synchronize()
    check_close(dx, dx_t, f"{label} d_inputs")
    check_close(dc, dc_t, f"{label} d_coeffs")
    assert not check_gave_up or nat.gave_up_count() == 0


def _tunings_for(nat, L):
    """Default table plus every compiled tile geometry that can serve a row of L elements."""
    out = [None]
    for waves, slots, carry in [(1, 1, 0), (1, 2, 0), (1, 4, 0), (1, 8, 0), (2, 1, 0), (2, 2, 0), (2, 4, 0),
                                (4, 1, 0), (4, 2, 0), (4, 4, 0), (4, 8, 0), (8, 2, 0), (8, 4, 0), (16, 2, 0), (16, 4, 0),
                                (1, 4, 1), (4, 2, 1), (4, 4, 1), (4, 8, 1), (8, 4, 1), (8, 8, 1), (16, 4, 1)]:
        tile = waves * slots * 256
        if carry == 0 and L + 3 > tile:
            continue
        if carry == 1 and (L + 3) // tile > 300:
            continue
        out.append(nat.Tuning(nat.FAMILY_TILE, waves, slots, carry))
    for waves, slots in [(4, 4), (8, 2), (8, 4), (16, 2), (8, 8)]:
        out.append(nat.Tuning(nat.FAMILY_STREAM, waves, slots, -1))
    # look-back with several tiles (of different rows) per workgroup
    for (waves, slots), tasks in zip([(4, 2), (4, 4), (8, 2), (8, 4)], [2, 3, 5, 64]):
        if (L + 3) // (waves * slots * 256) <= 300:
            out.append(nat.Tuning(nat.FAMILY_TILE, waves, slots, 1, tasks))
    # several workgroups per row, exchanging per-tile maps
    for (waves, slots), team in zip([(4, 2), (4, 4), (8, 2), (8, 4)], [2, 3, 4, 64]):
        out.append(nat.Tuning(nat.FAMILY_TEAM, waves, slots, -1, team))
    # teams that go on from row to row (rows of a whole number of tiles only)
    for waves, slots in [(4, 4), (8, 2), (8, 4), (8, 8)]:
        tile = waves * slots * 256
        if L % tile == 0 and L // tile <= 64:
            k = L // tile
            out.append(nat.Tuning(nat.FAMILY_SWEEP, waves, slots, -1, 0))      # team = tiles of a row (up to 16)
            out.append(nat.Tuning(nat.FAMILY_SWEEP, waves, slots, 3, 0))       # three teams share the rows
            if k % 2 == 0:
                out.append(nat.Tuning(nat.FAMILY_SWEEP, waves, slots, 2, k // 2))  # two tiles of a row per walker
    # the same launch shape with tiles stored two steps late (the backward is compiled for tiles of 4096 elements only)
    for waves, slots in [(8, 2), (8, 4), (4, 4), (16, 1), (16, 2)]:
        tile = waves * slots * 256
        if L % tile == 0 and L // tile <= 64:
            k = L // tile
            both = (waves, slots) in ((8, 2), (16, 1))
            out.append((nat.Tuning(nat.FAMILY_DRIFT, waves, slots, -1, 0), both))    # team = tiles of a row
            out.append((nat.Tuning(nat.FAMILY_DRIFT, waves, slots, 3, 0), both))     # three teams share the rows
            out.append((nat.Tuning(nat.FAMILY_DRIFT, waves, slots, 1, 1), both))     # one walker takes whole rows
            if k % 2 == 0:
                out.append((nat.Tuning(nat.FAMILY_DRIFT, waves, slots, 2, k // 2), both))  # two tiles of a row per walker
    return out


SEQLENS = [1, 2, 3, 5, 16, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 1025, 2047, 2048, 2049,
           4095, 4096, 4097, 5000, 8191, 8192, 8193, 16384, 16385, 40000, 65536, 100003]


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("L", SEQLENS)
def test_seqlen_sweep_all_geometries(nat, L, reverse):
    numseq = 7 if L > 4096 else 37
    x, c, dy = make_inputs((numseq, L), "signed" if L <= 64 else "uniform", seed=L)
    for tuning in _tunings_for(nat, L):
        backward_too = True
        if isinstance(tuning, tuple):
            tuning, backward_too = tuning
        label = f"L={L} rev={reverse} tune={None if tuning is None else (tuning.family, tuning.waves, tuning.slots, tuning.carry, tuning.tasks)}"
        print(label, flush=True)
        if backward_too:
            _run_both(nat, x, c, dy, reverse, tuning, label)
        else:
            _run_forward(nat, x, c, reverse, tuning, label)


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("shape", [(1, 4096), (2, 100), (255, 513), (256, 512), (25600, 48), (3, 5, 300), (2048,)])
def test_numseq_and_rank_sweep(nat, shape, reverse):
    x, c, dy = make_inputs(shape, "uniform", seed=sum(shape))
    _run_both(nat, x, c, dy, reverse, None, f"shape={shape} rev={reverse}")


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("L,width", [(100, 128), (1000, 1001), (4099, 4100), (70000, 70002)])
def test_row_padded_views(nat, L, width, reverse):
    """t[:, :L] of a wider tensor: rows start at varying 16-byte misalignments and the padding must
    stay untouched (the reference's kernels assume dense rows, linrec_pipe.cuh:14)."""
    xw, cw, dyw = make_inputs((9, width), "uniform", seed=L)
    dev = torch.device("cuda:0")
    xd, cd, dyd = (t.to(dev)[:, :L] for t in (xw, cw, dyw))
    y_t, dx_t, dc_t = truth(xw[:, :L], cw[:, :L], dyw[:, :L], reverse)
    from linrec_amd import _native
    ybuf = torch.full((9, width), float("nan"), device=dev)
    y = _native.fwd(xd, cd, reverse, out=ybuf[:, :L])
    torch.cuda.synchronize()
    check_close(y, y_t, "padded outputs")
    assert torch.isnan(ybuf[:, L:]).all(), "kernel wrote into the row padding"
    dxbuf = torch.full((9, width), float("nan"), device=dev)
    dcbuf = torch.full((9, width), float("nan"), device=dev)
    dx, dc = _native.bwd(dyd, cd, y, reverse, out=(dxbuf[:, :L], dcbuf[:, :L]))
    torch.cuda.synchronize()
    check_close(dx, dx_t, "padded d_inputs")
    check_close(dc, dc_t, "padded d_coeffs")
    assert torch.isnan(dxbuf[:, L:]).all() and torch.isnan(dcbuf[:, L:]).all()


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("offset", [1, 2, 3])
def test_misaligned_base_pointers(nat, offset, reverse):
    """Views that start 4, 8 or 12 bytes past a 16-byte boundary (all tensors alike)."""
    L, n = 3001, 5
    x, c, dy = make_inputs((n, L), "uniform", seed=offset)
    dev = torch.device("cuda:0")

    def shifted(t):
        buf = torch.full((n * L + 8,), float("nan"), device=dev)
        v = buf[offset:offset + n * L].view(n, L)
        v.copy_(t)
        return v

    xd, cd, dyd = shifted(x), shifted(c), shifted(dy)
    y_t, dx_t, dc_t = truth(x, c, dy, reverse)
    y = nat.fwd(xd, cd, reverse, out=shifted(torch.full((n, L), float("nan"))))
    dx, dc = nat.bwd(dyd, cd, y, reverse, out=(shifted(torch.full((n, L), float("nan"))),
                                               shifted(torch.full((n, L), float("nan")))))
    torch.cuda.synchronize()
    check_close(y, y_t, "misaligned outputs")
    check_close(dx, dx_t, "misaligned d_inputs")
    check_close(dc, dc_t, "misaligned d_coeffs")


@pytest.mark.parametrize("reverse", [False, True])
def test_bases_with_different_alignment_use_scalar_slots(nat, reverse):
    L, n = 2500, 3
    x, c, dy = make_inputs((n, L), "uniform", seed=77)
    dev = torch.device("cuda:0")
    xbuf = torch.empty(n * L + 4, device=dev)
    xd = xbuf[1:1 + n * L].view(n, L)
    xd.copy_(x)
    cd, dyd = c.to(dev), dy.to(dev)
    ybuf = torch.full((n * L + 4,), float("nan"), device=dev)
    yd = ybuf[1:1 + n * L].view(n, L)
    lib = nat.lib()
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
    rc = lib.linrec_fwd_f32(xd.data_ptr(), cd.data_ptr(), yd.data_ptr(), n, L, L, 1, int(reverse),
                            ws.data_ptr(), ws.numel(), None, stream)
    assert rc == 0, lib.linrec_hip_error_string(rc)
    torch.cuda.synchronize()
    y_t, dx_t, dc_t = truth(x, c, dy, reverse)
    check_close(yd, y_t, "mixed-alignment outputs")
    dxd, dcd = torch.full((n, L), float("nan"), device=dev), torch.full((n, L), float("nan"), device=dev)
    rc = lib.linrec_bwd_f32(dyd.data_ptr(), cd.data_ptr(), yd.data_ptr(), dxd.data_ptr(), dcd.data_ptr(),
                            n, L, L, 1, int(reverse), ws.data_ptr(), ws.numel(), None, stream)
    assert rc == 0
    torch.cuda.synchronize()
    check_close(dxd, dx_t, "mixed-alignment d_inputs")
    check_close(dcd, dc_t, "mixed-alignment d_coeffs")


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("shape", [(1024, 64), (4096, 256), (1001, 33), (4, 1000), (8192, 96), (12289, 17), (130, 2500),
                                   (2, 70001), (16384, 300)])
def test_transposed_views_column_and_segment_kernels(nat, shape, reverse):
    """Scan axis strided, rows adjacent.  Without a tuning: the segmented launches (reduce, carry,
    apply) for fewer than 4096 rows of at least 256 elements, the column kernels otherwise (their
    block form up to 32768 rows, the element-wise one for an odd row count).  Every family is also forced on every shape."""
    x, c, dy = make_inputs(shape, "uniform", seed=shape[0], transposed=True)
    assert x.stride() == (1, shape[0])
    xd = x.to("cuda:0")
    segmented = shape[0] < 4096 and shape[1] >= 256
    plan = nat.plan(xd, reverse)
    assert plan["family"] == (nat.FAMILY_SEGMENT if segmented else nat.FAMILY_COLUMN), plan
    if segmented:
        assert plan["tiles_per_row"] * plan["tasks"] >= shape[1] > (plan["tiles_per_row"] - 1) * plan["tasks"], plan
    _run_both(nat, x, c, dy, reverse, None, f"transposed {shape}")
    for depth in (4, 16):
        tuning = nat.Tuning(nat.FAMILY_COLUMN if shape[0] % 4 == 0 else nat.FAMILY_NAIVE, 0, depth, -1)
        _run_both(nat, x, c, dy, reverse, tuning, f"transposed {shape} depth={depth}")
    for rows_per_lane, segments in [(1, 2), (1, 7), (0, 64), (2, 3), (4, 5), (1, 2500)]:
        if shape[0] % max(rows_per_lane, 1) or shape[1] < segments:
            continue
        tuning = nat.Tuning(nat.FAMILY_SEGMENT, rows_per_lane, 8, -1, segments)
        _run_both(nat, x, c, dy, reverse, tuning, f"transposed {shape} rows/lane={rows_per_lane} segments={segments}")


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
def test_column_block_kernels(nat, reverse, dtype):
    """Scan axis strided, the 16 waves of a workgroup share rows and take runs of 8 positions each
    (steps of 128 positions; the backward with two rows per lane: runs of 4, steps of 64), or a wave
    is split into two groups of 32 lanes that share rows (steps of 256 positions).  Forced on row
    lengths around whole steps and on row counts that leave lanes without rows; chosen by the
    planner from 4096 rows (backward 6144; 16-bit storage 8192, backward 10240) on."""
    C = nat.FAMILY_COLUMN
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    # (rows per lane, lane groups per wave)
    forms = ((1, 1), (2, 1), (1, 2), (2, 2)) if dtype == torch.float32 else ((2, 1), (2, 2))
    dev = torch.device("cuda:0")
    for n, L in [(64, 1), (2, 2), (130, 7), (66, 127), (128, 128), (1000, 129), (62, 255), (190, 256), (34, 257),
                 (300, 1000), (4098, 300)]:
        x, c, dy = (t.to(dtype) for t in make_inputs((n, L), "uniform", seed=n + L, transposed=True))
        y_t, dx_t, dc_t = truth(x.float(), c.float(), dy.float(), reverse)
        xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
        assert xd.stride() == (1, n)
        for v, g in forms:
            if L == 1 and v > 1:
                continue  # a single position has no strided axis for adjacent rows to share
            tuning = nat.Tuning(C, v, 0, g, 0)
            plan = nat.plan(xd, reverse, False, tuning)
            assert (plan["carry"], plan["block"], plan["vec"], plan["grid"]) == (g, 1024, v, -(-(n // v) // (64 // g))), plan
            y = nat.fwd(xd, cd, reverse, tuning, out=_nan_like(xd))
            dx, dc = nat.bwd(dyd, cd, y, reverse, tuning, out=(_nan_like(xd), _nan_like(xd)))
            torch.cuda.synchronize()
            what = f"{n} x {L} rows/lane={v} groups={g}"
            check_close(y, y_t, what + " outputs", tol)
            dx_w, dc_w = (dx_t, dc_t) if dtype == torch.float32 else oracle.bwd(
                dy.float().numpy(), c.float().numpy(), y.float().cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
            check_close(dx, dx_w, what + " d_inputs", tol)
            check_close(dc, dc_w, what + " d_coeffs", tol)
    # the planner's own choice, both passes
    n = 8192 if dtype == torch.float32 else 24576
    x, c, dy = (t.to(dtype) for t in make_inputs((n, 300), "uniform", seed=5, transposed=True))
    xd = x.to(dev)
    for is_bwd in (False, True):
        plan = nat.plan(xd, reverse, is_bwd)
        assert (plan["family"], plan["block"]) == (C, 1024) and plan["carry"] == (2 if dtype == torch.float32 else 1), plan
    if dtype == torch.float32:
        _run_both(nat, x, c, dy, reverse, None, f"transposed {n} x 300")
    # a row with non-finite values stays alone with them, in both passes
    x, c, dy = (t.to(dtype) for t in make_inputs((130, 700), "uniform", seed=9, transposed=True))
    x[5, 300] = float("nan")
    c[77, 10] = float("inf")
    xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
    tuning = nat.Tuning(C, forms[-1][0], 0, forms[-1][1], 0)
    y = nat.fwd(xd, cd, reverse, tuning)
    clean = torch.ones(130, dtype=torch.bool)
    clean[5] = clean[77] = False
    assert torch.isfinite(y.cpu()[clean]).all() and not torch.isfinite(y.cpu()[5]).all() and not torch.isfinite(y.cpu()[77]).all()
    y_clean = torch.where(torch.isfinite(y), y, torch.zeros_like(y))
    dyd[5, 100] = float("nan")
    dx, dc = nat.bwd(dyd, cd, y_clean, reverse, tuning)
    torch.cuda.synchronize()
    assert torch.isfinite(dx.cpu()[clean]).all() and torch.isfinite(dc.cpu()[clean]).all()
    assert not torch.isfinite(dx.cpu()[5]).all() and not torch.isfinite(dx.cpu()[77]).all()


@pytest.mark.parametrize("reverse", [False, True])
def test_column_drift_kernels(nat, reverse):
    """Scan axis strided, teams of workgroups that share a block of 64 rows (128 with two rows per lane) and take
    its steps along the scan axis in turn, a step stored two of the workgroup's steps late.  Every compiled
    geometry (waves per workgroup, positions per run, rows per lane) is forced with team sizes from 1 to the
    number of waves on row lengths around whole steps, on fewer steps than team members allow and on row counts
    that leave lanes without rows; then the planner's own choice, non-finite values, a batch of time-major
    matrices, and a poll limit of one."""
    D = nat.FAMILY_COLDRIFT
    dev = torch.device("cuda:0")
    geometries = [(16, 8, 1, False), (16, 4, 1, True), (8, 16, 1, None)]  # last: the pass compiled (None: both)
    for n, L in [(64, 128), (2, 129), (130, 257), (66, 1000), (1000, 1290), (190, 2048), (34, 5000), (4098, 700)]:
        x, c, dy = make_inputs((n, L), "uniform", seed=n + L, transposed=True)
        y_t, dx_t, dc_t = truth(x, c, dy, reverse)
        xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
        assert xd.stride() == (1, n)
        for waves, run, v, only_bwd in geometries:
            if n % v:
                continue
            steps = -(-L // (waves * run))
            blocks = -(-(n // v) // 64)
            for team in sorted({1, 2, 3, min(waves, steps), min(8, steps)}):
                if team > steps or blocks * team > 256:
                    continue
                tuning = nat.Tuning(D, waves, run, v, team)
                what = f"{n} x {L} waves={waves} run={run} rows/lane={v} team={team}"
                y = torch.from_numpy(y_t).float().to(dev).t().contiguous().t() if only_bwd else None
                if only_bwd is not True:
                    plan = nat.plan(xd, reverse, False, tuning)
                    assert (plan["family"], plan["block"], plan["tasks"], plan["grid"], plan["tiles_per_row"]) == (
                        D, 64 * waves, team, blocks * team, steps), plan
                    y = nat.fwd(xd, cd, reverse, tuning, out=_nan_like(xd))
                    torch.cuda.synchronize()
                    check_close(y, y_t, what + " outputs")
                if only_bwd is not False:
                    dx, dc = nat.bwd(dyd, cd, y, reverse, tuning, out=(_nan_like(xd), _nan_like(xd)))
                    torch.cuda.synchronize()
                    check_close(dx, dx_t, what + " d_inputs")
                    check_close(dc, dc_t, what + " d_coeffs")
        assert nat.gave_up_count() == 0
    # the planner's own choice, both passes: teams of 8 on 2048 rows
    x, c, dy = make_inputs((2048, 4100), "sigmoid", seed=5, transposed=True)
    for is_bwd in (False, True):
        plan = nat.plan(x.to(dev), reverse, is_bwd)
        assert (plan["family"], plan["tasks"], plan["grid"]) == (D, 8, 256), plan
    _run_both(nat, x, c, dy, reverse, None, "transposed 2048 x 4100")
    # a batch of time-major matrices: 3 x (2100 timesteps x 1344 channels) scanned over time
    g = torch.Generator().manual_seed(11)
    xb, cb, dyb = (f((3, 2100, 1344), generator=g) for f in (torch.randn, torch.rand, torch.randn))
    xv, cv, dyv = (t.to(dev).transpose(1, 2) for t in (xb, cb, dyb))
    plan = nat.plan(xv, reverse, False)
    assert plan["family"] == D and plan["grid"] == 63 * plan["tasks"], plan
    y = nat.fwd(xv, cv, reverse)
    dx, dc = nat.bwd(dyv, cv, y, reverse)
    torch.cuda.synchronize()
    y_t, dx_t, dc_t = truth(xb.transpose(1, 2), cb.transpose(1, 2), dyb.transpose(1, 2), reverse)
    check_close(y, y_t, "batched outputs")
    check_close(dx, dx_t, "batched d_inputs")
    check_close(dc, dc_t, "batched d_coeffs")
    # a row with non-finite values stays alone with them, in both passes
    x, c, dy = make_inputs((130, 3000), "uniform", seed=9, transposed=True)
    x[5, 300] = float("nan")
    c[77, 10] = float("inf")
    xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
    y = nat.fwd(xd, cd, reverse, nat.Tuning(D, 16, 8, 1, 4))
    clean = torch.ones(130, dtype=torch.bool)
    clean[5] = clean[77] = False
    assert torch.isfinite(y.cpu()[clean]).all() and not torch.isfinite(y.cpu()[5]).all() and not torch.isfinite(y.cpu()[77]).all()
    y_clean = torch.where(torch.isfinite(y), y, torch.zeros_like(y))
    dyd[5, 100] = float("nan")
    dx, dc = nat.bwd(dyd, cd, y_clean, reverse, nat.Tuning(D, 8, 16, 1, 4))
    torch.cuda.synchronize()
    assert torch.isfinite(dx.cpu()[clean]).all() and torch.isfinite(dc.cpu()[clean]).all()
    assert not torch.isfinite(dx.cpu()[5]).all() and not torch.isfinite(dx.cpu()[77]).all()
    # a poll limit of one: waits run out, the value entering a step comes from the rows' own data instead
    x, c, dy = make_inputs((700, 6000), "uniform", seed=3, transposed=True)
    y_t, dx_t, dc_t = truth(x, c, dy, reverse)
    xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
    old = nat.lib().linrec_set_spin_limit(1)
    try:
        y = nat.fwd(xd, cd, reverse, nat.Tuning(D, 16, 8, 1, 8))
        dx, dc = nat.bwd(dyd, cd, y, reverse, nat.Tuning(D, 8, 16, 1, 8))
        torch.cuda.synchronize()
    finally:
        nat.lib().linrec_set_spin_limit(old)
    print("column drift, poll limit 1: waits that ran out:", nat.gave_up_count(), flush=True)
    check_close(y, y_t, "poll limit 1 outputs")
    check_close(dx, dx_t, "poll limit 1 d_inputs")
    check_close(dc, dc_t, "poll limit 1 d_coeffs")
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0  # (the other tests take a count of zero as the sign that nobody had to fall back)


@pytest.mark.parametrize("seed", range(8))
def test_block_range_row_counts_through_the_operator(nat, seed):
    """Random (batch, time, channels) and (time, channels) tensors whose row counts fall where the
    planner picks the column block kernels, scanned over time through the public operator and
    autograd: channel counts that make lanes of one wave belong to different batches, odd counts
    (one row per lane), 16-bit storage, both directions."""
    import linrec_amd
    rng = np.random.default_rng(1000 + seed)
    dev = torch.device("cuda:0")
    dtype = [torch.float32, torch.float32, torch.bfloat16, torch.float16][seed % 4]
    batch = int(rng.integers(1, 10))
    lo = 4096 if dtype == torch.float32 else 8192
    rows = int(rng.integers(lo, 34000))
    channels = max(1, rows // batch) + int(rng.integers(0, 2))
    T = int(rng.integers(256, 700))
    reverse = bool(seed & 1)
    shape = (batch, T, channels) if batch > 1 else (T, channels)
    g = torch.Generator().manual_seed(seed)
    x, c, dy = (f(shape, generator=g).to(dtype) for f in (torch.randn, torch.rand, torch.randn))
    xt = x.to(dev).transpose(-1, -2)
    plans = [nat.plan(xt, reverse, b) for b in (False, True)]
    # (16-bit storage has no block form for single rows per lane, which an odd channel count needs)
    blocked = dtype == torch.float32 or channels % 2 == 0
    assert (plans[0]["family"] == nat.FAMILY_COLUMN and plans[0]["carry"] >= 1) == blocked, (shape, plans)
    xr, cr = x.to(dev).requires_grad_(), c.to(dev).requires_grad_()
    y = linrec_amd.linrec(xr, cr, reverse=reverse, dim=-2)
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    assert y.is_contiguous() and xr.grad.is_contiguous() and cr.grad.is_contiguous()
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    xs, cs, dys = (t.float().transpose(-1, -2) for t in (x, c, dy))
    y_t = oracle.fwd(xs.numpy(), cs.numpy(), reverse, dtype=np.float64)
    dx_t, dc_t = oracle.bwd(dys.numpy(), cs.numpy(), y.detach().float().cpu().transpose(-1, -2).numpy().astype(np.float64),
                            reverse, dtype=np.float64)
    what = f"{shape} {dtype} reverse={reverse} plans {[(p['family'], p['carry'], p['vec']) for p in plans]}"
    check_close(y.transpose(-1, -2), y_t, what + " outputs", tol)
    check_close(xr.grad.transpose(-1, -2), dx_t, what + " d_inputs", tol)
    check_close(cr.grad.transpose(-1, -2), dc_t, what + " d_coeffs", tol)


def test_segment_tuning_limits(nat):
    x = torch.zeros(5000, 64, device="cuda:0").t()
    with pytest.raises(NotImplementedError):
        nat.plan(x, tuning=nat.Tuning(nat.FAMILY_SEGMENT, 0, 8, -1, 4097))  # more segments than the library takes
    with pytest.raises(NotImplementedError):
        nat.plan(x, tuning=nat.Tuning(nat.FAMILY_SEGMENT, 8, 8, -1, 4))  # eight floats per lane: no such kernel
    with pytest.raises(NotImplementedError):
        nat.plan(x.t(), tuning=nat.Tuning(nat.FAMILY_SEGMENT))  # unit-stride scan axis
    # a workspace smaller than the plan asks for is refused before anything is launched
    lib = nat.lib()
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda:0")
    rc = lib.linrec_fwd_f32(x.data_ptr(), x.data_ptr(), torch.empty_like(x).data_ptr(), 64, 5000, 1, 64, 0,
                            ws.data_ptr(), ws.numel(), None, torch.cuda.current_stream().cuda_stream)
    assert rc == -2


@pytest.mark.parametrize("elem", [torch.float32, torch.bfloat16], ids=["4B", "2B"])
def test_transpose_entry_point(nat, elem):
    """linrec_transpose through the C ABI: tile-edge shapes, batches, bases that are not 16-byte
    aligned; bit-exact against torch's transpose."""
    dev = torch.device("cuda:0")
    lib = nat.lib()
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(11)
    for (b, r, c) in [(1, 64, 64), (1, 1000, 77), (3, 129, 257), (2, 512, 1024), (1, 20000, 64), (1, 5, 3), (4, 63, 2),
                      (1, 1, 300), (1, 300, 1)]:
        for off_src, off_dst in [(0, 0), (3, 1)]:
            src = torch.randn(b * r * c + off_src, generator=g).to(elem).to(dev)[off_src:].view(b, r, c)
            dst = torch.full((b * c * r + off_dst,), float("nan"), dtype=elem, device=dev)
            rc = lib.linrec_transpose(src.element_size(), src.data_ptr(), dst[off_dst:].data_ptr(), b, r, c, stream)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(dst[off_dst:].view(b, c, r), src.transpose(1, 2)), (b, r, c, off_src, off_dst)
            assert off_dst == 0 or torch.isnan(dst[0]).item()
    src = torch.zeros(8, device=dev)
    assert lib.linrec_transpose(8, src.data_ptr(), src.data_ptr(), 1, 2, 2, stream) == -1  # element size
    assert lib.linrec_transpose(4, src.data_ptr(), src.data_ptr(), 1, -2, 2, stream) == -1
    assert lib.linrec_transpose(4, None, None, 1, 0, 2, stream) == 0  # nothing to do


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["f32", "f16"])
def test_time_major_data_with_few_rows(nat, reverse, dtype):
    """The scan axis is the strided one and rows are few.  Adjacent rows (a transposed matrix) are
    served in place by the segmented launches; rows further apart are transposed into dense rows by
    the binding, scanned there and transposed back.  Results keep the inputs' strides either way."""
    dev = torch.device("cuda:0")
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -9
    g = torch.Generator().manual_seed(21)

    def check(x, c, dy, what, re_laid_out):
        assert nat._few_rows_on_strided_axis(x, nat.row_layout(x), None) == re_laid_out, what
        if not re_laid_out and x.size(-1) >= 256:
            # (fp32 rows that fill the chip in teams along the scan axis take the column drift kernels)
            assert nat.plan(x, reverse)["family"] in (nat.FAMILY_SEGMENT, nat.FAMILY_COLDRIFT), what
        y = nat.fwd(x, c, reverse)
        dx, dc = nat.bwd(dy, c, y, reverse)
        torch.cuda.synchronize()
        assert y.stride() == x.stride() and dx.stride() == x.stride() and dc.stride() == x.stride(), what
        y_t, _, _ = truth(x.float(), c.float(), dy.float(), reverse)
        dx_t, dc_t = oracle.bwd(dy.float().cpu().numpy(), c.float().cpu().numpy(),
                                y.float().cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
        check_close(y, y_t, what + " outputs", tol)
        check_close(dx, dx_t, what + " d_inputs", tol)
        check_close(dc, dc_t, what + " d_coeffs", tol)

    for (n, L) in [(64, 5000), (1000, 777), (7, 333), (2048, 4096), (2048, 1500)]:
        x, c, dy = (f((L, n), generator=g).to(dtype).to(dev).t() for f in (torch.randn, torch.rand, torch.randn))
        check(x, c, dy, f"transposed {n} x {L}", False)
        assert (nat.plan(x, reverse)["family"] == nat.FAMILY_COLDRIFT) == ((n, L) == (2048, 4096) and dtype == torch.float32)
    # leading dims that collapse into the rows of one transposed matrix: (L, A, B) seen as (A, B, L)
    x, c, dy = (f((300, 5, 12), generator=g).to(dtype).to(dev).permute(1, 2, 0) for f in (torch.randn, torch.rand, torch.randn))
    check(x, c, dy, "permuted (5, 12, 300)", False)
    # coefficients close to one: what enters a segment carries far into it, so the maps of all segments in
    # front of it matter (with uniform coefficients a segment forgets its entry within a few steps)
    x, c, dy = (f((6000, 96), generator=g).to(dev) for f in (torch.randn, torch.rand, torch.randn))
    x, c, dy = (x.to(dtype).t(), (1.0 - 0.01 * c).to(dtype).t(), dy.to(dtype).t())
    check(x, c, dy, "coefficients in [0.99, 1]", False)
    # one row with strided elements (a column of a matrix): segments of the one row side by side
    x, c, dy = (f((5000, 8), generator=g).to(dtype).to(dev)[:, 3] for f in (torch.randn, torch.rand, torch.randn))
    assert x.dim() == 1 and x.stride() == (8,) and nat.plan(x, reverse)["tiles_per_row"] > 100
    check(x, c, dy, "a column of a matrix", False)
    # rows two elements apart (every other row of a transposed matrix): re-laid out by the binding
    x, c, dy = (f((300, 120), generator=g).to(dtype).to(dev).t()[::2] for f in (torch.randn, torch.rand, torch.randn))
    check(x, c, dy, "every other row of a transposed matrix", True)
    # the same with the result tensors of a transposed dense matrix (the binding's transpose kernel)
    x, c, dy = (f((400, 96), generator=g).to(dtype).to(dev).t() for f in (torch.randn, torch.rand, torch.randn))
    nat._RELAYOUT_UNIT_ROW_STRIDE = True
    try:
        check(x, c, dy, "transposed 96 x 400 through the re-layout", True)
    finally:
        nat._RELAYOUT_UNIT_ROW_STRIDE = False


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_batches_of_time_major_matrices(nat, reverse, dtype):
    """(batch, time, channels) scanned over dim 1.  The transposed views do not collapse into
    uniformly strided rows; the batched entry points take them as they are (column kernels and their
    segmented form, with a batch stride), so results and gradients come back dense in the caller's
    layout."""
    import linrec_amd
    dev = torch.device("cuda:0")
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    g = torch.Generator().manual_seed(22)
    S, C, N = nat.FAMILY_SEGMENT, nat.FAMILY_COLUMN, nat.FAMILY_NAIVE
    for shape, family, tunings in [((3, 700, 130), S, [nat.Tuning(S, 1, 8, -1, 3), nat.Tuning(C, 0, 8), nat.Tuning(N, 0, 8), nat.Tuning(C, 2, 0, 1, 0)]),
                                   ((2, 300, 33), S, [nat.Tuning(S, 0, 8, -1, 7), nat.Tuning(N, 0, 8)]),
                                   ((5, 64, 8), C, [nat.Tuning(S, 2, 8, -1, 2)]),
                                   ((2, 3, 260, 16), S, [])]:
        x, c, dy = (f(shape, generator=g).to(dtype).to(dev) for f in (torch.randn, torch.rand, torch.randn))
        xt, ct, dyt = (t.transpose(-1, -2) for t in (x, c, dy))
        assert nat.row_layout(xt) is None
        B, L, Ch = x.numel() // (shape[-1] * shape[-2]), shape[-2], shape[-1]
        assert nat.batched_layout(xt) == (B, Ch, L, L * Ch, 1, Ch)
        assert nat.plan(xt, reverse)["family"] == family
        xr, cr = x.clone().requires_grad_(), c.clone().requires_grad_()
        y = linrec_amd.linrec(xr, cr, reverse=reverse, dim=-2)
        y.backward(dy)
        torch.cuda.synchronize()
        assert y.is_contiguous() and xr.grad.is_contiguous() and cr.grad.is_contiguous()
        y_t, _, _ = truth(xt.float(), ct.float(), dyt.float(), reverse)
        dx_t, dc_t = oracle.bwd(dyt.float().cpu().numpy(), ct.float().cpu().numpy(),
                                y.detach().transpose(-1, -2).float().cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
        check_close(y.transpose(-1, -2), y_t, f"{shape} outputs", tol)
        check_close(xr.grad.transpose(-1, -2), dx_t, f"{shape} d_inputs", tol)
        check_close(cr.grad.transpose(-1, -2), dc_t, f"{shape} d_coeffs", tol)
        for tuning in tunings:
            yk = nat.fwd(xt, ct, reverse, tuning, out=torch.full_like(x, float("nan")).transpose(-1, -2))
            dxk, dck = nat.bwd(dyt, ct, yk, reverse, tuning, out=(torch.full_like(x, float("nan")).transpose(-1, -2),
                                                                 torch.full_like(x, float("nan")).transpose(-1, -2)))
            torch.cuda.synchronize()
            what = f"{shape} tuning {(tuning.family, tuning.waves, tuning.slots, tuning.tasks)}"
            check_close(yk, y_t, what + " outputs", tol)
            check_close(dxk, dx_t, what + " d_inputs", tol)
            check_close(dck, dc_t, what + " d_coeffs", tol)
    # views that start inside a 16-byte slot, and tensors whose phases disagree
    big = [f((2, 301, 24), generator=g).to(dtype).to(dev) for f in (torch.randn, torch.rand)]
    x, c = (t[:, 1:, 4:20].transpose(1, 2) for t in big)  # channel stride 24, 16 channels, offset 28 elements
    assert nat.batched_layout(x) == (2, 16, 300, 301 * 24, 1, 24)
    y = nat.fwd(x, c, reverse)
    y2 = nat.fwd(x, c.contiguous().transpose(1, 2).contiguous().transpose(1, 2), reverse)
    torch.cuda.synchronize()
    want = oracle.fwd(x.float().cpu().numpy(), c.float().cpu().numpy(), reverse, dtype=np.float64)
    check_close(y, want, "offset views", tol)
    check_close(y2, want, "coefficients at another phase", tol)
    # mixed layouts: dense inputs, coefficients as a batch of transposed matrices (the binding's batched transpose)
    xd = torch.randn((3, 40, 500), generator=g).to(dtype).to(dev)
    cm = torch.rand((3, 500, 40), generator=g).to(dtype).to(dev).transpose(1, 2)
    assert nat._as_transposed_matrices(cm) == (3, 500, 40)
    check_close(nat.fwd(xd, cm, reverse), oracle.fwd(xd.float().cpu().numpy(), cm.float().cpu().numpy(), reverse, dtype=np.float64),
                "mixed layouts", tol)


def test_batched_entry_points_reject_what_they_cannot_describe(nat):
    dev = torch.device("cuda:0")
    lib = nat.lib()
    x = torch.zeros(4 * 50 * 8, device=dev)
    y = torch.empty_like(x)
    s = torch.cuda.current_stream().cuda_stream
    f32 = nat.DTYPES[torch.float32]
    # unit stride along the scan axis: to be described as rows
    assert lib.linrec_fwd_batched(f32, x.data_ptr(), x.data_ptr(), y.data_ptr(), 4, 8, 50, 400, 50, 1, 0, None, 0, None, s) == -3
    # tile kernels take no batch stride
    tile = nat.Tuning(nat.FAMILY_TILE, 4, 4, 0)
    assert lib.linrec_fwd_batched(f32, x.data_ptr(), x.data_ptr(), y.data_ptr(), 4, 8, 50, 400, 1, 8, 0, None, 0,
                                  ctypes.byref(tile), s) == -3
    assert lib.linrec_fwd_batched(f32, x.data_ptr(), x.data_ptr(), y.data_ptr(), -1, 8, 50, 400, 1, 8, 0, None, 0, None, s) == -1
    assert lib.linrec_fwd_batched(f32, x.data_ptr(), x.data_ptr(), y.data_ptr(), 0, 8, 50, 400, 1, 8, 0, None, 0, None, s) == 0
    # one batch is the unbatched call
    g = torch.Generator().manual_seed(3)
    xv, cv = torch.randn(50, 8, generator=g).to(dev), torch.rand(50, 8, generator=g).to(dev)
    y1, y2 = torch.empty_like(xv), torch.empty_like(xv)
    assert lib.linrec_fwd_batched(f32, xv.data_ptr(), cv.data_ptr(), y1.data_ptr(), 1, 8, 50, 400, 1, 8, 0, None, 0, None, s) == 0
    assert lib.linrec_fwd_f32(xv.data_ptr(), cv.data_ptr(), y2.data_ptr(), 8, 50, 1, 8, 0, None, 0, None, s) == 0
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("reverse", [False, True])
def test_rows_beyond_one_per_cu_take_a_second_launch(nat, reverse):
    """257 to 352 long ragged rows: the first 256 go to one workgroup each, the rest to a launch of their
    own (a look-back chain for fewer than 6, teams of workgroups from there on), which needs a workspace
    although the first does not.  Row strides that put the second launch at another 16-byte phase."""
    dev = torch.device("cuda:0")
    for n, L, width in [(257, 9001, 9001), (261, 9001, 9003), (313, 8200, 8200), (352, 8202, 8202), (300, 20003, 20004)]:
        g = torch.Generator().manual_seed(n)
        x, c, dy = (torch.randn(n, L, generator=g), torch.rand(n, L, generator=g), torch.randn(n, L, generator=g))
        def padded(t, fill=None):
            buf = torch.full((n, width), float("nan"), device=dev)
            if fill is None:
                buf[:, :L] = t.to(dev)
            return buf[:, :L]
        xd, cd, dyd = padded(x), padded(c), padded(dy)
        plan = nat.plan(xd, reverse)
        assert (plan["family"], plan["tail_rows"], plan["grid"]) == (nat.FAMILY_STREAM, n - 256, 256), plan
        assert plan["workspace_bytes"] > 0
        y = nat.fwd(xd, cd, reverse, out=padded(None, 0))
        dx, dc = nat.bwd(dyd, cd, y, reverse, out=(padded(None, 0), padded(None, 0)))
        torch.cuda.synchronize()
        y_t, _, _ = truth(x, c, dy, reverse)
        dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y.cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
        check_close(y, y_t, f"{n} x {L} outputs")
        check_close(dx, dx_t, f"{n} x {L} d_inputs")
        check_close(dc, dc_t, f"{n} x {L} d_coeffs")
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
def test_little_work_in_many_rows_goes_to_small_teams_with_the_largest_tiles(nat, reverse):
    """A quarter of the chip's row count and more, at most four tiles of 8192 elements per compute unit: teams that
    wait, with tiles of 16384 elements, in both directions, teams of two and three among them."""
    dev = torch.device("cuda:0")
    for n, L, team in [(100, 32768, 2), (150, 49152, 3), (96, 65536, 4), (64, 131072, 8)]:
        g = torch.Generator().manual_seed(n)
        x, c, dy = (torch.randn(n, L, generator=g), torch.rand(n, L, generator=g), torch.randn(n, L, generator=g))
        xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
        for is_bwd in (False, True):
            plan = nat.plan(xd, reverse, is_bwd)
            assert (plan["family"], plan["slots"], plan["tasks"]) == (nat.FAMILY_SWEEP, 8, team), plan
        y = nat.fwd(xd, cd, reverse)
        dx, dc = nat.bwd(dyd, cd, y, reverse)
        torch.cuda.synchronize()
        y_t, _, _ = truth(x, c, dy, reverse)
        dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y.cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
        check_close(y, y_t, f"{n} x {L} outputs")
        check_close(dx, dx_t, f"{n} x {L} d_inputs")
        check_close(dc, dc_t, f"{n} x {L} d_coeffs")
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
def test_more_than_2048_rows_of_whole_tiles_run_forward_in_teams(nat, reverse):
    """Beyond 2048 rows the forward still goes to the teams whose tiles are stored two steps late: tiles of 8192
    elements in 16 waves of two slots (rows of two such tiles included), tiles of 4096 in 16 waves of one slot where
    only those divide the row and it has enough of them (the planner's generated thresholds); the backward to them as
    well up to its own threshold, else to the teams that wait or to one workgroup per row."""
    dev = torch.device("cuda:0")
    T = nat.plan_thresholds()
    k = T["drift_min_small_tiles_per_row"]
    k += 1 - k % 2  # (odd: whole tiles of 4096 elements but not of 8192)
    assert T["drift_fwd_two_tiles_min_rows"] <= 2304
    for n, L, slots, team in [(2100, 4096 * (k + 1), 2, (k + 1) // 2), (2200, 4096 * k, 1, k), (2304, 16384, 2, 2)]:
        g = torch.Generator().manual_seed(n)
        x, c, dy = (torch.randn(n, L, generator=g), torch.rand(n, L, generator=g), torch.randn(n, L, generator=g))
        xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
        plan = nat.plan(xd, reverse)
        assert (plan["family"], plan["waves"], plan["slots"], plan["tasks"]) == (nat.FAMILY_DRIFT, 16, slots, team), plan
        bwd_family = nat.plan(xd, reverse, True)["family"]
        assert bwd_family == (nat.FAMILY_DRIFT if n <= nat.plan_thresholds()["drift_bwd_max_rows"] else bwd_family)
        assert bwd_family in (nat.FAMILY_SWEEP, nat.FAMILY_STREAM, nat.FAMILY_DRIFT)
        y = nat.fwd(xd, cd, reverse)
        dx, dc = nat.bwd(dyd, cd, y, reverse)
        torch.cuda.synchronize()
        y_t, _, _ = truth(x, c, dy, reverse)
        dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y.cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
        check_close(y, y_t, f"{n} x {L} outputs")
        check_close(dx, dx_t, f"{n} x {L} d_inputs")
        check_close(dc, dc_t, f"{n} x {L} d_coeffs")
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
def test_broadcast_inputs_get_dense_results(nat, reverse):
    """Expanded tensors (zero strides: a value per row repeated along the scan axis, a row repeated for
    every row, a scalar) are valid inputs; results must not inherit strides under which elements share
    an address."""
    import linrec_amd
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(31)
    n, L = 37, 500
    per_row = torch.randn(n, 1, generator=g).to(dev)
    one_row = torch.rand(1, L, generator=g).to(dev)
    dense = torch.randn(n, L, generator=g).to(dev)
    dy = torch.randn(n, L, generator=g).to(dev)
    for x, c, what in [(per_row.expand(n, L), one_row.expand(n, L), "both expanded"),
                       (dense, torch.full((), 0.9, device=dev).expand(n, L), "scalar coefficient"),
                       (per_row.expand(n, L), torch.rand(n, L, generator=g).to(dev), "input constant along the scan"),
                       (per_row[:, 0].expand(L, n).t(), one_row.expand(n, L), "expanded, then transposed")]:
        assert nat.row_layout(x) is None or x.stride(-1) != 0
        xr, cr = x.detach().requires_grad_(), c.detach().requires_grad_()
        y = linrec_amd.linrec(xr, cr, reverse=reverse)
        y.backward(dy)
        torch.cuda.synchronize()
        assert y.is_contiguous() or y.stride() == x.stride(), what
        assert len(set(y.stride())) == y.dim() and 0 not in y.stride(), what
        y_t, dx_t, dc_t = truth(x.contiguous(), c.contiguous(), dy, reverse)
        check_close(y, y_t, what + " outputs")
        check_close(xr.grad, dx_t, what + " d_inputs")
        check_close(cr.grad, dc_t, what + " d_coeffs")


@pytest.mark.parametrize("reverse", [False, True])
def test_arbitrary_strides_naive_kernel(nat, reverse):
    g = torch.Generator().manual_seed(5)
    big = torch.randn(6, 40, 3, generator=g)
    x, c, dy = big[:, ::2, 0], torch.rand(6, 40, 3, generator=g)[:, ::2, 0], torch.randn(6, 40, 3, generator=g)[:, ::2, 0]
    dev = torch.device("cuda:0")
    xd = big.to(dev)[:, ::2, 0]
    assert xd.stride() == (120, 6)
    cd = torch.empty_strided(xd.size(), xd.stride(), device=dev).copy_(c)
    dyd = torch.empty_strided(xd.size(), xd.stride(), device=dev).copy_(dy)
    y_t, dx_t, dc_t = truth(x, c, dy, reverse)
    y = nat.fwd(xd, cd, reverse)
    dx, dc = nat.bwd(dyd, cd, y, reverse)
    torch.cuda.synchronize()
    check_close(y, y_t, "strided outputs")
    check_close(dx, dx_t, "strided d_inputs")
    check_close(dc, dc_t, "strided d_coeffs")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L", [700, 6134, 40000])
def test_offset_views_through_the_operator(L, dtype):
    """Inputs that start inside a 16-byte slot, results allocated by the operator: the results get
    the inputs' phase (so the wide accesses stay), and a caller-supplied result buffer of another
    phase is served too, through element-sized slots and, for long rows, a workspace."""
    import linrec_amd
    from linrec_amd import _native as nat
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(L)
    x, c, dy = (torch.randn(3, L, generator=g).to(dtype), torch.rand(3, L, generator=g).to(dtype),
                torch.randn(3, L, generator=g).to(dtype))

    def shifted(t, by):
        buf = torch.full((t.numel() + 16,), float("nan"), dtype=dtype, device=dev)
        v = buf[by:by + t.numel()].view(t.shape)
        v.copy_(t)
        return v

    xd, cd = shifted(x, 3).requires_grad_(), shifted(c, 3).requires_grad_()
    y = linrec_amd.linrec(xd, cd)
    assert nat._phase(y) == nat._phase(xd) == 3
    assert nat.plan(xd)["vec"] == (4 if dtype == torch.float32 else 8)
    gx, gc = torch.autograd.grad(y, (xd, cd), dy.to(dev))  # d_outputs arrives with phase 0
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    y_t = oracle.fwd(f64(x), f64(c), False)
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y), False)
    tol = TOL_NORMWISE if dtype == torch.float32 else 1.05 * 2.0 ** -8
    check_close(y.float(), y_t, "offset outputs", tol)
    check_close(gx.float(), dx_t, "offset d_inputs", tol)
    check_close(gc.float(), dc_t, "offset d_coeffs", tol)
    # result buffer with a different phase than the inputs
    out = shifted(torch.full((3, L), float("nan")).to(dtype), 5)
    y2 = nat.fwd(xd.detach(), cd.detach(), False, out=out)
    torch.cuda.synchronize()
    assert torch.equal(y2, y.detach()) or (y2.float() - y.detach().float()).abs().max() <= tol * float(np.abs(y_t).max())
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
class TestValues:
    def test_closed_forms_on_device(self, nat, reverse):
        dev = torch.device("cuda:0")
        x = torch.randn(11, 9000, generator=torch.Generator().manual_seed(1)).to(dev)
        assert torch.equal(nat.fwd(x, torch.zeros_like(x), reverse), x)
        ones = nat.fwd(x, torch.ones_like(x), reverse).cpu().double()
        xs = x.cpu().double()
        want = xs.flip(-1).cumsum(-1).flip(-1) if reverse else xs.cumsum(-1)
        assert (ones - want).abs().max() / want.abs().max() < 1e-5
        assert not nat.fwd(torch.zeros_like(x), torch.rand_like(x), reverse).any()

    def test_growing_and_negative_coeffs_short_rows(self, nat, reverse):
        g = torch.Generator().manual_seed(2)
        x = torch.randn(64, 48, generator=g)
        c = (torch.rand(64, 48, generator=g) * 3.0 - 1.5)
        _run_both(nat, x, c, torch.randn(64, 48, generator=g), reverse, None, "growth")

    def test_nonfinite_rows_do_not_leak(self, nat, reverse):
        x, c, dy = make_inputs((6, 5000), "uniform", seed=3)
        x2, c2 = x.clone(), c.clone()
        x2[1, 2500] = float("nan")
        c2[4, 100] = float("inf")
        c2[2, -1 if reverse else 0] = float("nan")  # first coefficient in scan order: never used
        dev = torch.device("cuda:0")
        base = nat.fwd(x.to(dev), c.to(dev), reverse)
        got = nat.fwd(x2.to(dev), c2.to(dev), reverse)
        torch.cuda.synchronize()
        for r in (0, 2, 3, 5):
            assert torch.equal(got[r], base[r]), r
        assert not torch.isfinite(got[1]).all() and not torch.isfinite(got[4]).all()
        # the part of row 1 scanned before the NaN is untouched
        keep = slice(2501, None) if reverse else slice(0, 2500)
        assert torch.equal(got[1, keep], base[1, keep])


def test_flip_equivalence_at_full_size(nat):
    """reverse=True equals flip -> forward -> flip, a size-independent property, at the README shape."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(512, 65536, device=dev, generator=g)
    c = torch.rand(512, 65536, device=dev, generator=g)
    a = nat.fwd(x, c, True)
    b = nat.fwd(x.flip(-1).contiguous(), c.flip(-1).contiguous(), False).flip(-1)
    assert torch.equal(a, b)


def test_workspace_survives_many_launches_and_other_shapes(nat):
    """The look-back workspace is never cleared between launches; alternate shapes and directions."""
    dev = torch.device("cuda:0")
    cases = []
    for i, (shape, rev) in enumerate([((3, 50000), False), ((40, 9000), True), ((1, 300000), False), ((3, 50000), True)]):
        x, c, dy = make_inputs(shape, "near1", seed=i)
        cases.append((x.to(dev), c.to(dev), rev, truth(x, c, dy, rev)[0]))
    for rep in range(6):
        for x, c, rev, y_t in cases:
            y = nat.fwd(x, c, rev)
            check_close(y, y_t, f"rep {rep}")
    assert nat.gave_up_count() == 0


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("rows,tiles,slots,team", [(1, 130, 2, 130), (3, 256, 2, 256), (2, 192, 4, 96), (5, 96, 4, 96),
                                                   (1, 200, 4, 200), (7, 65, 2, 65), (3, 512, 4, 0), (1, 1024, 4, 0),
                                                   (1, 130, 1, 130), (3, 256, 1, 256), (2, 240, 1, 240), (7, 65, 1, 65)])
def test_drift_teams_of_more_than_one_collecting_wave(nat, rows, tiles, slots, team, reverse):
    """Teams of more than 64 workgroups: every wave of a workgroup collects up to 64 of the team mates' maps
    and the waves' shares are composed after the barrier.  Forced team sizes on a few long rows (rows of
    `tiles` tiles of 8 waves x `slots` slots, or of 16 waves x 1 slot), and the planner's own choice (team 0),
    which for so few rows is one team of the whole chip.  The backward is compiled for tiles of 4096 elements."""
    waves = 16 if slots == 1 else 8
    L = tiles * waves * slots * 256
    x, c, dy = make_inputs((rows, L), "near1", seed=rows * 1000 + tiles)
    tuning = nat.Tuning(nat.FAMILY_DRIFT, waves, slots, -1, team) if team else None
    plan = nat.plan(x, reverse, False, tuning)
    assert plan["family"] == nat.FAMILY_DRIFT and plan["tasks"] == (team or 256) and plan["tasks"] > 64, plan
    label = f"drift {rows} x {tiles} tiles, team {plan['tasks']}"
    if slots <= 2 or tuning is None:
        _run_both(nat, x, c, dy, reverse, tuning, label)
    else:
        _run_forward(nat, x, c, reverse, tuning, label)


@pytest.mark.parametrize("reverse", [False, True])
def test_rows_with_a_partial_last_tile_run_in_drift_teams(nat, reverse):
    """fp32 rows of whole 16-byte slots whose length is not a whole number of tiles: the drift kernels' last tile of a
    row is a partial one (down to a single slot, up to a tile less a slot), the teams need not divide the tiles of a
    row, and the walk starts one tile further along in every row.  Forced geometries and team sizes on few and many
    rows, the planner's own choice, and a poll limit of one."""
    D = nat.FAMILY_DRIFT
    dev = torch.device("cuda:0")
    names = nat.kernel_table()
    for shape, teams in [((3, 8192 * 2 + 4), (0, 2, 3)), ((5, 8192 * 3 + 4096), (0, 3)), ((7, 8192 * 5 - 4), (0, 4, 5)),
                         ((33, 8192 * 4 + 1000), (0, 2, 5)), ((260, 8192 * 2 + 8), (0,)), ((2, 8192 * 13 + 8188), (0, 9, 14)),
                         ((1, 8192 * 40 + 12), (0, 7, 41))]:
        x, c, dy = make_inputs(shape, "near1", seed=shape[0] * 1000 + shape[1] % 977)
        for team in teams:
            for fw, bw in [((16, 2), (16, 1)), ((8, 4), (16, 1))]:
                tf = nat.Tuning(D, fw[0], fw[1], -1, team)
                # (the backward's tiles are half the forward's: twice the team, where one is asked for; rows of whole
                # such tiles take the kernel for them, whose teams divide the tiles of a row)
                kb = -(-shape[1] // 4096)
                team_b = min(2 * team, kb)
                if team_b and shape[1] % 4096 == 0 and kb % team_b:
                    team_b = kb
                tb = nat.Tuning(D, bw[0], bw[1], -1, team_b)
                pf, pb = nat.plan(x.to(dev), reverse, False, tf), nat.plan(x.to(dev), reverse, True, tb)
                assert "ragged" in names[pf["kernel_id"]] and pf["tiles_per_row"] == -(-shape[1] // 8192), pf
                assert ("ragged" in names[pb["kernel_id"]]) == (shape[1] % 4096 != 0) and pb["tiles_per_row"] == -(-shape[1] // 4096), pb
                if team:
                    assert pf["tasks"] == team, pf
                label = f"drift {shape} forward {fw} team {pf['tasks']}, backward team {pb['tasks']}"
                y = _run_forward(nat, x, c, reverse, tf, label)
                _run_backward(nat, dy, c, y, reverse, tb, label)
    assert nat.gave_up_count() == 0
    # the planner's own choice: teams that fill the chip, whatever the tiles of a row
    for shape, fwd, bwd in [((335, 100000), (16, 2, 13), (16, 1, 25)), ((100, 250000), (16, 2, 28), (16, 1, 61)),
                            ((16, 1000000), (8, 4, 123), (16, 1, 245)), ((1024, 50000), (16, 2, 7), (16, 1, 13))]:
        x, c, dy = make_inputs(shape, "sigmoid", seed=shape[0])
        for is_bwd, want in ((False, fwd), (True, bwd)):
            plan = nat.plan(x.to(dev), reverse, is_bwd)
            assert plan["family"] == D and "ragged" in names[plan["kernel_id"]], plan
            assert (plan["waves"], plan["slots"]) == want[:2] and plan["grid"] <= 256 and plan["grid"] % plan["tasks"] == 0, plan
        _run_both(nat, x, c, dy, reverse, None, f"drift {shape}, default plan")
    assert nat.gave_up_count() == 0
    # a poll limit of one: waits run out, the value entering a tile comes from the row's own data instead
    x, c, dy = make_inputs((6, 8192 * 50 + 5000), "near1", seed=4)
    old = nat.lib().linrec_set_spin_limit(1)
    try:
        y = _run_forward(nat, x, c, reverse, nat.Tuning(D, 16, 2, -1, 17), "poll limit 1, forward", check_gave_up=False)
        _run_backward(nat, dy, c, y, reverse, nat.Tuning(D, 16, 1, -1, 33), "poll limit 1, backward", check_gave_up=False)
    finally:
        nat.lib().linrec_set_spin_limit(old)
    print("drift with partial tiles, poll limit 1: waits that ran out:", nat.gave_up_count(), flush=True)
    for ws in list(nat._workspaces.values()):
        ws[:16].view(torch.int32)[1] = 0  # (the other tests take a count of zero as the sign that nobody had to fall back)


@pytest.mark.parametrize("kind", ["look-back", "chain", "team", "sweep", "drift", "drift-200", "drift-16-waves"])
def test_tiny_poll_limit_ends_in_right_results_not_a_hang(nat, kind):
    """Failure handling, forced from the host: with a poll limit of one, a tile whose predecessors
    have not published by its second look gives up waiting and computes the value that enters it from
    the row's own data.  Every wave still exits, the results are right, the header counts the events,
    and the workspace serves the next launch.  The same for the team, sweep and drift kernels' waits
    for their team mates' maps."""
    dev = torch.device("cuda:0")
    lib = nat.lib()
    n, L = 2, 4096 * 600
    x, c = torch.randn(n, L, device=dev), torch.rand(n, L, device=dev)
    y = torch.empty_like(x)
    ws = torch.zeros(1 << 17, dtype=torch.uint8, device=dev)  # its lower half holds header, counters, descriptors
    tune = {"look-back": nat.Tuning(nat.FAMILY_TILE, 4, 4, 1), "chain": nat.Tuning(nat.FAMILY_TILE, 4, 4, 1, 2),
            "team": nat.Tuning(nat.FAMILY_TEAM, 8, 4, -1, 4), "sweep": nat.Tuning(nat.FAMILY_SWEEP, 8, 4, -1, 0),
            "drift": nat.Tuning(nat.FAMILY_DRIFT, 8, 2, -1, 0),            # the planner's teams of 120: two collecting waves
            "drift-200": nat.Tuning(nat.FAMILY_DRIFT, 8, 2, -1, 200),       # four collecting waves
            "drift-16-waves": nat.Tuning(nat.FAMILY_DRIFT, 16, 1, -1, 200)}[kind]
    stream = torch.cuda.current_stream().cuda_stream
    want = oracle.fwd(x.cpu().numpy(), c.cpu().numpy(), False, dtype=np.float64)
    old = lib.linrec_set_spin_limit(1)
    try:
        rc = lib.linrec_fwd_f32(x.data_ptr(), c.data_ptr(), y.data_ptr(), n, L, L, 1, 0, ws.data_ptr(),
                                ws.numel(), ctypes.byref(tune), stream)
        assert rc == 0
        torch.cuda.synchronize()
    finally:
        lib.linrec_set_spin_limit(old)
    hdr = ws[:16].view(torch.int32).cpu().tolist()
    assert hdr[0] == 1, hdr  # the launch completed and advanced the sequence number
    gave_up = hdr[1]
    print(kind, "waits that ran out:", gave_up, flush=True)
    check_close(y, want, "with a poll limit of one")  # whether or not a wait ran out
    # completion counters are back to zero
    assert not ws[16:16 + 1024].any()
    # the same workspace serves the next launch correctly
    y.fill_(float("nan"))
    rc = lib.linrec_fwd_f32(x.data_ptr(), c.data_ptr(), y.data_ptr(), n, L, L, 1, 0, ws.data_ptr(),
                            ws.numel(), ctypes.byref(tune), stream)
    assert rc == 0
    torch.cuda.synchronize()
    check_close(y, want, "after recovery")
    hdr2 = ws[:16].view(torch.int32).cpu().tolist()
    assert hdr2[0] == 2 and hdr2[1] == gave_up, (hdr, hdr2)


def test_workspace_errors(nat):
    dev = torch.device("cuda:0")
    lib = nat.lib()
    x = torch.randn(2, 20000, device=dev)
    y = torch.empty_like(x)
    tune = nat.Tuning(nat.FAMILY_TILE, 4, 4, 1)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.linrec_fwd_f32(x.data_ptr(), x.data_ptr(), y.data_ptr(), 2, 20000, 20000, 1, 0, None, 0,
                              ctypes.byref(tune), s) == -2
    ws = torch.zeros(64, dtype=torch.uint8, device=dev)
    assert lib.linrec_fwd_f32(x.data_ptr(), x.data_ptr(), y.data_ptr(), 2, 20000, 20000, 1, 0, ws.data_ptr(), 64,
                              ctypes.byref(tune), s) == -2
    bad = nat.Tuning(nat.FAMILY_TILE, 3, 5, 0)
    assert lib.linrec_fwd_f32(x.data_ptr(), x.data_ptr(), y.data_ptr(), 2, 100, 20000, 1, 0, None, 0,
                              ctypes.byref(bad), s) == -3
    assert lib.linrec_fwd_f32(None, x.data_ptr(), y.data_ptr(), 2, 100, 20000, 1, 0, None, 0, None, s) == -1


def test_kernel_attrs_report_no_scratch(nat):
    names = nat.kernel_table()
    assert len(names) == nat.lib().linrec_kernel_count()
    for i, name in enumerate(names):
        a = nat.kernel_attrs(i)
        assert a["scratch_bytes"] == 0, (name, a)
        assert 0 < a["num_regs"] <= 256, (name, a)


def _golden_cases():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["name"])
def test_committed_known_answers_on_the_device(nat, case, dtype):
    """The hand-derived integer fixtures, through the HIP kernels: exact in fp32 arithmetic, so the
    results equal the fixture rounded once to the storage type.  Each case is also run embedded in
    a long row of zeros ahead of it, which takes it through the kernels that cut rows into tiles."""
    dev = torch.device("cuda:0")
    t = lambda key: torch.tensor(case[key], dtype=torch.float32)
    x, c = t("x"), t("c")
    rev = case["reverse"]
    for pad in (0, 20000):
        def place(v, fill=0.0):
            if pad == 0:
                return v.to(dtype).to(dev)
            z = torch.full((v.shape[0], pad), fill)
            return (torch.cat([v, z], -1) if rev else torch.cat([z, v], -1)).to(dtype).to(dev)

        def cut(v):
            return v if pad == 0 else (v[:, :x.shape[1]] if rev else v[:, pad:])

        xd, cd = place(x), place(c, 1.0)
        y = nat.fwd(xd, cd, rev)
        assert torch.equal(cut(y).cpu(), t("y").to(dtype)), (case["name"], pad, cut(y))
        if "dy" in case:
            dx, dc = nat.bwd(place(t("dy")), cd, y, rev)
            # the saved outputs were rounded to the storage type; the fixtures stay exact when they fit it
            if torch.equal(t("y").to(dtype).float(), t("y")):
                assert torch.equal(cut(dx).cpu(), t("dx").to(dtype)), (case["name"], pad, cut(dx))
                assert torch.equal(cut(dc).cpu(), t("dc").to(dtype)), (case["name"], pad, cut(dc))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_short_rows_packed_several_to_a_wave(nat, reverse, dtype):
    """Rows of at most 32 slots: 1 to 32 lanes per row, 64 / lanes rows per wave.  Every group size,
    ragged last slots, row counts around a wave's worth, padded rows (padding must stay untouched),
    and more lanes per row than the row needs."""
    dev = torch.device("cuda:0")
    ve = 4 if dtype == torch.float32 else 8
    tol = TOL_NORMWISE if dtype == torch.float32 else 1.05 * 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    for L in [1, 2, ve, ve + 1, 2 * ve, 3 * ve, 4 * ve - 1, 5 * ve, 8 * ve, 9 * ve, 15 * ve + 3, 16 * ve, 17 * ve, 31 * ve + 1, 32 * ve]:
        for numseq in [1, 3, 16, 17, 1000]:
            # rows on slot boundaries, padded by a slot, or packed densely (then they start anywhere in a slot)
            width = [-(-L // ve) * ve, -(-L // ve) * ve + ve, L + 1][(L + numseq) % 3]
            if -(-(L + (0 if width % ve == 0 else ve - 1)) // ve) > 32:
                width = -(-L // ve) * ve
            g = torch.Generator().manual_seed(L * 131 + numseq)
            xw, cw, dyw = (torch.randn(numseq, width, generator=g).to(dtype), (torch.rand(numseq, width, generator=g) * 1.8 - 0.9).to(dtype),
                           torch.randn(numseq, width, generator=g).to(dtype))
            xd, cd, dyd = (t.to(dev)[:, :L] for t in (xw, cw, dyw))
            plan = nat.plan(xd, reverse)
            assert plan["family"] == nat.FAMILY_GROUP, (L, numseq, plan)
            tunings = [None]
            if plan["tasks"] < 32:
                tunings.append(nat.Tuning(nat.FAMILY_GROUP, 0, 0, -1, 32))
            y_t = oracle.fwd(f64(xw[:, :L]), f64(cw[:, :L]), reverse)
            for tun in tunings:
                label = f"L={L} numseq={numseq} width={width} rev={reverse} lanes={plan['tasks'] if tun is None else 32}"
                ybuf = torch.full((numseq, width), float("nan"), dtype=dtype, device=dev)
                y = nat.fwd(xd, cd, reverse, tun, out=ybuf[:, :L])
                dxbuf, dcbuf = (torch.full((numseq, width), float("nan"), dtype=dtype, device=dev) for _ in range(2))
                dx, dc = nat.bwd(dyd, cd, y, reverse, tun, out=(dxbuf[:, :L], dcbuf[:, :L]))
                torch.cuda.synchronize()
                dx_t, dc_t = oracle.bwd(f64(dyw[:, :L]), f64(cw[:, :L]), f64(y), reverse)
                check_close(y.float(), y_t, label + " outputs", tol)
                check_close(dx.float(), dx_t, label + " d_inputs", tol)
                check_close(dc.float(), dc_t, label + " d_coeffs", tol)
                for buf in (ybuf, dxbuf, dcbuf):
                    assert torch.isnan(buf[:, L:]).all(), label + ": wrote into the row padding"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("reverse", [False, True])
def test_dense_short_rows_scanned_as_one_flat_array(nat, reverse, dtype):
    """Dense rows that are not whole 16-byte slots: the flat kernels scan the tensor as one array cut at
    the row starts.  Row lengths from two elements (several rows to a slot) to sixty slots, row counts that leave the
    last slot, the last wave and the look-behind row partly empty, both chunk sizes."""
    dev = torch.device("cuda:0")
    ve = 4 if dtype == torch.float32 else 8
    tol = TOL_NORMWISE if dtype == torch.float32 else 1.05 * 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    F = nat.FAMILY_FLAT
    for L in [2, 3, ve - 1, ve, ve + 1, 2 * ve - 1, 3 * ve + 2, 7 * ve + 3, 16 * ve + 1, 33 * ve - 1, 40 * ve - 1, 60 * ve - 3]:
        for numseq in [2, 3, 17, 257, 1000, 4099]:
            if numseq * L > 600000:
                continue
            g = torch.Generator().manual_seed(L * 977 + numseq)
            x, c, dy = (torch.randn(numseq, L, generator=g).to(dtype), (torch.rand(numseq, L, generator=g) * 1.8 - 0.9).to(dtype),
                        torch.randn(numseq, L, generator=g).to(dtype))
            xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
            default = nat.plan(xd, reverse)["family"]
            assert (default == F) == (L % ve != 0 and L <= 40 * ve), (L, numseq, default)
            y_t = oracle.fwd(f64(x), f64(c), reverse)
            for slots in ((2, 4) if dtype == torch.float32 else (2,)):
                tun = nat.Tuning(F, 0, slots)
                label = f"L={L} numseq={numseq} rev={reverse} rows of slots per wave={slots}"
                y = nat.fwd(xd, cd, reverse, tun, out=torch.full_like(xd, float("nan")))
                dx, dc = nat.bwd(dyd, cd, y, reverse, tun, out=(torch.full_like(xd, float("nan")), torch.full_like(xd, float("nan"))))
                torch.cuda.synchronize()
                dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y), reverse)
                check_close(y, y_t, label + " outputs", tol)
                check_close(dx, dx_t, label + " d_inputs", tol)
                check_close(dc, dc_t, label + " d_coeffs", tol)
    # through the operator and autograd, default plan
    import linrec_amd
    g = torch.Generator().manual_seed(77)
    x, c, dy = (f((12, 50, 30), generator=g).to(dtype).to(dev) for f in (torch.randn, torch.rand, torch.randn))
    assert nat.plan(x, reverse)["family"] == F
    xr, cr = x.clone().requires_grad_(), c.clone().requires_grad_()
    y = linrec_amd.linrec(xr, cr, reverse=reverse)
    y.backward(dy)
    y_t = oracle.fwd(f64(x), f64(c), reverse)
    dx_t, dc_t = oracle.bwd(f64(dy), f64(c), f64(y), reverse)
    check_close(y, y_t, "operator outputs", tol)
    check_close(xr.grad, dx_t, "operator d_inputs", tol)
    check_close(cr.grad, dc_t, "operator d_coeffs", tol)


@pytest.mark.parametrize("reverse", [False, True])
def test_flat_kernels_keep_nonfinite_values_to_their_row(nat, reverse):
    """The cut at a row start is a flag, not a multiplication by zero: a NaN or an infinity in one row,
    or in the coefficient no row uses, leaves every other row bit for bit as it was."""
    dev = torch.device("cuda:0")
    x, c, dy = make_inputs((64, 30), "uniform", seed=9)
    x2, c2, dy2 = x.clone(), c.clone(), dy.clone()
    first = 29 if reverse else 0
    x2[5, 7] = float("nan")
    c2[6, 20] = float("inf")
    x2[20, 29 - first] = float("inf")        # the last element a row's scan reaches
    c2[9, first] = float("nan")              # the coefficient the definition never uses
    dy2[30, 3] = float("nan")
    dy2[31, first] = float("inf")            # the last element the backward scan reaches
    assert nat.plan(x.to(dev), reverse)["family"] == nat.FAMILY_FLAT
    base = nat.fwd(x.to(dev), c.to(dev), reverse)
    got = nat.fwd(x2.to(dev), c2.to(dev), reverse)
    for r in range(64):
        if r not in (5, 6, 20):
            assert torch.equal(got[r], base[r]), r
    assert not torch.isfinite(got[5]).all() and not torch.isfinite(got[6]).all() and not torch.isfinite(got[20]).all()
    before_nan = slice(8, None) if reverse else slice(0, 7)
    assert torch.equal(got[5, before_nan], base[5, before_nan])
    bdx, bdc = nat.bwd(dy.to(dev), c.to(dev), base, reverse)
    gdx, gdc = nat.bwd(dy2.to(dev), c2.to(dev), base, reverse)
    for r in range(64):
        if r not in (6, 30, 31):
            assert torch.equal(gdx[r], bdx[r]) and torch.equal(gdc[r], bdc[r]), r
    assert not torch.isfinite(gdx[30]).all() and not torch.isfinite(gdx[31]).all()


def test_short_rows_keep_nonfinite_values_to_their_row(nat):
    dev = torch.device("cuda:0")
    x, c, _ = make_inputs((64, 32), "uniform", seed=9)
    x2, c2 = x.clone(), c.clone()
    x2[5, 7] = float("nan")
    c2[6, 20] = float("inf")
    base = nat.fwd(x.to(dev), c.to(dev))
    got = nat.fwd(x2.to(dev), c2.to(dev))
    assert nat.plan(x.to(dev))["family"] == nat.FAMILY_GROUP
    for r in range(64):
        if r not in (5, 6):
            assert torch.equal(got[r], base[r]), r
    assert torch.equal(got[5, :7], base[5, :7]) and not torch.isfinite(got[5, 7:]).any()
    assert torch.equal(got[6, :20], base[6, :20]) and not torch.isfinite(got[6, 20:]).all()


@pytest.mark.parametrize("cus", [64, 120])
def test_grids_sized_for_a_smaller_device_give_the_same_results(nat, cus):
    """The planner sizes every launch whose workgroups wait for each other by the compute-unit count it was
    told (here: fewer than the device has, as on a partition of it); teams and grids shrink, the results
    do not change.  Long rows in teams, a single row in one team, time-major data in teams along the scan axis."""
    dev = torch.device("cuda:0")
    lib = nat.lib()
    assert lib.linrec_set_compute_units(-1) == 0  # no override in force
    cases = [((96, 65536), False), ((40, 8192 * 24), False), ((5, 4096 * 130), False), ((1, 4096 * 300), False),
             ((300, 65536 + 4), False), ((1300, 4096), True), ((700, 6000), True)]
    try:
        nat.set_compute_units(cus)  # (also forgets the workspace sizes the binding remembers per layout)
        for shape, transposed in cases:
            x, c, dy = make_inputs(shape, "uniform", seed=shape[0], transposed=transposed)
            xd, cd, dyd = x.to(dev), c.to(dev), dy.to(dev)
            assert xd.stride() == x.stride()
            for reverse in (False, True):
                pf, pb = nat.plan(xd, reverse, False), nat.plan(xd, reverse, True)
                print(cus, shape, reverse, "families", pf["family"], pb["family"], "grids", pf["grid"], pb["grid"], flush=True)
                for p in (pf, pb):
                    if p["workspace_bytes"] > 0 and p["family"] != nat.FAMILY_TILE and p["family"] != nat.FAMILY_SEGMENT:
                        assert p["grid"] <= 2 * cus, p  # (at most two workgroups per compute unit, forward sweeps)
                y = nat.fwd(xd, cd, reverse)
                dx, dc = nat.bwd(dyd, cd, y, reverse)
                torch.cuda.synchronize()
                y_t, _, _ = truth(x, c, dy, reverse)
                dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y.cpu().numpy().astype(np.float64), reverse, dtype=np.float64)
                check_close(y, y_t, f"{cus} CUs {shape} outputs")
                check_close(dx, dx_t, f"{cus} CUs {shape} d_inputs")
                check_close(dc, dc_t, f"{cus} CUs {shape} d_coeffs")
    finally:
        nat.set_compute_units(0)
    assert nat.gave_up_count() == 0
