"""Tensors of more than 2^31 elements: every address beyond the 2^31-th element has to be formed
in 64 bits, in every kernel family.  Inputs are drawn on the device; the float64 recurrence is
checked on a sample of rows (the first, the ones around the 2^31-th element, the last), and the
result buffers are pre-filled with NaN, so an element no lane wrote anywhere in the tensor shows up
in a full-tensor reduction on the device."""
import numpy as np
import pytest
import torch

from tests.util import check_close, truth

pytestmark = pytest.mark.gpu

CASES = {
    # name: (numseq, seqlen, transposed, reverse, dtype, expected family)
    "stream_f32": (90000, 24578, False, False, torch.float32, "STREAM"),       # rows that are not whole slots
    "lookback_f32": (70144, 32778, False, False, torch.float32, "TILE"),       # ... and long enough for look-back tiles
    "drift_ragged_f32": (70144, 32776, False, False, torch.float32, "DRIFT"),  # whole slots, a partial last tile
    "drift_rows_f32": (56000, 40960, False, False, torch.float32, "DRIFT"),  # (its backward: teams that wait, SWEEP)
    "tile_f32": (1100000, 2048, False, True, torch.float32, "TILE"),
    "flat_f32": (72000000, 30, False, True, torch.float32, "FLAT"),
    "column_f32": (4194304, 520, True, False, torch.float32, "COLUMN"),
    "segment_f32": (700, 3100000, True, True, torch.float32, "SEGMENT"),
    "coldrift_f32": (4000, 537000, True, True, torch.float32, "COLDRIFT"),
    "colblock_f32": (16000, 134300, True, True, torch.float32, "COLUMN"),
    "drift_f32": (20, 1 << 27, False, True, torch.float32, "DRIFT"),  # (its backward: teams that wait, SWEEP)
    "team_f32": (18, (1 << 27) + 14, False, False, torch.float32, "TEAM"),
    "stream_bf16": (70000, 32768, False, True, torch.bfloat16, "STREAM"),
}


def _rows_to_check(numseq, row_elems):
    crossing = (1 << 31) // row_elems  # the row that holds element 2^31 of a dense tensor
    picks = {0, 1, crossing - 1, crossing, crossing + 1, numseq - 2, numseq - 1}
    return sorted(r for r in picks if 0 <= r < numseq)


@pytest.mark.parametrize("name", list(CASES))
def test_more_than_two_to_the_31_elements(name):
    from linrec_amd import _native as nat
    numseq, seqlen, transposed, reverse, dtype, family = CASES[name]
    assert numseq * seqlen > (1 << 31)
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(len(name))
    base = (seqlen, numseq) if transposed else (numseq, seqlen)

    def draw(kind):
        t = torch.empty(base, dtype=dtype, device=dev)
        # filled in chunks of the leading dimension to keep the generator's temporaries small
        step = max(1, (1 << 28) // base[1])
        for i in range(0, base[0], step):
            blk = t[i:i + step]
            if kind == "normal":
                blk.copy_(torch.randn(blk.shape, device=dev, generator=g))
            else:
                blk.copy_(torch.rand(blk.shape, device=dev, generator=g))
        return t.t() if transposed else t

    def poisoned():
        t = torch.full(base, float("nan"), dtype=dtype, device=dev)
        return t.t() if transposed else t

    x, c = draw("normal"), draw("uniform")
    plan = nat.plan(x, reverse, False)
    assert plan["family"] == getattr(nat, "FAMILY_" + family), plan
    assert (plan["carry"] >= 1) == name.startswith("colblock") or family not in ("COLUMN", "SEGMENT"), plan
    print(f"{name}: {numseq} x {seqlen}, plan {plan}", flush=True)
    y = nat.fwd(x, c, reverse, out=poisoned())
    torch.cuda.synchronize()
    assert not torch.isnan(y).any().item(), "forward left elements unwritten"
    dy = draw("normal")
    dx, dc = nat.bwd(dy, c, y, reverse, out=(poisoned(), poisoned()))
    torch.cuda.synchronize()
    assert not torch.isnan(dx).any().item() and not torch.isnan(dc).any().item(), "backward left elements unwritten"
    assert nat.gave_up_count() == 0

    rows = _rows_to_check(numseq, seqlen)
    if seqlen > (1 << 24):
        rows = [rows[0], rows[-1]]  # rows this long take the CPU a second each
    idx = torch.tensor(rows, device=dev)
    xs, cs, dys, ys, dxs, dcs = (t.index_select(0, idx).float().cpu() for t in (x, c, dy, y, dx, dc))
    del x, c, dy, y, dx, dc
    torch.cuda.empty_cache()
    # the truth of the backward is taken from the outputs the forward stored (what autograd saves)
    y_t, _, _ = truth(xs, cs, dys, reverse)
    from oracle import oracle
    dx_t, dc_t = oracle.bwd(dys.numpy(), cs.numpy(), ys.numpy().astype(np.float64), reverse, dtype=np.float64)
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -8
    check_close(ys, y_t, f"{name} outputs rows {rows}", tol)
    check_close(dxs, dx_t, f"{name} d_inputs rows {rows}", tol)
    check_close(dcs, dc_t, f"{name} d_coeffs rows {rows}", tol)
