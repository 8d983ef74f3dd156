"""Tuning sweep and kernel-attribute report for the gfx950 kernel table.

Counterpart of the reference's eval/tune.py:58-134 (grid search over compiled configurations with
time, throughput and difference to a reference) and eval/func_attrs.py:25-60 (register / spill
report).  Every compiled geometry that can serve the shape is timed with HIP events on rotating
buffer sets and checked against the library's sequential host loop in float64 on the same values
(max|difference| / max|reference|), as the reference checks every configuration against its
one-thread-per-row kernel (eval/tune.py:98-102).

    python -m linrec_amd.tune --shape 512 65536 [--dtype f32|f16|bf16] [--reverse] [--transposed] [--mixed-phase]
                              [--only TEXT] [--attrs] [--csv out.csv]
    python -m linrec_amd.tune --memory-probe [--shape 512 65536]
    python -m linrec_amd.tune --write-table [PATH]
    python -m linrec_amd.tune --launch-model [--shape 512 65536]

`--only TEXT` keeps the geometries whose label contains TEXT (one kernel under a profiler).
`--write-table` measures the crossovers between the long-row kernels that the launch planner decides by (one
sweep per threshold: the two kernels on either side, timed over a range of the quantity the rule is written in)
and writes them as csrc/plan_thresholds.inc, the file the planner is compiled with - the counterpart of the
dispatch table the reference's grid search writes (eval/tune.py:104-134).  Without PATH the file is printed.
`--launch-model` times the memory-only model of the drift launch the planner makes for the shape (the same persistent
workgroups, teams, tiles and order of accesses, no scan, no exchange), with its stores two steps late and at once
and with one and two tiles of loads ahead, next to the scan kernels themselves and to the streaming kernel of
thousands of small workgroups in address order; and when the model's workgroups, which all do the same work, end.
`--memory-probe` times no scan at all: the memory-only kernel with a pass's mix of streams (2 in and 1 out,
3 in and 2 out) over tensors of the given size, its 16 KiB blocks launched in address order and in orders
that keep some address bits the same among the blocks in flight, which is what a launch with one
workgroup per row does to the bits that number the block inside the row.
"""
import argparse
import csv
import sys

import torch

from . import _native as nat

TILE_GEOMETRIES = [(1, 1), (1, 2), (1, 4), (1, 8), (2, 1), (2, 2), (2, 4), (4, 1), (4, 2), (4, 4), (4, 8),
                   (8, 2), (8, 4), (16, 2), (16, 4)]
CARRY_GEOMETRIES = [(1, 4), (4, 2), (4, 4), (4, 8), (8, 4), (8, 8), (16, 4)]
CHAIN_GEOMETRIES = [(4, 2), (4, 4), (8, 2), (8, 4)]
STREAM_GEOMETRIES = [(4, 4), (8, 2), (8, 4), (16, 2), (8, 8)]
TEAM_GEOMETRIES = [(4, 2), (4, 4), (8, 2), (8, 4)]
SWEEP_GEOMETRIES = [(4, 4), (8, 2), (8, 4), (8, 8)]
DRIFT_GEOMETRIES = [(8, 4), (8, 2), (4, 4), (16, 2), (16, 1), (8, 1)]  # the fp32 backward is compiled for tiles of 4096 elements (8 x 2, 16 x 1); 16-bit storage: 16 x 1 in both passes, 16 x 2 and 8 x 1 forward; rows that end in a partial tile: fp32 16 x 2 and 8 x 4 forward, 16 x 1 backward, 16-bit 16 x 2 forward, 8 x 2 backward


def candidates(t):
    """(label, Tuning or None) for every compiled kernel that accepts tensor `t`."""
    out = [("table default", None)]
    lay = nat.row_layout(t)
    if lay is None:
        return out
    _, L, _, es = lay
    if es == 1 or L == 1:
        for lanes in (1, 2, 4, 8, 16, 32):
            out.append((f"group x{lanes}", nat.Tuning(nat.FAMILY_GROUP, 0, 0, -1, lanes)))
        for rows in (2, 4):
            out.append((f"flat s{rows}", nat.Tuning(nat.FAMILY_FLAT, 0, rows)))
        for w, s in TILE_GEOMETRIES:
            out.append((f"tile w{w} s{s}", nat.Tuning(nat.FAMILY_TILE, w, s, 0)))
        for w, s in CARRY_GEOMETRIES:
            out.append((f"tile w{w} s{s} look-back", nat.Tuning(nat.FAMILY_TILE, w, s, 1, 1)))
        for w, s in CHAIN_GEOMETRIES:
            for tasks in (4, 16):
                out.append((f"chain w{w} s{s} x{tasks}", nat.Tuning(nat.FAMILY_TILE, w, s, 1, tasks)))
        for w, s in STREAM_GEOMETRIES:
            out.append((f"stream w{w} s{s}", nat.Tuning(nat.FAMILY_STREAM, w, s)))
        for w, s in TEAM_GEOMETRIES:
            for team in (2, 4, 8):
                out.append((f"team w{w} s{s} x{team}", nat.Tuning(nat.FAMILY_TEAM, w, s, -1, team)))
        for w, s in SWEEP_GEOMETRIES:
            out.append((f"sweep w{w} s{s}", nat.Tuning(nat.FAMILY_SWEEP, w, s)))
        for w, s in DRIFT_GEOMETRIES:
            out.append((f"drift w{w} s{s}", nat.Tuning(nat.FAMILY_DRIFT, w, s)))  # the planner's team size
            for team in (16, 64, 128, 256):
                out.append((f"drift w{w} s{s} x{team}", nat.Tuning(nat.FAMILY_DRIFT, w, s, -1, team)))
    else:
        # strided scan axis: rows per lane (access width) x timesteps per batch
        for width in (1, 2, 4, 8):
            fam = nat.FAMILY_COLUMN if width > 1 else nat.FAMILY_NAIVE
            for depth in (4, 8, 16):
                out.append((f"column rows {width} depth {depth}", nat.Tuning(fam, width, depth)))
        # block form: the waves of a workgroup share rows; rows per lane x lane groups per wave
        for width in (1, 2):
            for groups in (1, 2):
                out.append((f"column block rows {width} groups {groups}", nat.Tuning(nat.FAMILY_COLUMN, width, 0, groups)))
        # column blocks in teams along the scan axis: waves per workgroup, positions per run, rows per lane, team size
        for w, run, width in ((16, 8, 1), (16, 4, 1), (8, 16, 1), (16, 8, 2), (16, 4, 2), (8, 16, 2)):  # (two rows per lane: 16-bit storage)
            out.append((f"column drift w{w} run {run} rows {width}", nat.Tuning(nat.FAMILY_COLDRIFT, w, run, width)))
            for team in (2, 4, 8, 16):
                out.append((f"column drift w{w} run {run} rows {width} x{team}", nat.Tuning(nat.FAMILY_COLDRIFT, w, run, width, team)))
        # the scan axis cut into segments: rows per lane x segments
        for width in (1, 2, 4):
            for segments in (8, 32, 128, 512):
                out.append((f"segment rows {width} x{segments}", nat.Tuning(nat.FAMILY_SEGMENT, width, 8, -1, segments)))
    return out


def _event_ms(fn, iters, warmup):
    for i in range(warmup):
        fn(i)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for i in range(iters):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def sequential_reference(x, c, dy, reverse):
    """outputs, d_inputs, d_coeffs of the library's sequential host loop (linrec_host_fwd_f64 / _bwd_f64) in
    float64 on the values of the device tensors x, c, dy: float64 CPU tensors."""
    xh, ch, dyh = (t.detach().to("cpu", torch.float64) for t in (x, c, dy))
    y = nat.fwd(xh, ch, reverse)
    dx, dc = nat.bwd(dyh, ch, y, reverse)
    return y, dx, dc


def normwise_error(got, want64):
    """max|got - want| / max|want| in float64 (the figure the parity tests are written in)."""
    scale = want64.abs().max().item()
    return (got.double() - want64).abs().max().item() / (scale if scale > 0 else 1.0)


def sweep(shape, reverse=False, transposed=False, sets=3, iters=50, warmup=10, device="cuda:0", dtype=torch.float32,
          mixed_phase=False, only=None):
    """List of dict rows: one per candidate geometry, forward and backward time and GB/s (a pass a
    geometry is not compiled for is left out of its row).
    `mixed_phase`: the coefficients start one element off the other tensors' 16-byte phase, which
    forces element-sized accesses (the price of the wide accesses, measured)."""
    dev = torch.device(device)
    n = shape[0] * shape[1]
    es = torch.empty((), dtype=dtype).element_size()
    bufs = []
    for _ in range(sets):
        if transposed:
            x, c, dy = (f(shape[1], shape[0], device=dev).to(dtype).t() for f in (torch.randn, torch.rand, torch.randn))
        else:
            x, c, dy = (f(shape, device=dev).to(dtype) for f in (torch.randn, torch.rand, torch.randn))
        if mixed_phase and not transposed:
            buf = torch.empty(n + 8, dtype=dtype, device=dev)
            c = buf[1:1 + n].view(shape).copy_(c)
        y, dx, dc = (torch.empty_strided(x.size(), x.stride(), dtype=dtype, device=dev) for _ in range(3))
        bufs.append((x, c, dy, y, dx, dc))
    # Every candidate is checked against the library's sequential host loop in float64 on the same values (the
    # role of the one-thread-per-row kernel in the reference's grid search, eval/tune.py:98-102): a float64
    # recurrence that shares no code with the device kernels.
    ref_y, ref_dx, ref_dc = (t.to(dev) for t in sequential_reference(bufs[0][0], bufs[0][1], bufs[0][2], reverse))
    saved_y = ref_y.to(dtype)  # the saved outputs the backward passes run on
    for b in bufs:
        b[3].copy_(nat.fwd(b[0], b[1], reverse))
    names = nat.kernel_table()
    rows = []
    for label, tun in candidates(bufs[0][0]):
        if only is not None and only not in label:
            continue
        row = {"geometry": label}
        try:
            pl = nat.plan(bufs[0][0], reverse, False, tun)
            if tun is not None and pl["family"] != tun.family:
                raise NotImplementedError
            y = nat.fwd(bufs[0][0], bufs[0][1], reverse, tun)
            diff = normwise_error(y, ref_y)
            f = _event_ms(lambda i: nat.fwd(bufs[i % sets][0], bufs[i % sets][1], reverse, tun, out=bufs[i % sets][4]),
                          iters, warmup)
            row.update(kernel=names[pl["kernel_id"]], grid=pl["grid"], team=pl["tasks"], fwd_us=f * 1e3,
                       fwd_GBps=3 * es * n / f / 1e6, fwd_err_vs_sequential=diff)
        except (RuntimeError, NotImplementedError):
            row.update(kernel="-", grid=0, team=0, fwd_us=float("nan"), fwd_GBps=float("nan"), fwd_err_vs_sequential=float("nan"))
        try:
            pl = nat.plan(bufs[0][0], reverse, True, tun)
            if tun is not None and pl["family"] != tun.family:
                raise NotImplementedError
            dx, dc = nat.bwd(bufs[0][2], bufs[0][1], saved_y, reverse, tun)
            diff = max(normwise_error(dx, ref_dx), normwise_error(dc, ref_dc))
            b = _event_ms(lambda i: nat.bwd(bufs[i % sets][2], bufs[i % sets][1], bufs[i % sets][3], reverse, tun,
                                            out=(bufs[i % sets][4], bufs[i % sets][5])), iters, warmup)
            row.update(bwd_kernel=names[pl["kernel_id"]], bwd_team=pl["tasks"], bwd_us=b * 1e3, bwd_GBps=5 * es * n / b / 1e6,
                       bwd_err_vs_sequential=diff)
        except (RuntimeError, NotImplementedError):
            row.update(bwd_kernel="-", bwd_team=0, bwd_us=float("nan"), bwd_GBps=float("nan"), bwd_err_vs_sequential=float("nan"))
        if row["kernel"] != "-" or row["bwd_kernel"] != "-":
            rows.append(row)
    return rows


def memory_probe(shape, sets=3, iters=40, warmup=8, device="cuda:0"):
    """Rows of dicts: GB/s of the memory-only kernel for the forward's and the backward's mix of streams
    over tensors of shape[0] * shape[1] floats (a power of two), blocks launched in address order and with
    address bits held among the blocks in flight."""
    dev = torch.device(device)
    n = shape[0] * shape[1]
    assert n % 4096 == 0 and (n // 4096) & (n // 4096 - 1) == 0, "a power of two of 16 KiB blocks"
    index_bits = (n // 4096).bit_length() - 1
    srcs = [[torch.randn(n, device=dev) for _ in range(3)] for _ in range(sets)]
    dsts = [[torch.empty(n, device=dev) for _ in range(2)] for _ in range(sets)]
    row_bits = (shape[1] * 4).bit_length() - 1  # one workgroup per row holds address bits 14 .. row_bits - 1
    cases = [("address order", (0, 0))]
    if 14 < row_bits <= 14 + index_bits:
        cases.append((f"bits 14-{row_bits - 1} held (one workgroup per row of {shape[1]} floats)", (0, row_bits - 14)))
    for lo, bits in [(1, 3), (1, 1), (2, 1), (3, 1), (4, 1), (5, 1), (6, 1), (7, 1), (8, 1), (9, 1), (3, 4), (6, 3), (8, 3)]:
        if lo + bits <= index_bits:
            cases.append((f"bits {14 + lo}-{14 + lo + bits - 1} held" if bits > 1 else f"bit {14 + lo} held", (lo, bits)))
    rows = []
    for label, hold in cases:
        f = _event_ms(lambda i: nat.stream_mix(srcs[i % sets][:2], dsts[i % sets][:1], hold), iters, warmup)
        b = _event_ms(lambda i: nat.stream_mix(srcs[i % sets], dsts[i % sets], hold), iters, warmup)
        rows.append({"blocks in flight": label, "2_in_1_out_us": f * 1e3, "2_in_1_out_GBps": 12 * n / f / 1e6,
                     "3_in_2_out_us": b * 1e3, "3_in_2_out_GBps": 20 * n / b / 1e6})
    return rows



def launch_model(shape, sets=3, iters=40, warmup=8, device="cuda:0"):
    """Rows of dicts for fp32 tensors of `shape` whose planned launches are drift launches: per pass the scan kernel,
    the memory-only model of its launch (variants of how far ahead it loads and how late it stores) and the streaming
    kernel with the pass's mix of streams; for the model also when its workgroups end (us after the first start)."""
    dev = torch.device(device)
    n = shape[0] * shape[1]
    srcs = [[torch.randn(shape, device=dev) for _ in range(3)] for _ in range(sets)]
    dsts = [[torch.empty(shape, device=dev) for _ in range(2)] for _ in range(sets)]
    for k in range(sets):
        srcs[k][1].uniform_()  # coefficients in [0, 1)
    names = nat.kernel_table()
    rows = []
    for is_bwd, nin, nout, bpe in ((False, 2, 1, 12), (True, 3, 2, 20)):
        what = "backward" if is_bwd else "forward"
        pl = nat.plan(srcs[0][0], False, is_bwd)
        if pl["family"] != nat.FAMILY_DRIFT:
            raise SystemExit(f"the planner's {what} launch for {shape} is not a drift launch ({names[pl['kernel_id']]})")
        waves, slots, team = pl["waves"], pl["slots"], pl["tasks"]
        grid = pl["grid"]
        if is_bwd:
            y = [nat.fwd(srcs[k][0], srcs[k][1]) for k in range(sets)]
            t = _event_ms(lambda i: nat.bwd(srcs[i % sets][2], srcs[i % sets][1], y[i % sets], False,
                                            out=(dsts[i % sets][0], dsts[i % sets][1])), iters, warmup)
        else:
            t = _event_ms(lambda i: nat.fwd(srcs[i % sets][0], srcs[i % sets][1], False, out=dsts[i % sets][0]), iters, warmup)

        def row(label, ms, ends=None):
            r = {"pass": what, "launch": label, "us": ms * 1e3, "GBps": bpe * n / ms / 1e6, "pct_of_8_TBps": round(bpe * n / ms / 1e6 / 80, 1)}
            r.update({"first_end_us": float("nan"), "mean_end_us": float("nan"), "last_end_us": float("nan")} if ends is None else ends)
            rows.append(r)

        row(f"scan kernel {names[pl['kernel_id']]}, {grid} workgroups in teams of {team}", t)
        kernel_ahead = 2 if (is_bwd and waves == 16 and slots == 1) else 1
        variants = [(kernel_ahead, 2, "as the kernel"), (kernel_ahead, 0, "stores at once"), (3 - kernel_ahead, 2, "")]
        for ahead, late, note in variants:
            try:
                nat.launch_model(srcs[0][:nin], dsts[0][:nout], shape, waves, slots, team, ahead, late)
            except NotImplementedError:
                continue
            t = _event_ms(lambda i: nat.launch_model(srcs[i % sets][:nin], dsts[i % sets][:nout], shape, waves, slots, team, ahead, late),
                          iters, warmup)
            stamps = torch.zeros(2 * grid, dtype=torch.int64, device=dev)
            nat.launch_model(srcs[0][:nin], dsts[0][:nout], shape, waves, slots, team, ahead, late, stamps)
            st = stamps.view(grid, 2).cpu().double() * 0.01  # 100 MHz clock -> us
            ends = st[:, 1] - st[:, 0].min()
            row(f"memory-only model w{waves} s{slots} teams of {team}, {ahead} tile{'s' * (ahead > 1)} ahead, stores {late} steps late"
                + (f" ({note})" if note else ""), t,
                {"first_end_us": ends.min().item(), "mean_end_us": ends.mean().item(), "last_end_us": ends.max().item()})
        t = _event_ms(lambda i: nat.stream_mix([a.view(-1) for a in srcs[i % sets][:nin]], [a.view(-1) for a in dsts[i % sets][:nout]]),
                      iters, warmup)
        row(f"streaming kernel, {n // 4096} workgroups of 4096 floats in address order", t)
    return rows


# ---- the planner's crossover thresholds ------------------------------------------------------------
class Crossover:
    """One threshold of the planner: `name` in csrc/plan_thresholds.inc, the swept `values` of the quantity the
    rule is written in, `shape(v)` -> (rows, length) of the problem timed at v, the tunings on either side
    ({pass: Tuning}; `low` serves the small values - the fastest of a list, where the planner has several kernels to
    fall back on - and `high` the large ones) and the passes whose times are added.
    kind 'first_high': the threshold is the smallest value from which `high` is faster on all larger values
    tried; 'last_low': the largest value up to which `low` is at least as fast on all smaller values tried."""

    def __init__(self, name, what, values, shape, low, high, passes=("fwd", "bwd"), kind="first_high", dtype=torch.float32):
        self.name, self.what, self.values, self.shape = name, what, values, shape
        self.low, self.high, self.passes, self.kind, self.dtype = low, high, passes, kind, dtype


def _t(family, waves=0, slots=0, carry=-1, tasks=0):
    return nat.Tuning(family, waves, slots, carry, tasks)


def _both(t):
    return {"fwd": t, "bwd": t}


_DRIFT = {"fwd": _t(nat.FAMILY_DRIFT, 16, 2), "bwd": _t(nat.FAMILY_DRIFT, 16, 1)}
_DRIFT_SMALL = {"fwd": _t(nat.FAMILY_DRIFT, 16, 1), "bwd": _t(nat.FAMILY_DRIFT, 16, 1)}

CROSSOVERS = [
    Crossover("stream_min_rows", "long rows that are not whole slots (65542 elements): one team of workgroups per row "
              "against one workgroup per row, by the number of rows", [64, 96, 112, 128, 129, 144, 160, 192],
              lambda v: (v, 65542), _both(_t(nat.FAMILY_TEAM)), _both(_t(nat.FAMILY_STREAM))),
    Crossover("stream_max_len", "600 long rows that are not whole slots: one workgroup per row against look-back tiles of "
              "16384 elements, by the row length", [16386, 20002, 24578, 28002, 32770, 40002, 49154, 65542],
              lambda v: (600, v), _both(_t(nat.FAMILY_STREAM)), _both(_t(nat.FAMILY_TILE, 8, 8, 1, 1))),
    Crossover("team_min_rows", "a few very long rows that are not whole slots (1048582 elements): look-back tiles against "
              "one team of 64 workgroups per row, by the number of rows", [2, 3, 4, 5, 6, 8, 12],
              lambda v: (v, 1048582), _both(_t(nat.FAMILY_TILE, 8, 8, 1, 1)), _both(_t(nat.FAMILY_TEAM))),
    Crossover("drift_bwd_max_rows", "backward of many rows of 32768 elements: drift teams (tiles stored two steps "
              "late) against sweep teams (tiles of 8192 elements, exchange waited for), by the number of rows",
              [1024, 1536, 2048, 3072, 4096], lambda v: (v, 32768), _DRIFT_SMALL, _both(_t(nat.FAMILY_SWEEP, 8, 4)),
              passes=("bwd",), kind="last_low"),
    Crossover("drift_bwd_few_rows_min_tiles_per_cu", "backward of 32 long rows: sweep teams with tiles of 16384 "
              "elements against drift teams, by the tiles of 8192 elements per compute unit",
              [2, 3, 4, 6, 8, 12, 16], lambda v: (32, v * 65536), _both(_t(nat.FAMILY_SWEEP, 8, 8)), _DRIFT_SMALL,
              passes=("bwd",)),
    Crossover("little_work_max_tiles_per_cu", "128 rows with little work: sweep teams with tiles of 16384 elements "
              "against drift teams, by the tiles of 8192 elements per compute unit", [2, 4, 6, 8, 12],
              lambda v: (128, v * 16384), _both(_t(nat.FAMILY_SWEEP, 8, 8)), _DRIFT, kind="last_low"),
    Crossover("drift_min_small_tiles_per_row", "forward of 600 rows that are whole tiles of 4096 elements but not of "
              "8192: one workgroup per row, or sweep teams, against drift teams, by the tiles of a row", [5, 7, 9, 11, 13, 15, 17],
              lambda v: (600, v * 4096), [_both(_t(nat.FAMILY_STREAM)), _both(_t(nat.FAMILY_SWEEP, 8, 2))], _DRIFT_SMALL,
              passes=("fwd",)),
    Crossover("drift_bwd_short_rows_min_rows", "backward of rows of four tiles of 4096 elements: one workgroup per "
              "row against drift teams, by the number of rows", [128, 256, 384, 512, 768, 1024, 2048],
              lambda v: (v, 16384), _both(_t(nat.FAMILY_STREAM)), _DRIFT_SMALL, passes=("bwd",)),
    Crossover("drift_fwd_min_tiles_per_row", "forward of 600 rows of whole tiles of 8192 elements: one workgroup per "
              "row, or sweep teams, against drift teams, by the tiles of a row", [2, 3, 4, 5, 6],
              lambda v: (600, v * 8192), [_both(_t(nat.FAMILY_STREAM)), _both(_t(nat.FAMILY_SWEEP, 8, 4))], _DRIFT,
              passes=("fwd",)),
    Crossover("drift_fwd_two_tiles_min_rows", "forward of rows of two tiles of 8192 elements: one workgroup per row, or "
              "sweep teams, against drift teams of two, by the number of rows", [512, 768, 1024, 1536, 2048, 3072, 4096],
              lambda v: (v, 16384), [_both(_t(nat.FAMILY_STREAM)), _both(_t(nat.FAMILY_SWEEP, 8, 2))], _DRIFT,
              passes=("fwd",)),
    # 16-bit storage (measured on bf16; fp16 moves the same bytes)
    Crossover("half_team_fwd_min_rows", "bf16 forward of a few ragged very long rows (1048584 elements): look-back tiles "
              "against one team of 64 workgroups per row, by the number of rows", [2, 3, 4, 6, 8, 16, 32],
              lambda v: (v, 1048584), _both(_t(nat.FAMILY_TILE, 8, 4, 1, 1)), _both(_t(nat.FAMILY_TEAM)), passes=("fwd",),
              dtype=torch.bfloat16),
    Crossover("half_team_bwd_min_rows", "bf16 backward of a few ragged very long rows (1048584 elements): look-back tiles "
              "against one team of 64 workgroups per row, by the number of rows", [2, 3, 4, 6, 8, 16, 32],
              lambda v: (v, 1048584), _both(_t(nat.FAMILY_TILE, 8, 4, 1, 1)), _both(_t(nat.FAMILY_TEAM)), passes=("bwd",),
              dtype=torch.bfloat16),
    Crossover("half_drift_fwd_small_tiles_max_rows", "bf16 forward of rows that are whole tiles of 8192 elements but not "
              "of 16384 (nine tiles): drift teams against one workgroup per row, or sweep teams, by the number of rows",
              [64, 96, 112, 127, 144, 160, 200, 256], lambda v: (v, 8192 * 9), _DRIFT_SMALL,
              [_both(_t(nat.FAMILY_STREAM)), _both(_t(nat.FAMILY_SWEEP, 8, 2))], passes=("fwd",), kind="last_low", dtype=torch.bfloat16),
    Crossover("half_drift_fwd_min_tiles_per_cu", "bf16 forward of 16 long rows: look-back tiles, one team per row or sweep "
              "teams against drift teams with tiles of 16384 elements, by the tiles per compute unit",
              [1, 2, 3, 4, 6, 8], lambda v: (16, v * 262144),
              [_both(_t(nat.FAMILY_TILE)), _both(_t(nat.FAMILY_TEAM)), _both(_t(nat.FAMILY_SWEEP, 8, 2))],
              _both(_t(nat.FAMILY_DRIFT, 16, 2)), passes=("fwd",), dtype=torch.bfloat16),
    Crossover("half_drift_bwd_min_tiles_per_cu", "bf16 backward of 16 long rows: look-back tiles, one team per row or sweep "
              "teams against drift teams with tiles of 8192 elements, by the tiles per compute unit",
              [1, 2, 3, 4, 6, 8], lambda v: (16, v * 131072),
              [_both(_t(nat.FAMILY_TILE)), _both(_t(nat.FAMILY_TEAM)), _both(_t(nat.FAMILY_SWEEP, 8, 2))],
              _DRIFT_SMALL, passes=("bwd",), dtype=torch.bfloat16),
]


def _time_tunings(shape, tunings, passes, sets=3, iters=30, warmup=6, device="cuda:0", rounds=2, dtype=torch.float32):
    """Microseconds of the listed passes added up, for each {pass: Tuning} of `tunings` on tensors of `shape`
    (the candidates take turns, the least of `rounds` counts); inf where the library has no such kernel."""
    dev = torch.device(device)
    bufs = []
    for _ in range(sets):
        x, c, dy = (f(shape, device=dev).to(dtype) for f in (torch.randn, torch.rand, torch.randn))
        y = nat.fwd(x, c)
        bufs.append((x, c, dy, y, torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)))
    best = [float("inf")] * len(tunings)
    for _ in range(rounds):
        for k, tun in enumerate(tunings):
            total = 0.0
            try:
                for p in passes:
                    pl = nat.plan(bufs[0][0], False, p == "bwd", tun[p])
                    if pl["family"] != tun[p].family:
                        raise NotImplementedError
                    if p == "fwd":
                        total += _event_ms(lambda i: nat.fwd(bufs[i % sets][0], bufs[i % sets][1], False, tun[p], out=bufs[i % sets][4]),
                                           iters, warmup) * 1e3
                    else:
                        total += _event_ms(lambda i: nat.bwd(bufs[i % sets][2], bufs[i % sets][1], bufs[i % sets][3], False, tun[p],
                                                             out=(bufs[i % sets][5], bufs[i % sets][6])), iters, warmup) * 1e3
            except (RuntimeError, NotImplementedError):
                total = float("inf")
            best[k] = min(best[k], total)
    return best


STICKY = 0.03  # a threshold only moves past values where one side is more than this fraction faster


def measure_crossover(x, log=None, current=None):
    """(threshold, [(value, shape, us_low, us_high)]) of one Crossover on the current device.
    `current`: the value in force.  Where two kernels' curves cross at a shallow angle the crossing moves with the box
    and the run; the value in force is kept unless some value tried between it and the newly measured crossing
    shows one side more than STICKY faster (either choice costs less than that in between)."""
    rows = []
    for v in x.values:
        lows = x.low if isinstance(x.low, list) else [x.low]
        highs = x.high if isinstance(x.high, list) else [x.high]
        times = _time_tunings(x.shape(v), lows + highs, x.passes, dtype=x.dtype)
        lo, hi = min(times[:len(lows)]), min(times[len(lows):])
        rows.append((v, x.shape(v), lo, hi))
        if log:
            log(f"{x.name}: {v} {x.shape(v)} low {lo:.1f} us high {hi:.1f} us")
    high_wins = [hi < lo for _, _, lo, hi in rows]
    if x.kind == "first_high":
        k = len(rows)
        while k > 0 and high_wins[k - 1]:
            k -= 1
        # (never faster: one past the largest value tried)
        threshold = rows[k][0] if k < len(rows) else rows[-1][0] + 1
    else:
        k = 0
        while k < len(rows) and not high_wins[k]:
            k += 1
        # (never at least as fast: one below the smallest value tried)
        threshold = rows[k - 1][0] if k > 0 else rows[0][0] - 1
    if current is not None and current != threshold:
        # values whose choice differs between the two thresholds
        if x.kind == "first_high":
            between = [(lo, hi) for v, _, lo, hi in rows if min(current, threshold) <= v < max(current, threshold)]
        else:
            between = [(lo, hi) for v, _, lo, hi in rows if min(current, threshold) < v <= max(current, threshold)]
        if all(abs(lo - hi) <= STICKY * min(lo, hi) for lo, hi in between):
            if log:
                log(f"{x.name}: measured {threshold}, within {STICKY:.0%} of the value in force everywhere in between: {current} kept")
            threshold = current
    return threshold, rows


TABLE_HEADER = """// Crossover thresholds of the launch planner for long rows on the unit-stride axis (fp32; the half_* ones for 16-bit
// storage), on the full part (256 compute units; the planner scales row counts to the device in hand).
//
// GENERATED by `python -m linrec_amd.tune --write-table` (the counterpart of the table the reference's grid search
// writes, eval/tune.py:104-134): every line is the smallest value of the swept quantity from which the second
// kernel was faster than the first on all larger values tried (or the largest up to which the first held its own);
// the timings behind each line stand above it.  A value in force is kept where every value tried between it and the
// new crossing has the two kernels within 3 % of each other (shallow crossings move with the box and the run).
// Edit by re-running the command on the device, not by hand.
//
// LINREC_THRESHOLD(name, value)
"""


def write_table(path=None, only=None, log=None):
    """Measures every Crossover and returns the text of csrc/plan_thresholds.inc (written to `path` if given).
    `only`: names to measure; the others keep the values the library is compiled with."""
    current = nat.plan_thresholds()
    device = torch.cuda.get_device_name(0)
    out = [TABLE_HEADER.rstrip("\n"), f"// measured on: {device}, {nat.lib().linrec_compute_units()} compute units"]
    for x in CROSSOVERS:
        out.append("//")
        out.append(f"// {x.name}: {x.what}")
        if only is not None and x.name not in only:
            out.append("// (not measured in this run: value kept)")
            out.append(f"LINREC_THRESHOLD({x.name}, {current[x.name]})")
            continue
        threshold, rows = measure_crossover(x, log, current.get(x.name))
        passes = " + ".join(x.passes)
        for v, shape, lo, hi in rows:
            out.append(f"//   {v:>6}  {shape[0]} x {shape[1]}: {passes} {lo:.1f} us against {hi:.1f} us")
        out.append(f"LINREC_THRESHOLD({x.name}, {threshold})")
    missing = set(current) - {x.name for x in CROSSOVERS}
    assert not missing, f"thresholds without a sweep: {missing}"
    text = "\n".join(out) + "\n"
    if path:
        with open(path, "w") as f:
            f.write(text)
    return text


def attrs_report():
    """numRegs / LDS / scratch of every compiled kernel (hipFuncGetAttributes)."""
    return [dict(kernel=name, **nat.kernel_attrs(i)) for i, name in enumerate(nat.kernel_table())]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--shape", type=int, nargs=2, default=[512, 65536], metavar=("NUMSEQ", "SEQLEN"))
    ap.add_argument("--dtype", choices=list(DTYPES), default="f32", help="storage type (arithmetic is fp32)")
    ap.add_argument("--reverse", action="store_true")
    ap.add_argument("--transposed", action="store_true", help="inputs are transposed views (strided scan axis)")
    ap.add_argument("--mixed-phase", action="store_true",
                    help="offset the coefficients by one element: element-sized instead of 16-byte accesses")
    ap.add_argument("--only", default=None, metavar="TEXT", help="only the geometries whose label contains TEXT")
    ap.add_argument("--memory-probe", action="store_true",
                    help="time the memory-only kernel with address bits held among the blocks in flight instead")
    ap.add_argument("--launch-model", action="store_true",
                    help="time the memory-only model of the shape's drift launches next to the scan kernels instead")
    ap.add_argument("--attrs", action="store_true", help="print the register / LDS / scratch table instead")
    ap.add_argument("--write-table", nargs="?", const="-", default=None, metavar="PATH",
                    help="measure the planner's crossover thresholds and write csrc/plan_thresholds.inc (to PATH, or print it)")
    ap.add_argument("--thresholds", nargs="*", default=None, metavar="NAME", help="with --write-table: only these thresholds")
    ap.add_argument("--csv", default=None)
    a = ap.parse_args(argv)
    if a.write_table is not None:
        text = write_table(None if a.write_table == "-" else a.write_table, a.thresholds,
                           log=lambda m: print(m, file=sys.stderr, flush=True))
        if a.write_table == "-":
            print(text, end="")
        return
    if a.attrs:
        rows = attrs_report()
    elif a.memory_probe:
        rows = memory_probe(tuple(a.shape))
    elif a.launch_model:
        rows = launch_model(tuple(a.shape))
    else:
        rows = sweep(tuple(a.shape), a.reverse, a.transposed, dtype=DTYPES[a.dtype], mixed_phase=a.mixed_phase, only=a.only)
    if not rows:
        sys.exit("nothing to report")
    cols = list(rows[0])
    width = {c: max(len(c), max(len(f"{r[c]:.1f}" if isinstance(r[c], float) else str(r[c])) for r in rows)) for c in cols}
    print("  ".join(f"{c:>{width[c]}s}" for c in cols))
    for r in rows:
        print("  ".join(f"{r[c]:{width[c]}.1f}" if isinstance(r[c], float) else f"{str(r[c]):>{width[c]}s}" for c in cols), flush=True)
    if a.csv:
        with open(a.csv, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=cols)
            w.writeheader()
            w.writerows(rows)


if __name__ == "__main__":
    main()
