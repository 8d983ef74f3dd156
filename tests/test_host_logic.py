"""CPU-only tests: the C ABI library loads and exports every symbol its header declares, the launch
planner (pure host code) picks sensible kernels, the tensor-layout canonicalisation is right, and
the operator plumbing (custom ops, fake functions, autograd rule, errors) behaves like the
reference's (linrec/impl/cuda/ops.py:17-39,85-101).  The host path of the library is exercised on
CPU tensors; no GPU kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import linrec_amd
from linrec_amd import _native as nat
from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "linrec_hip.h")).read()
    declared = set(re.findall(r"^\s*(?:int|int64_t|size_t|const char\*|void)\s+(linrec_\w+)\s*\(", header, flags=re.M))
    assert len(declared) == 37, declared
    lib = ctypes.CDLL(nat.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/linrec_hip.h but not exported"
    assert declared == set(nat.EXPORTS), (declared ^ set(nat.EXPORTS))
    assert lib.linrec_hip_abi_version() == 1


def test_planner_thresholds_come_from_the_generated_table():
    """csrc/plan_thresholds.inc (written by `python -m linrec_amd.tune --write-table`) is what the library is compiled
    with, every threshold in it has a sweep in the harness that can measure it again, and the file carries the
    timings it was derived from."""
    from linrec_amd import tune
    text = open(os.path.join(ROOT, "linrec_amd", "csrc", "plan_thresholds.inc")).read()
    in_file = {m.group(1): int(m.group(2)) for m in re.finditer(r"^LINREC_THRESHOLD\((\w+), (-?\d+)\)", text, flags=re.M)}
    assert in_file == nat.plan_thresholds() and len(in_file) >= 7
    assert {x.name for x in tune.CROSSOVERS} == set(in_file)
    assert text.startswith(tune.TABLE_HEADER) and "measured on:" in text
    for x in tune.CROSSOVERS:  # (the lines of timings above each value)
        block = text[text.index(f"// {x.name}:"):text.index(f"LINREC_THRESHOLD({x.name},")]
        assert block.count(" us against ") == len(x.values), x.name


def test_table_writer_keeps_a_value_in_force_across_a_shallow_crossing(monkeypatch):
    """The threshold writer on timings given by hand: the crossing is found from the measured curves, and a value in
    force is kept unless some value between it and the new crossing shows one kernel more than 3 % faster."""
    from linrec_amd import tune
    curves = {}
    monkeypatch.setattr(tune, "_time_tunings", lambda shape, tunings, passes, **kw: list(curves[shape[0]]))
    mk = lambda kind: tune.Crossover("t", "test", [2, 4, 6, 8], lambda v: (v, 1024), {"fwd": None}, {"fwd": None},
                                     passes=("fwd",), kind=kind)
    # (low, high) per value: high takes over from 6 on, 2 % ahead at 4
    curves.update({2: (10.0, 11.0), 4: (20.0, 19.6), 6: (30.0, 25.0), 8: (40.0, 33.0)})
    assert tune.measure_crossover(mk("first_high"))[0] == 4          # smallest value from which high wins
    assert tune.measure_crossover(mk("last_low"))[0] == 2            # largest value up to which low holds
    assert tune.measure_crossover(mk("first_high"), current=6)[0] == 6   # 4 is within 3 %: the value in force stays
    assert tune.measure_crossover(mk("first_high"), current=8)[0] == 4   # 6 is 17 % apart: it moves
    assert tune.measure_crossover(mk("last_low"), current=4)[0] == 4     # (last_low 4 means: low up to 4; 4 is within 3 %)
    assert tune.measure_crossover(mk("last_low"), current=6)[0] == 2     # low at 6 costs 20 %
    # never faster / always faster: one past the ends
    curves.update({v: (1.0, 2.0) for v in (2, 4, 6, 8)})
    assert tune.measure_crossover(mk("first_high"))[0] == 9 and tune.measure_crossover(mk("last_low"))[0] == 8
    curves.update({v: (2.0, 1.0) for v in (2, 4, 6, 8)})
    assert tune.measure_crossover(mk("first_high"))[0] == 2 and tune.measure_crossover(mk("last_low"))[0] == 1


def test_error_strings():
    lib = nat.lib()
    for code in (0, -1, -2, -3, -4, -5):
        assert lib.linrec_hip_error_string(code)
    with pytest.raises(NotImplementedError):
        nat.check(-3, "x")
    with pytest.raises(RuntimeError):
        nat.check(-1, "x")


def test_planner_follows_the_compute_unit_count():
    """Grids of the kernels whose workgroups wait for each other are sized by the device's CU count
    (asked once per device; 256 assumed on a host without one), never by a constant."""
    lib = nat.lib()
    assert lib.linrec_set_compute_units(-1) == 0  # no override in force
    if not torch.cuda.is_available():
        assert lib.linrec_compute_units() == 256
    x = torch.empty(16, 1048576)
    try:
        seen = {}
        for cus in (256, 128, 64, 20):
            lib.linrec_set_compute_units(cus)
            assert lib.linrec_compute_units() == cus
            for is_bwd in (False, True):
                p = nat.plan(x, False, is_bwd)
                # teams whose tiles are stored two steps late
                assert p["family"] == nat.FAMILY_DRIFT
                # one workgroup per CU at most; whole teams only
                assert p["grid"] <= cus and p["grid"] % p["tasks"] == 0
                seen[(cus, is_bwd)] = p["grid"]
            # one team of workgroups per row: never more workgroups than CUs
            t = nat.plan(torch.empty(8, 1048579), False, False)  # (rows that are not whole slots)
            assert t["family"] == nat.FAMILY_TEAM and t["grid"] <= cus and t["tasks"] == cus // 8
            # a single very long row: one team of the whole device
            w = nat.plan(torch.empty(1, 1 << 25), False, False)
            assert w["family"] == nat.FAMILY_DRIFT and w["grid"] == w["tasks"] <= cus, (cus, w)
            # teams along a strided scan axis: whole teams, never more workgroups than CUs
            for is_bwd in (False, True):
                c = nat.plan(torch.empty(16384, 4096).t(), False, is_bwd)
                assert c["grid"] <= max(cus, 64) or c["family"] != nat.FAMILY_COLDRIFT, (cus, c)
                if c["family"] == nat.FAMILY_COLDRIFT:
                    assert c["grid"] == 64 * c["tasks"] <= cus
            # one workgroup per row from half the CUs on, teams below
            assert nat.plan(torch.empty(cus // 2 + 1, 24578))["family"] == nat.FAMILY_STREAM
            assert nat.plan(torch.empty(cus // 2, 24578))["family"] == nat.FAMILY_TEAM
        assert seen[(256, False)] == 256 and seen[(128, False)] == 128 and seen[(64, False)] == 64
        assert seen[(256, True)] == 256 and seen[(128, True)] == 128 and seen[(64, True)] == 64
        # a team that cannot be resident at once is refused rather than left to wait for absent mates
        lib.linrec_set_compute_units(8)
        with pytest.raises(NotImplementedError):
            nat.plan(x, False, True, nat.Tuning(nat.FAMILY_SWEEP, 8, 4, 4, 16))
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(2, 1048580), False, False, nat.Tuning(nat.FAMILY_TEAM, 8, 4, -1, 16))
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(16384, 4096).t(), False, False, nat.Tuning(nat.FAMILY_COLDRIFT, 16, 8, 1, 4))
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(1, 1 << 25), False, False, nat.Tuning(nat.FAMILY_DRIFT, 8, 4, -1, 64))
    finally:
        lib.linrec_set_compute_units(0)


def test_every_benchmarked_kernel_has_a_measured_traffic_figure():
    """bench.py reports the HBM bytes per launch that the counters showed for the kernel it times; a
    planner change that picks another kernel for one of its configurations must not turn that into null
    unnoticed.  The plan needs no device (256 compute units are assumed without one)."""
    import bench
    names = nat.kernel_table()
    missing = []
    for key, cfg in bench.CONFIGS.items():
        shape = cfg["shape"]
        x = torch.empty(shape[::-1]).t() if cfg["transposed"] else torch.empty(shape)
        for is_bwd in (False, True):
            kernel = names[nat.plan(x, cfg["reverse"], is_bwd)["kernel_id"]]
            if not bench.MEASURED_TRAFFIC_BYTES.get((key, kernel)):
                missing.append((key, "bwd" if is_bwd else "fwd", kernel))
    assert not missing, missing
    for (key, kernel), nbytes in bench.MEASURED_TRAFFIC_BYTES.items():
        elems = int(np.prod(bench.CONFIGS[key]["shape"])) * (2 if kernel.startswith(("bf16_", "f16_")) else 4)
        per_elem = 5 if "BWD" in kernel else 3
        # nothing reads or writes less than the algorithm has to; the segmented scan reads its inputs twice
        assert 0.97 * per_elem * elems <= nbytes <= 1.75 * per_elem * elems, (key, kernel, nbytes)


def test_noalloc_entry_point_rejects_what_its_static_scratch_cannot_hold():
    """linrec_fwd_noalloc turns a call down, before anything touches a device, when the launch would need
    more workspace than the library's static array (no pointer is dereferenced on the host)."""
    lib = nat.lib()
    fake = ctypes.c_void_p(1 << 20)
    limit = 4 << 20
    # one row of 2^31 - 8 floats: look-back tiles of 16384 elements, 131072 descriptors
    n = (1 << 31) - 8
    need = lib.linrec_workspace_bytes_dtype(0, 1, n, n, 1, 0, 0, None)
    assert need > limit
    assert lib.linrec_fwd_noalloc(0, fake, fake, fake, 1, n, n, 1, 0, None, None) == -5
    assert b"scratch" in lib.linrec_hip_error_string(-5)
    # ... but where a kernel that needs less serves the problem, the call falls back to it: many long rows go to one
    # workgroup per row, a strided scan axis to as many segments as the array holds maps for (or one lane per row)
    def noalloc_plan(numseq, seqlen, row_stride, elem_stride, dtype=0, tuning=None):
        pl = nat.Plan()
        rc = lib.linrec_plan_noalloc(dtype, fake, numseq, seqlen, row_stride, elem_stride, 0,
                                     ctypes.byref(tuning) if tuning else None, ctypes.byref(pl))
        return rc, pl.asdict()
    for rows, L in [(33000, 32768), (40001, 32768), (20001, 65536), (300, 8388608)]:
        assert lib.linrec_workspace_bytes_dtype(0, rows, L, L, 1, 0, 0, None) > limit, (rows, L)
        rc, pl = noalloc_plan(rows, L, L, 1)
        # (300 rows: the 44 rows beyond one per compute unit in a second launch of teams, whose maps fit)
        assert rc == 0 and pl["family"] == nat.FAMILY_STREAM and pl["workspace_bytes"] <= limit, (rows, L, rc, pl)
        assert (pl["workspace_bytes"] == 0) == (pl["tail_rows"] == 0)
    rc, pl = noalloc_plan(300, 65536, 65536, 1)  # (teams that exchange 2400 maps: the table's choice fits)
    assert rc == 0 and pl["family"] == nat.FAMILY_DRIFT and 0 < pl["workspace_bytes"] <= limit
    assert noalloc_plan(300, 8388608, 8388608, 1, tuning=nat.Tuning(nat.FAMILY_SWEEP))[0] == -5  # the caller's tuning stands
    assert noalloc_plan(3, 1 << 30, 1 << 30, 1)[0] == -5  # too few rows for one workgroup each
    rc, pl = noalloc_plan(3000, 200000, 1, 3000)  # transposed: segments, fewer than the table would take
    assert lib.linrec_workspace_bytes_dtype(0, 3000, 200000, 1, 3000, 0, 0, None) > limit
    assert rc == 0 and pl["family"] == nat.FAMILY_SEGMENT and pl["workspace_bytes"] <= limit and pl["tiles_per_row"] >= 2, pl
    rc, pl = noalloc_plan(300000, 4096, 1, 300000)  # too many rows for two segments' maps: one lane per two rows
    assert rc == 0 and pl["family"] == nat.FAMILY_COLUMN and pl["workspace_bytes"] == 0, pl
    # invalid arguments are reported as by linrec_fwd
    assert lib.linrec_fwd_noalloc(0, None, fake, fake, 4, 100000, 100000, 1, 0, None, None) == -1
    assert lib.linrec_fwd_noalloc(7, fake, fake, fake, 4, 100000, 100000, 1, 0, None, None) == -3
    assert lib.linrec_fwd_noalloc(0, fake, fake, fake, 0, 100000, 100000, 1, 0, None, None) == 0


def _plan(shape, reverse=False, is_bwd=False, tuning=None, strides=None):
    t = torch.empty(shape) if strides is None else torch.empty_strided(shape, strides)
    return nat.plan(t, reverse, is_bwd, tuning)


class TestPlanner:
    def test_benchmark_configs(self):
        names = nat.kernel_table()
        p1 = _plan((64, 4096))
        assert p1["family"] == nat.FAMILY_TILE and p1["carry"] == 0 and p1["grid"] == 64
        p2 = _plan((512, 65536))  # teams of 8 workgroups per row of 8 tiles, 32 teams, a tile stored two steps late
        assert p2["family"] == nat.FAMILY_DRIFT and (p2["waves"], p2["slots"], p2["tasks"], p2["grid"], p2["tiles_per_row"]) == (16, 2, 8, 256, 8)
        assert "drift_w16_s2_MODE_FWD_0" == names[p2["kernel_id"]] and p2["workspace_bytes"] > 0
        p2b = _plan((512, 65536), is_bwd=True)  # the backward holds three tensors: tiles of 4096 elements, a slot for each of 16 waves
        assert p2b["family"] == nat.FAMILY_DRIFT and (p2b["waves"], p2b["slots"], p2b["tasks"], p2b["grid"], p2b["tiles_per_row"]) == (16, 1, 16, 256, 16)
        assert "drift_w16_s1_MODE_BWD_1" == names[p2b["kernel_id"]] and p2b["block"] == 1024
        p3 = _plan((16384, 2048), reverse=True)
        assert (p3["waves"], p3["slots"], p3["carry"]) == (4, 2, 0) and "FWD_1" in names[p3["kernel_id"]]
        p4 = _plan((16, 1048576))  # rows of whole tiles: teams of 128 (a whole row in flight each) that go from row to row
        assert p4["family"] == nat.FAMILY_DRIFT and p4["carry"] == 1 and p4["workspace_bytes"] > 0
        assert (p4["waves"], p4["slots"]) == (8, 4)  # (teams of more than 64: the kernel of 8 waves)
        with pytest.raises(NotImplementedError):     # 16 waves of two slots are compiled for teams of at most 64
            _plan((16, 1048576), tuning=nat.Tuning(nat.FAMILY_DRIFT, 16, 2, -1, 128))
        assert _plan((16, 1048576), tuning=nat.Tuning(nat.FAMILY_DRIFT, 16, 2, -1, 64))["tasks"] == 64
        assert (p4["tasks"], p4["grid"], p4["tiles_per_row"]) == (128, 256, 128)
        p4bw = _plan((16, 1048576), is_bwd=True)  # the backward: one team of the whole launch, tiles of 4096 elements
        assert (p4bw["family"], p4bw["waves"], p4bw["slots"], p4bw["tasks"], p4bw["grid"], p4bw["tiles_per_row"]) == (nat.FAMILY_DRIFT, 16, 1, 256, 256, 256)
        p4d = _plan((16, 1048576 + 4))  # whole slots, a partial last tile: the drift kernels all the same
        assert p4d["family"] == nat.FAMILY_DRIFT and p4d["tiles_per_row"] == 129 and "drift_ragged_w8_s4" in names[p4d["kernel_id"]]
        assert p4d["tasks"] == 128 and p4d["grid"] == 256  # (a team need not divide the tiles of such a row)
        p4r = _plan((16, 1048576 + 3))  # rows that are not whole slots: one team per row
        assert p4r["family"] == nat.FAMILY_TEAM and p4r["grid"] == 16 * p4r["tasks"] and 2 <= p4r["tasks"] <= 64
        for rows, is_bwd in ((1, False), (2, False), (3, True), (6, True)):
            # a few very long rows: one team of the whole chip, every wave of a workgroup collecting maps
            p4b = _plan((rows, 1 << 23), is_bwd=is_bwd)
            assert p4b["family"] == nat.FAMILY_DRIFT and (p4b["tasks"], p4b["grid"]) == (256, 256), (rows, p4b)
        p4c = _plan((1, 1 << 20))  # too few tiles to give every workgroup of the chip a few: one look-back tile per workgroup
        assert p4c["family"] == nat.FAMILY_TILE and p4c["carry"] == 1 and p4c["grid"] == p4c["tiles_per_row"]
        p5 = nat.plan(torch.empty(256, 262144).t())
        assert p5["family"] == nat.FAMILY_COLUMN and p5["vec"] == 2  # 8 bytes of rows per lane

    def test_backward_runs_against_forward_direction(self):
        names = nat.kernel_table()
        for rev in (False, True):
            f = names[_plan((8, 100), rev, False)["kernel_id"]]
            b = names[_plan((8, 100), rev, True)["kernel_id"]]
            assert f.endswith(f"FWD_{int(rev)}") and b.endswith(f"BWD_{int(not rev)}"), (f, b)
            f = names[_plan((8, 1000), rev, False)["kernel_id"]]
            b = names[_plan((8, 1000), rev, True)["kernel_id"]]
            assert f.endswith(f"FWD_{int(rev)}_0") and b.endswith(f"BWD_{int(not rev)}_0"), (f, b)

    def test_every_row_fits_its_tile_or_is_chained(self):
        for L in [1, 2, 255, 256, 257, 1024, 2048, 2049, 4096, 4097, 8192, 8193, 16384, 100000, 2 ** 24]:
            for n in [1, 2, 95, 96, 1000, 100000]:
                p = _plan((n, L)) if n * L <= 2 ** 31 else None
                if p is None:
                    continue
                tile = p["waves"] * p["slots"] * 64 * p["vec"]
                if p["family"] == nat.FAMILY_TILE and not p["carry"]:
                    assert L <= tile, (n, L, p)
                if p["family"] == nat.FAMILY_TILE and p["carry"]:
                    assert p["tiles_per_row"] * tile >= L and p["workspace_bytes"] >= 16 * n * p["tiles_per_row"]

    def test_misaligned_rows_reserve_one_more_slot(self):
        p = _plan((4, 256))
        assert (p["waves"], p["slots"]) == (1, 1)
        p = _plan((4, 255), strides=(255, 1))  # rows start at varying 16-byte phases: 65 slots, a tile of 128
        assert p["waves"] * p["slots"] == 2
        # rows in the lower part of a tile-size bucket take fewer waves with more slots each
        assert [(q["waves"], q["slots"]) for q in (_plan((100, 320)), _plan((100, 400)), _plan((100, 600)), _plan((100, 800)))] == \
            [(1, 2), (2, 1), (2, 2), (4, 1)]

    def test_tuning_overrides(self):
        p = _plan((3, 20000), tuning=nat.Tuning(nat.FAMILY_TILE, 4, 4, 1, 3))
        assert (p["waves"], p["slots"], p["carry"], p["tasks"]) == (4, 4, 1, 3) and p["grid"] == 5 * 1
        with pytest.raises(NotImplementedError):
            _plan((3, 20000), tuning=nat.Tuning(nat.FAMILY_TILE, 4, 4, 0))  # row does not fit one tile
        with pytest.raises(NotImplementedError):
            _plan((3, 100), tuning=nat.Tuning(nat.FAMILY_TILE, 3, 5, 0))    # not compiled
        p = _plan((300, 20000), tuning=nat.Tuning(nat.FAMILY_STREAM, 16, 2))
        assert p["family"] == nat.FAMILY_STREAM and p["block"] == 1024

    def test_teams_are_chosen_where_rows_are_whole_tiles(self):
        fam = lambda shape, bwd=False, **kw: nat.plan(torch.empty(shape, **kw), False, bwd)["family"]
        D, W, ST = nat.FAMILY_DRIFT, nat.FAMILY_SWEEP, nat.FAMILY_STREAM
        # fp32 rows of whole tiles, up to 2048 of them: the forward always, the backward from 128 rows on and
        # for rows up to 131072 elements
        for shape in [(300, 65536), (256, 65536), (200, 65536), (512, 65536), (1024, 131072), (2048, 65536),
                      (16, 1 << 20), (8, 1 << 22), (4, 1 << 20)]:
            assert fam(shape) == D, shape
        # ... but not where a quarter of the chip's workgroups have a row each and all of them together at most
        # four tiles of 8192 elements per compute unit: the older kernels fill and drain faster, and the teams
        # that wait take their largest tiles in both directions, in teams of two if need be
        assert fam((96, 65536)) == W and fam((200, 32768)) == ST and fam((200, 32768), True) == ST
        for shape, team in [((128, 65536), 4), ((100, 32768), 2), ((150, 49152), 3), ((64, 131072), 8)]:
            for bwd in (False, True):
                q = nat.plan(torch.empty(shape), False, bwd)
                assert (q["family"], q["slots"], q["tasks"]) == (W, 8, team), (shape, bwd, q)
        assert fam((130, 65536)) == D and fam((63, 131072)) == D and fam((128, 65536), dtype=torch.bfloat16) == W
        for shape in [(300, 65536), (256, 65536), (512, 65536), (1024, 131072), (128, 131072), (2048, 32768)]:
            assert fam(shape, True) == D, shape
        # (the crossovers come from the generated table the library is compiled with)
        T = nat.plan_thresholds()
        # rows of few tiles of 4096 elements (and fewer than four of 8192) are left to one workgroup each, except
        # the backward of enough rows with at least four such tiles
        assert T["drift_min_small_tiles_per_row"] > 6 and 128 < T["drift_bwd_short_rows_min_rows"] <= 2048
        short_bwd = lambda n: D if n >= T["drift_bwd_short_rows_min_rows"] else ST
        # (the forward of rows of two tiles of 8192 elements: teams of two from drift_fwd_two_tiles_min_rows rows on)
        two_fwd = lambda n: D if n >= T["drift_fwd_two_tiles_min_rows"] else ST
        assert [fam(shape, b) for shape in [(2048, 16384), (768, 16384), (400, 24576), (130, 16384)] for b in (False, True)] == \
            [two_fwd(2048), short_bwd(2048), two_fwd(768), short_bwd(768), ST, short_bwd(400), ST, short_bwd(130)]
        n2 = T["drift_fwd_two_tiles_min_rows"]
        q = nat.plan(torch.empty(n2, 16384))
        assert (q["family"], q["waves"], q["slots"], q["tasks"], q["tiles_per_row"]) == (D, 16, 2, 2, 2), q
        assert fam((n2 - 1, 16384)) == ST and T["drift_fwd_min_tiles_per_row"] >= 2
        # beyond 2048 rows the forward keeps its tiles of 8192 elements
        q = nat.plan(torch.empty(4096, 32768))
        assert (q["family"], q["waves"], q["slots"], q["tasks"]) == (D, 16, 2, 4), q
        n = T["drift_bwd_short_rows_min_rows"]
        # (rows of seven such tiles: enough work in all for the rule on little work in many rows not to apply)
        assert fam((n, 28672), True) == D and fam((n - 1, 28672), True) != D
        k = T["drift_min_small_tiles_per_row"]
        k += 1 - k % 2  # (an odd number of tiles of 4096 elements: not whole tiles of 8192)
        assert fam((600, 4096 * k)) == D and fam((600, 4096 * (k - 2))) == W and fam((768, 4096 * (k - 2))) == ST
        # the backward of 16 to 127 rows with little work in all: teams that wait, with tiles of 16384 elements
        assert fam((96, 65536), True) == W and fam((24, 262144), True) == W
        assert fam((16, 1 << 20), True) == D and fam((100, 131072), True) == D and fam((128, 262144), True) == D
        assert fam((512, 262144), True) == D and fam((256, 262144), True) == D
        # more than 2048 rows: the forward still, in its tiles of 8192 elements; the backward in teams that wait (up to
        # 1024 rows of 16 tiles and more) or one workgroup per row; ragged rows one workgroup per row
        q = nat.plan(torch.empty(4096, 65536))
        assert (q["family"], q["waves"], q["slots"], q["tasks"], q["grid"]) == (D, 16, 2, 8, 256), q
        m = T["drift_bwd_max_rows"]
        assert 1024 <= m and fam((m, 65536), True) == D and fam((m + 256, 65536), True) == W
        assert fam((m + 256, 131072), True) == ST and fam((4096, 24576 + 6)) == ST and fam((4096, 65536 + 8)) == D
        # rows that are not whole slots, from the generated length on: look-back tiles of 16384 elements
        assert fam((4096, T["stream_max_len"] - 4)) == ST and fam((4096, T["stream_max_len"])) == nat.FAMILY_TILE and T["stream_max_len"] % 4
        q = nat.plan(torch.empty(300, 65536 + 6))
        assert (q["family"], q["waves"], q["slots"], q["carry"], q["tiles_per_row"]) == (nat.FAMILY_TILE, 8, 8, 1, 5), q
        assert fam((300, 65536 + 6), dtype=torch.bfloat16) == ST   # (16-bit storage: one workgroup per row)
        assert fam((3, 1 << 20)) == nat.FAMILY_TILE   # three tiles for every workgroup of a team of the whole chip: too few
        slots = lambda shape, bwd=False: nat.plan(torch.empty(shape), False, bwd)["slots"]
        # stream tiles of 16384 elements: long rows of whole such tiles, or many rows
        assert slots((m + 256, 131072), True) == 8 and slots((256, 131072), True) == 1
        assert slots((256, 32768 + 8192)) == 4
        # tiles of 4096 elements where they pad the row less, and for rows up to 16384 elements
        assert slots((1024, 16384)) == 2 and slots((3355, 10000)) == 2 and slots((1677, 20000)) == 2
        assert slots((700, 24576)) == 4 and slots((838, 24570)) == 4 and slots((800, 26002)) == 2
        assert fam((300, 24576 + 6)) == nat.FAMILY_STREAM          # rows that are not whole slots
        assert fam((300, 65536 + 4)) == D and fam((838, 40000)) == D   # whole slots, a partial last tile: drift teams
        # ... whose rows beyond one per CU, if few, go to a second launch of their own (teams per row)
        p = nat.plan(torch.empty(300, 24576 + 6))
        assert (p["tail_rows"], p["grid"]) == (44, 256) and p["workspace_bytes"] > 0
        assert [nat.plan(torch.empty(n, 24576 + 6))["tail_rows"] for n in (256, 257, 352, 353, 600)] == [0, 1, 96, 0, 0]
        assert nat.plan(torch.empty(300, 24576 + 6), tuning=nat.Tuning(nat.FAMILY_STREAM))["tail_rows"] == 0
        assert fam((300, 12288)) == nat.FAMILY_STREAM              # three tiles per row: not worth an exchange
        assert fam((T["team_min_rows"], (1 << 20) + 6)) == nat.FAMILY_TEAM          # few rows that are not whole slots: one team per row
        assert fam((T["team_min_rows"] - 1, (1 << 20) + 6)) == nat.FAMILY_TILE      # fewer: look-back tiles
        assert fam((300, 65536 + 4), dtype=torch.bfloat16) == nat.FAMILY_STREAM and fam((96, 65536), dtype=torch.bfloat16) == nat.FAMILY_SWEEP
        assert fam((300, 65536 + 8), dtype=torch.bfloat16) == D and fam((300, 65536 + 8), True, dtype=torch.bfloat16) == D
        # 16-bit storage: teams whose tiles are stored two steps late serve the backward of up to drift_bwd_max_rows
        # rows of whole tiles of 8192 elements (16 waves of one slot) and the forward of any number of rows of four and
        # more tiles of 16384 elements (16 waves of two slots), where the launch has two (forward: four) tiles for every
        # compute unit; the forward of fewer than 128 rows (up to 255 of 32 tiles and more) also in tiles of 8192
        for dt in (torch.bfloat16, torch.float16):
            for shape, bwd, slots in [((1, 1 << 25), False, 2), ((1, 1 << 25), True, 1), ((1, 1 << 22), False, 1), ((1, 1 << 22), True, 1)]:
                q = nat.plan(torch.empty(shape, dtype=dt), False, bwd)
                assert (q["family"], q["waves"], q["slots"], q["tasks"], q["grid"]) == (D, 16, slots, 256, 256), q
            q = nat.plan(torch.empty(16, 1 << 20, dtype=dt))
            assert (q["family"], q["waves"], q["slots"], q["tasks"], q["grid"]) == (D, 16, 2, 64, 256), q
            q = nat.plan(torch.empty(16, 8192 * 129, dtype=dt))
            assert (q["family"], q["waves"], q["slots"], q["tasks"], q["grid"]) == (D, 16, 1, 43, 215), q  # (five teams of 43: 215 of 256 workgroups)
            assert fam((2, 1 << 22), dtype=dt) == D and fam((1, 1 << 20), dtype=dt) == nat.FAMILY_TILE
            assert fam((1, 1 << 20), True, dtype=dt) == nat.FAMILY_TILE
            assert [fam((n, 1 << 22), b, dtype=dt) for n in (3, 4, 5, 6) for b in (False, True)] == [D] * 8
            assert [fam((n, 65536), True, dtype=dt) for n in (127, 300, 512, T["drift_bwd_max_rows"])] == [D] * 4
            assert fam((T["drift_bwd_max_rows"] + 1, 65536), True, dtype=dt) == ST
            assert [fam((n, 65536), dtype=dt) for n in (128, 200, 256, 300, 512, 5000)] == [W, ST, D, D, D, D]
            assert [fam((n, 32768), dtype=dt) for n in (512, 2048)] == [ST, ST]       # rows of two tiles of 16384
            # rows of whole tiles of 8192 elements only: up to half_drift_fwd_small_tiles_max_rows rows, and up to 255
            # rows of 32 tiles and more
            few = T["half_drift_fwd_small_tiles_max_rows"]
            assert fam((few, 8192 * 41), dtype=dt) == D and fam((few + 1, 8192 * 31), dtype=dt) != D
            # (rows of an odd number of such tiles: teams with the forward's tiles of 16384 elements, the last one half full,
            # where they divide the rows evenly; bf16 300 x 73728 27.6 us against 30.3 us for one workgroup per row)
            assert [fam((n, 8192 * 9), dtype=dt) for n in (128, 200, 300)] == [W, ST, D]
            assert [fam((n, 8192 * 33), dtype=dt) for n in (64, 128, 160, 250, 256)] == [D, D, D, D, ST]
            # a few rows: the tiles per compute unit the table asks for (forward: of 16384 elements)
            for bwd, per_cu, tile in ((False, T["half_drift_fwd_min_tiles_per_cu"], 16384), (True, T["half_drift_bwd_min_tiles_per_cu"], 8192)):
                assert fam((16, per_cu * 16 * tile), bwd, dtype=dt) == D
                assert fam((16, (per_cu * 16 - 1) * tile), bwd, dtype=dt) != D or (not bwd and per_cu * 16 - 1 >= 64)
            q = nat.plan(torch.empty(512, 65536, dtype=dt))
            assert (q["waves"], q["slots"], q["tasks"], q["grid"]) == (16, 2, 4, 256), q
            assert fam((24, 262144), dtype=dt) == nat.FAMILY_TEAM
            assert fam((24, 262144), True, dtype=dt) == (D if 24 * 32 >= 256 * T["half_drift_bwd_min_tiles_per_cu"] else nat.FAMILY_TEAM)
            # one or two rows of whole tiles of 4096 elements only: the forward in 8 waves, the backward in tiles of 8192
            # elements, the last one half full
            q = nat.plan(torch.empty(2, 4096 * 1001, dtype=dt))
            assert (q["family"], q["waves"], q["slots"], q["tiles_per_row"]) == (D, 8, 1, 1001), q
            q = nat.plan(torch.empty(2, 4096 * 1001, dtype=dt), False, True)
            assert (q["family"], q["waves"], q["slots"], q["tiles_per_row"]) == (D, 8, 2, 501), q
            # a caller who names the family and nothing else gets the tiles of 8192 elements where the rows are whole ones
            q = nat.plan(torch.empty(512, 65536, dtype=dt), tuning=nat.Tuning(D))
            assert (q["waves"], q["slots"], q["tasks"]) == (16, 1, 8), q
            # many rows of exactly two of the stream kernel's tiles: one workgroup walks the row
            assert [fam((n, 16384), b, dtype=dt) for n in (2048, 4096) for b in (False, True)] == [ST] * 4
            assert fam((1024, 16384), dtype=dt) == nat.FAMILY_TILE and fam((2048, 16000), dtype=dt) == nat.FAMILY_TILE
            # rows beyond one per CU get a launch of their own in the backward only
            tails = lambda n: [nat.plan(torch.empty(n, 65536 + 4, dtype=dt), False, b)["tail_rows"] for b in (False, True)]
            assert tails(288) == [0, 32] and tails(352) == [0, 96] and tails(400) == [0, 0]
        # 16-bit backward with less than two tiles for every compute unit: the teams that wait (from 32 rows on)
        assert fam((100, 32768), True, dtype=torch.bfloat16) == W and fam((100, 32768), dtype=torch.bfloat16) == W
        assert fam((64, 262144), True) == D
        pf, pb = nat.plan(torch.empty(300, 65536)), nat.plan(torch.empty(300, 65536), False, True)
        assert (pf["tasks"], pf["grid"]) == (8, 256) and (pb["tasks"], pb["grid"]) == (16, 256)
        p = nat.plan(torch.empty(40, 8192 * 24))                    # 24 tiles: teams of 24, 10 of them
        p2 = nat.plan(torch.empty(300, 4096 * 9))                   # whole tiles of 4096 elements only
        assert (p2["family"], p2["waves"], p2["slots"], p2["tasks"], p2["tiles_per_row"], p2["grid"]) == (D, 16, 1, 9, 9, 252)
        assert p["family"] == D and (p["tasks"], p["grid"]) == (24, 240)
        p = nat.plan(torch.empty(40, 8192 * 24), False, True)       # the backward of 16 to 127 rows waits
        assert p["family"] == W and p["tasks"] == 12

    def test_few_rows_on_a_strided_scan_axis_are_cut_into_segments(self):
        S, C = nat.FAMILY_SEGMENT, nat.FAMILY_COLUMN
        plan = lambda n, L, **kw: nat.plan(torch.empty(L, n, **kw).t())
        # (fp32: four rows per lane from 512 rows on where the scan axis is long enough for all the waves wanted)
        for n, L, vec, segments in [(64, 100000, 1, 962), (256, 65536, 2, 512), (700, 100000, 4, 368),
                                    (2200, 16384, 4, 114), (2048, 1024, 2, 32), (1000, 300, 2, 10), (72, 460476, 1, 900)]:
            p = plan(n, L)
            assert (p["family"], p["vec"], p["tiles_per_row"], p["block"]) == (S, vec, segments, 64), (n, L, p)
            # whole batches of 8 per segment, every position in exactly one segment
            assert p["tasks"] % 8 == 0 and (segments - 1) * p["tasks"] < L <= segments * p["tasks"]
            assert p["grid"] == -(-(segments * (n // vec)) // 64) <= 1024  # lanes numbered segment by segment, no padding
            # the maps take the upper half of the workspace
            assert p["workspace_bytes"] >= 2 * (2 * segments * n * 4)
        assert plan(65536, 4096)["family"] == C and plan(1024, 255)["family"] == C
        # plain column kernels: 16 timesteps in flight while the launch has at most one wave per SIMD
        assert [plan(n, 1024)["slots"] for n in (40000, 65536, 65600, 262144)] == [16, 16, 8, 8]
        # 16-bit storage: segments up to twice as many rows, and never less than 4 bytes of rows per lane
        assert plan(6000, 4096, dtype=torch.bfloat16)["family"] == S and plan(40000, 4096)["family"] == C
        p = plan(100000, 1024, dtype=torch.float16)
        assert (p["family"], p["vec"], p["slots"]) == (C, 2, 16)
        assert plan(100001, 1024, dtype=torch.float16)["vec"] == 1
        assert plan(1001, 5000)["vec"] == 1 and plan(1001, 5000)["family"] == S
        p = plan(2048, 16384, dtype=torch.bfloat16)
        assert (p["family"], p["vec"], p["tiles_per_row"]) == (S, 4, 128)
        p = nat.plan(torch.empty(16384, 4096).t(), tuning=nat.Tuning(S, 4, 8, -1, 16))
        assert (p["vec"], p["tiles_per_row"], p["tasks"]) == (4, 16, 1024)
        # rows further apart than one element stay with the element-wise kernel
        assert nat.plan(torch.empty(5000, 128).t()[::2])["family"] == nat.FAMILY_NAIVE

    def test_a_few_thousand_rows_on_a_strided_scan_axis_take_teams_along_the_scan_axis(self):
        """fp32 rows of at least 2048 elements, few enough that teams of workgroups along the scan axis are what
        fills the chip: blocks of 64 rows, steps of 128 positions, the team the power of two that fills 256 CUs."""
        D, S, C = nat.FAMILY_COLDRIFT, nat.FAMILY_SEGMENT, nat.FAMILY_COLUMN
        plan = lambda n, L, bwd=False, **kw: nat.plan(torch.empty(L, n, **kw).t(), False, bwd)
        names = nat.kernel_table()
        for n, L, team_f, team_b in [(4096, 16384, 4, 4), (4000, 16384, 4, 4), (2048, 16384, 8, 8), (3072, 16384, 4, 4),
                                     (2048, 4096, 8, 8), (4096, 2048, 4, 4), (1024, 100000, 16, 0), (8192, 4096, 0, 2),
                                     # teams of 4 and 8 from 65 % of the chip on, teams of 16 from seven eighths on
                                     (3000, 16384, 4, 4), (1300, 16384, 8, 8), (900, 32768, 16, 0),
                                     (768, 32768, 0, 0), (2560, 8192, 0, 0), (2200, 16384, 0, 0), (6144, 4096, 0, 0),
                                     (512, 65536, 0, 0), (4096, 2000, 0, 0)]:
            for bwd, team in ((False, team_f), (True, team_b)):
                p = plan(n, L, bwd)
                if not team:
                    assert p["family"] in (S, C), (n, L, bwd, p)
                    continue
                waves, run = (8, 16) if bwd else (16, 8)
                assert (p["family"], p["waves"], p["slots"], p["vec"], p["tasks"]) == (D, waves, run, 1, team), (n, L, bwd, p)
                assert p["grid"] == -(-n // 64) * team <= 256 and p["block"] == 64 * waves
                assert p["tiles_per_row"] == -(-L // 128) >= 8 * team // 2
                assert names[p["kernel_id"]] == f"coldrift_w{waves}_v1_u{run}_MODE_{'BWD' if bwd else 'FWD'}_{int(bwd)}"
                # a descriptor of two 64-bit words per row and step, in the lower half of the workspace
                assert p["workspace_bytes"] >= 2 * 16 * -(-n // 64) * 64 * p["tiles_per_row"]
        # 16-bit storage: two rows to a lane (blocks of 128 rows), teams of 4 from three quarters of the chip on and
        # teams of 8 from seven eighths on, every member with two steps at least
        for dtype, pfx in ((torch.bfloat16, "bf16_"), (torch.float16, "f16_")):
            for n, L, team in [(4096, 16384, 8), (8192, 4096, 4), (6144, 4096, 4), (4096, 2048, 8), (3600, 16384, 8),
                               (3072, 16384, 0), (2560, 8192, 0), (2048, 16384, 0), (2048, 4096, 0), (16384, 4096, 0),
                               (1024, 32768, 0), (4097, 16384, 0), (4096, 2000, 0), (5120, 4096, 0)]:
                for bwd in (False, True):
                    p = plan(n, L, bwd, dtype=dtype)
                    if not team:
                        assert p["family"] in (S, C), (n, L, bwd, p)
                        continue
                    waves, run = (8, 16) if bwd else (16, 8)
                    assert (p["family"], p["waves"], p["slots"], p["vec"], p["tasks"]) == (D, waves, run, 2, team), (n, L, bwd, p)
                    assert p["grid"] == -(-n // 128) * team <= 256 and p["block"] == 64 * waves
                    assert p["tiles_per_row"] == -(-L // 128) >= 2 * team
                    assert names[p["kernel_id"]] == f"{pfx}coldrift_w{waves}_v2_u{run}_MODE_{'BWD' if bwd else 'FWD'}_{int(bwd)}"
                    assert p["workspace_bytes"] >= 2 * 16 * -(-n // 128) * 128 * p["tiles_per_row"]
        # on request: any compiled geometry, teams of at most as many members as the workgroup has waves
        x = torch.empty(5000, 700).t()
        p = nat.plan(x, tuning=nat.Tuning(D, 8, 16, 1, 4))
        assert (p["family"], p["grid"], p["block"], p["tiles_per_row"]) == (D, 11 * 4, 512, 40)
        p = nat.plan(x, False, True, nat.Tuning(D, 16, 4, 1, 16))
        assert (p["grid"], p["block"], p["tiles_per_row"]) == (11 * 16, 1024, 79)
        for bad in (nat.Tuning(D, 8, 16, 1, 16), nat.Tuning(D, 16, 8, 1, 32), nat.Tuning(D, 16, 16, 1, 2), nat.Tuning(D, 16, 8, 2, 2)):
            with pytest.raises(NotImplementedError):
                nat.plan(x, tuning=bad)
        xh = torch.empty(5000, 700, dtype=torch.bfloat16).t()
        p = nat.plan(xh, tuning=nat.Tuning(D, 8, 16, 2, 4))   # 16-bit storage: two rows to a lane, or one on request
        assert (p["family"], p["vec"], p["grid"], p["tiles_per_row"]) == (D, 2, 6 * 4, 40)
        with pytest.raises(NotImplementedError):
            nat.plan(xh, tuning=nat.Tuning(D, 8, 16, 1, 4))
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(5000, 701, dtype=torch.bfloat16).t(), tuning=nat.Tuning(D, 8, 16, 2, 4))  # an odd number of rows
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(700, 5000), tuning=nat.Tuning(D))  # rows along the unit-stride axis

    def test_mid_sized_row_counts_on_a_strided_scan_axis_share_rows_among_the_waves_of_a_workgroup(self):
        S, C = nat.FAMILY_SEGMENT, nat.FAMILY_COLUMN
        plan = lambda n, L, bwd=False, **kw: nat.plan(torch.empty(L, n, **kw).t(), False, bwd)
        # the block form: plan.carry = lane groups per wave (0 for the plain column kernels)
        block = lambda p: p["carry"] if (p["family"], p["waves"], p["block"], p["workspace_bytes"]) == (C, 16, 1024, 0) else 0
        # the form with the most workgroups that still leaves every CU at most one
        for n, L, vec, groups in [(4096, 1024, 1, 2), (8192, 4096, 1, 2), (8193, 4096, 1, 1), (12288, 4096, 1, 1),
                                  (16384, 2048, 2, 2), (16384, 256, 1, 1), (15358, 2048, 1, 1), (15360, 1024, 2, 2), (16383, 2048, 1, 1),
                                  (16386, 2048, 2, 1), (20000, 2048, 2, 1),
                                  (32768, 2048, 2, 1), (20001, 2048, 1, 1),
                                  (7000, 2048, 1, 1), (7008, 2048, 1, 2), (5000, 2048, 1, 2)]:  # lines off 128-byte boundaries
            p = plan(n, L)
            assert block(p) == groups and (p["vec"], p["slots"], p["grid"]) == (vec, 8, -(-(n // vec) // (64 // groups))), (n, L, p)
            assert p["tiles_per_row"] == -(-L // (128 * groups))
        # the backward with two rows per lane holds three tensors: runs of 4 positions
        assert [(block(p), p["vec"], p["slots"], p["tiles_per_row"]) for p in (plan(24576, 2048, True), plan(32767, 2048, True))] == \
            [(1, 2, 4, 32), (1, 1, 8, 16)]
        assert block(plan(32768, 2048, True)) == 1 and not block(plan(32770, 2048)) and not block(plan(4095, 1024))
        # a second round of workgroups that is at least half full
        assert [block(plan(n, 2048)) for n in (49150, 49152, 61440, 61442)] == [0, 1, 1, 0] and plan(50000, 2048)["vec"] == 2
        assert plan(4095, 1024)["family"] == S and not block(plan(16384, 255))
        # the backward with two lane groups from 6144 rows on
        # (8192 rows: teams of two along the scan axis, the column drift kernels)
        assert [block(plan(n, 8192, True)) for n in (4096, 6143, 6144, 8192, 8193)] == [0, 0, 2, 0, 1]
        # 16-bit storage: 4 bytes of rows per lane; forward from 8192 rows, backward from 10240, two lane groups
        # up to 16384 rows
        for n, fwd, bwd in [(8190, 0, 0), (8192, 2, 0), (10240, 2, 2), (16384, 2, 2), (16386, 1, 1), (24576, 1, 1), (65536, 1, 1), (65538, 0, 0)]:
            p, pb = plan(n, 1024, dtype=torch.bfloat16), plan(n, 1024, True, dtype=torch.float16)
            assert (block(p), block(pb)) == (fwd, bwd), (n, p, pb)
            assert not fwd or (p["vec"], p["slots"]) == (2, 8)
            assert not bwd or (pb["vec"], pb["slots"], pb["tiles_per_row"]) == (2, 4, 16 // bwd)
        assert not block(plan(16385, 1024, dtype=torch.bfloat16))     # an odd row count: no two rows per lane
        # on request for other row counts (family COLUMN, carry = lane groups), any compiled geometry
        p = nat.plan(torch.empty(300, 130).t(), tuning=nat.Tuning(C, 2, 8, 1, 0))
        assert block(p) == 1 and (p["vec"], p["grid"]) == (2, 2)
        p = nat.plan(torch.empty(300, 130).t(), tuning=nat.Tuning(C, 1, 0, 2, 0))
        assert block(p) == 2 and (p["vec"], p["grid"], p["tiles_per_row"]) == (1, 5, 2)
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(300, 131).t(), tuning=nat.Tuning(C, 2, 8, 1, 0))
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(300, 130).t(), False, True, nat.Tuning(C, 2, 8, 1, 0))  # no such backward kernel
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(300, 130).t(), tuning=nat.Tuning(C, 1, 0, 4, 0))  # four lane groups: not compiled
        assert not block(nat.plan(torch.empty(2048, 16384).t(), tuning=nat.Tuning(C)))

    def test_short_rows_share_a_wave(self):
        G = nat.FAMILY_GROUP
        for L, lanes in [(4, 1), (8, 2), (16, 4), (24, 8), (64, 16), (100, 32), (128, 32)]:
            p = _plan((1000, L))
            assert (p["family"], p["tasks"]) == (G, lanes), (L, p)
            assert p["grid"] * 4 * (64 // lanes) >= 1000
        assert _plan((1000, 132))["family"] == nat.FAMILY_TILE
        # rows that start inside a slot take one slot more (rows with gaps between them: the flat kernels
        # take the dense ones)
        for L, lanes in [(1, 1), (5, 2), (30, 16), (125, 32)]:
            p = _plan((1000, L), strides=(L + 1, 1)) if L > 1 else _plan((1000, L))
            assert (p["family"], p["tasks"]) == (G, lanes), (L, p)
        assert _plan((1000, 126), strides=(127, 1))["family"] == nat.FAMILY_TILE

    def test_dense_short_rows_that_are_not_whole_slots_are_scanned_as_one_flat_array(self):
        F, G = nat.FAMILY_FLAT, nat.FAMILY_GROUP
        for L, slots in [(2, 2), (3, 2), (5, 2), (30, 2), (63, 2), (65, 4), (129, 4), (159, 4)]:  # (also rows shorter than a slot)
            p = _plan((1000, L))
            assert (p["family"], p["slots"], p["vec"], p["block"], p["workspace_bytes"]) == (F, slots, 4, 256, 0), (L, p)
            assert p["grid"] * 4 * 64 * slots * 4 >= 1000 * L
        assert _plan((1000, 121))["family"] == G and _plan((1000, 105))["family"] == F  # 28 to 32 lanes of a group: group
        # not for whole slots, rows of one element or longer than 40 slots, a single row, gaps, misaligned bases
        for shape, kw in [((1000, 32), {}), ((1000, 1), {}), ((1000, 161), {}), ((1, 30), {}), ((1000, 30), dict(strides=(31, 1)))]:
            assert _plan(shape, **kw)["family"] != F, (shape, kw)
        assert nat.plan(torch.empty(30001)[1:].view(1000, 30))["family"] == nat.FAMILY_GROUP
        assert _plan((1000, 239), tuning=nat.Tuning(F))["family"] == F       # up to 60 slots on request
        with pytest.raises(NotImplementedError):
            _plan((1000, 241), tuning=nat.Tuning(F))
        for L in (30, 4, 7):  # (16-bit storage: rows of half a slot as well)
            p = nat.plan(torch.empty(1000, L, dtype=torch.bfloat16))
            assert (p["family"], p["slots"], p["vec"]) == (F, 2, 8)
        assert nat.plan(torch.empty(1000, 32, dtype=torch.bfloat16))["family"] == nat.FAMILY_GROUP
        assert _plan((1000, 32), strides=(36, 1))["family"] == G      # padded rows that do
        p = _plan((1000, 5), strides=(8, 1))
        assert (p["family"], p["tasks"]) == (G, 2)
        p = nat.plan(torch.empty(1000, 256, dtype=torch.bfloat16))
        assert (p["family"], p["tasks"], p["vec"]) == (G, 32, 8)
        p = nat.plan(torch.empty(1000 * 64 + 4)[1:1 + 64000].view(1000, 64))  # base off a slot boundary
        assert (p["family"], p["tasks"]) == (G, 32)
        p = _plan((1000, 16), tuning=nat.Tuning(G, 0, 0, -1, 16))     # more lanes than needed
        assert p["tasks"] == 16
        with pytest.raises(NotImplementedError):
            _plan((1000, 64), tuning=nat.Tuning(G, 0, 0, -1, 8))      # fewer than the row has slots

    def test_sweep_family_takes_rows_of_whole_tiles_only(self):
        W = nat.FAMILY_SWEEP
        p = _plan((512, 65536), tuning=nat.Tuning(W))
        assert (p["family"], p["waves"], p["slots"], p["tasks"], p["tiles_per_row"], p["grid"]) == (W, 8, 4, 8, 8, 512)
        assert p["workspace_bytes"] >= 16 * 512 * 8
        p = _plan((10, 1 << 20), tuning=nat.Tuning(W))           # 128 tiles per row: teams of 16, one per row
        assert (p["tasks"], p["grid"]) == (16, 160)
        p = _plan((512, 65536), tuning=nat.Tuning(W, 8, 4, 5, 4))  # five teams of four
        assert (p["tasks"], p["grid"]) == (4, 20)
        for shape, strides in [((512, 65537), None), ((512, 65536), (65537, 1)), ((512, 8192 * 3), None)]:
            tun = nat.Tuning(W) if shape[1] != 8192 * 3 else nat.Tuning(W, 8, 4, -1, 2)  # 2 does not divide 3
            with pytest.raises(NotImplementedError):
                _plan(shape, tuning=tun, strides=strides)
        with pytest.raises(NotImplementedError):
            nat.plan(torch.empty(512 * 65536 + 4)[1:1 + 512 * 65536].view(512, 65536), tuning=nat.Tuning(W))

    def test_empty_and_invalid(self):
        lib = nat.lib()
        plan = nat.Plan()
        assert lib.linrec_plan_f32(None, 0, 10, 10, 1, 0, 0, None, ctypes.byref(plan)) == 0 and plan.kernel_id == -1
        assert lib.linrec_plan_f32(None, 4, -1, 10, 1, 0, 0, None, ctypes.byref(plan)) == -1
        assert lib.linrec_plan_f32(None, 4, 10, 5, 1, 0, 0, None, ctypes.byref(plan)) == -1  # rows overlap
        assert lib.linrec_plan_f32(None, 4, 2 ** 31, 2 ** 31, 1, 0, 0, None, ctypes.byref(plan)) == -4
        assert lib.linrec_workspace_bytes(16, 1 << 20, 1 << 20, 1, 0, 0, None) > 0
        assert lib.linrec_workspace_bytes(4096, 24582, 24582, 1, 0, 0, None) == 0  # one workgroup per row: nobody waits
        assert lib.linrec_workspace_bytes_for_tiles(0) == 0
        assert lib.linrec_workspace_bytes_for_tiles(1000) >= 16 + 16 * 1000

    def test_kernel_table_is_consistent(self):
        names = nat.kernel_table()
        assert len(names) == len(set(names)) == nat.lib().linrec_kernel_count()
        assert nat.lib().linrec_kernel_name(len(names)) is None


class TestLayout:
    def test_layouts_address_every_element_where_the_tensor_has_it(self):
        """Random views (slices, steps, permutations, broadcasts) of random tensors: whenever row_layout
        or batched_layout describes a tensor, the strides it reports reach every element at the storage
        offset torch gives it, and no two elements share one."""
        from torch._subclasses.fake_tensor import FakeTensorMode
        rng = np.random.default_rng(7)
        described = {"rows": 0, "batched": 0, "neither": 0}

        def offsets(t):  # storage offset of every element, in row-major index order
            idx = np.indices(tuple(t.shape)).reshape(t.dim(), -1)
            return (idx * np.array(t.stride(), dtype=np.int64)[:, None]).sum(0)

        with FakeTensorMode():
            for case in range(900):
                rank = int(rng.integers(1, 5))
                shape = [int(rng.integers(1, 7)) for _ in range(rank)]
                t = torch.empty(shape, device="cuda")
                if rank >= 3 and case % 3 == 0:
                    t = t.transpose(-1, -2)  # a batch of transposed matrices, before anything else is done to it
                for _ in range(int(rng.integers(0, 4))):
                    op = int(rng.integers(0, 5))
                    d = int(rng.integers(0, t.dim()))
                    if op == 0 and t.dim() > 1:
                        t = t.transpose(d, int(rng.integers(0, t.dim())))
                    elif op == 1 and t.size(d) > 1:
                        t = t.narrow(d, int(rng.integers(0, 2)), t.size(d) - 1)
                    elif op == 2 and t.size(d) > 2:
                        t = t[(slice(None),) * d + (slice(None, None, 2),)]
                    elif op == 3 and t.size(d) == 1:
                        t = t.expand(*[int(rng.integers(2, 4)) if i == d else -1 for i in range(t.dim())])
                    elif op == 4 and t.dim() > 2:
                        t = t.permute(*rng.permutation(t.dim()).tolist())
                if t.numel() == 0:
                    continue
                off = offsets(t)
                lay, bl = nat.row_layout(t), nat.batched_layout(t)
                assert lay is None or bl is None
                if lay is not None:
                    n, L, rs, es = lay
                    want = (np.arange(n)[:, None] * rs + np.arange(L)[None, :] * es).reshape(-1)
                    described["rows"] += 1
                elif bl is not None:
                    B, C, L, bs, rs, es = bl
                    want = (np.arange(B)[:, None, None] * bs + np.arange(C)[None, :, None] * rs
                            + np.arange(L)[None, None, :] * es).reshape(-1)
                    described["batched"] += 1
                else:
                    described["neither"] += 1
                    continue
                assert np.array_equal(off, want), (case, tuple(t.shape), t.stride(), lay, bl)
                assert len(np.unique(off)) == off.size or (lay is not None and lay[1] == 1), (case, t.stride(), lay, bl)
        assert min(described.values()) > 5, described

    def test_library_rejects_strides_under_which_elements_share_an_address(self):
        lib = nat.lib()
        p = nat.Plan()
        plan = lambda n, L, rs, es: lib.linrec_plan_f32(None, n, L, rs, es, 0, 0, None, ctypes.byref(p))
        assert plan(6, 40, 40, 1) == 0 and plan(6, 40, 1, 6) == 0 and plan(6, 40, 120, 3) == 0 and plan(3, 40, 2, 6) == 0
        for n, L, rs, es in [(6, 40, 1, 0), (6, 40, 0, 1), (6, 40, 39, 1), (6, 40, 1, 5), (6, 40, 3, 2), (1, 40, 40, 0),
                             (6, 1, 0, 1)]:
            assert plan(n, L, rs, es) == -1, (n, L, rs, es)

    def test_row_layout(self):
        assert nat.row_layout(torch.empty(5, 7)) == (5, 7, 7, 1)
        assert nat.row_layout(torch.empty(2, 3, 7)) == (6, 7, 7, 1)
        assert nat.row_layout(torch.empty(7)) == (1, 7, 7, 1)
        assert nat.row_layout(torch.empty(5, 10)[:, :7]) == (5, 7, 10, 1)
        assert nat.row_layout(torch.empty(7, 5).t()) == (5, 7, 1, 5)
        assert nat.row_layout(torch.empty(2, 3, 10)[:, :, :7]) == (6, 7, 10, 1)
        assert nat.row_layout(torch.empty(4, 3, 7)[::2]) is None          # leading dims do not collapse
        assert nat.row_layout(torch.empty(1, 7).expand(5, 7)) is None     # overlapping rows
        assert nat.row_layout(torch.empty(5, 0)) == (0, 0, 1, 1)

    def test_output_like_keeps_strides_of_uniform_rows(self):
        t = torch.empty(7, 5).t()
        assert nat.output_like(t).stride() == t.stride()
        assert nat.output_like(torch.empty(5, 10)[:, :7]).stride() == (10, 1)
        assert nat.output_like(torch.empty(4, 3, 7)[::2]).is_contiguous()


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, dtype=dtype, generator=g), torch.rand(shape, dtype=dtype, generator=g) * 1.6 - 0.8,
            torch.randn(shape, dtype=dtype, generator=g))


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", [(1,), (9,), (4, 33), (2, 3, 17), (70000, 3)])
def test_host_path_matches_checker(shape, dtype, reverse):
    x, c, dy = _rand(shape, dtype, 1)
    y = linrec_amd.linrec(x, c, reverse)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    np.testing.assert_array_equal(y.numpy(), oracle.fwd(x.numpy(), c.numpy(), reverse, dtype=npdt))
    dx, dc = linrec_amd.linrec_bwd(dy, c, y, reverse)
    dx_t, dc_t = oracle.bwd(dy.numpy(), c.numpy(), y.numpy(), reverse, dtype=npdt)
    np.testing.assert_allclose(dx.numpy(), dx_t, rtol=1e-6 if dtype == torch.float32 else 1e-14, atol=1e-6)
    np.testing.assert_allclose(dc.numpy(), dc_t, rtol=1e-6 if dtype == torch.float32 else 1e-14, atol=1e-6)


@pytest.mark.parametrize("reverse", [False, True])
def test_host_path_layouts(reverse):
    x, c, dy = _rand((6, 40), torch.float64, 2)
    want = oracle.fwd(x.numpy(), c.numpy(), reverse)
    # transposed storage, row-padded views, non-collapsible leading dims, mismatched coeff strides
    xt, ct = x.t().contiguous().t(), c.t().contiguous().t()
    yt = linrec_amd.linrec(xt, ct, reverse)
    assert yt.stride() == xt.stride()
    np.testing.assert_array_equal(yt.numpy(), want)
    wide = torch.zeros(6, 50, dtype=torch.float64)
    wide[:, :40] = x
    np.testing.assert_array_equal(linrec_amd.linrec(wide[:, :40], c, reverse).numpy(), want)
    x3 = torch.stack([x, x * 2, x * 3])[::2]
    c3 = torch.stack([c, c, c])[::2]
    y3 = linrec_amd.linrec(x3, c3, reverse)
    np.testing.assert_array_equal(y3[0].numpy(), want)
    np.testing.assert_allclose(y3[1].numpy(), 3 * want, rtol=1e-14)
    # broadcast inputs (zero strides): the result is a dense tensor of its own
    xb, cb = x[:, :1].expand(6, 40), c[:1].expand(6, 40)
    yb = linrec_amd.linrec(xb, cb, reverse)
    assert yb.is_contiguous()
    np.testing.assert_array_equal(yb.numpy(), oracle.fwd(xb.contiguous().numpy(), cb.contiguous().numpy(), reverse))


class TestOperatorContract:
    def test_autograd_matches_checker_and_reverse_gets_none(self):
        for reverse in (False, True):
            x, c, dy = _rand((3, 25), torch.float64, 3)
            x.requires_grad_()
            c.requires_grad_()
            y = linrec_amd.linrec(x, c, reverse)
            gx, gc = torch.autograd.grad(y, (x, c), dy)
            dx_t, dc_t = oracle.bwd(dy.numpy(), c.detach().numpy(), y.detach().numpy(), reverse)
            np.testing.assert_allclose(gx.numpy(), dx_t, rtol=1e-13)
            np.testing.assert_allclose(gc.numpy(), dc_t, rtol=1e-13)

    def test_saved_tensors_are_coeffs_and_outputs(self):
        x, c, _ = _rand((2, 9), torch.float64, 4)
        x.requires_grad_()
        c.requires_grad_()
        y = linrec_amd.linrec(x, c)
        saved = y.grad_fn.saved_tensors if hasattr(y.grad_fn, "saved_tensors") else None
        if saved is not None:
            assert len(saved) == 2
            assert saved[0].data_ptr() == c.data_ptr() and torch.equal(saved[1], y)

    def test_gradcheck_float64(self):
        x, c, _ = _rand((2, 7), torch.float64, 5)
        x.requires_grad_()
        c.requires_grad_()
        for reverse in (False, True):
            assert torch.autograd.gradcheck(lambda a, b: linrec_amd.linrec(a, b, reverse), (x, c))

    def test_opcheck(self):
        x, c, dy = _rand((3, 11), torch.float32, 6)
        torch.library.opcheck(torch.ops.linrec_amd.linrec_fwd.default, (x, c, False))
        torch.library.opcheck(torch.ops.linrec_amd.linrec_fwd.default, (x.requires_grad_(), c.requires_grad_(), True))
        y = linrec_amd.linrec(x.detach(), c.detach())
        torch.library.opcheck(torch.ops.linrec_amd.linrec_bwd.default, (dy, c.detach(), y, False))

    def test_non_unit_stride_grad_is_accepted(self):
        x, c, dy = _rand((5, 12), torch.float64, 7)
        x.requires_grad_()
        y = linrec_amd.linrec(x, c)
        g_strided = dy.t().contiguous().t()  # stride(-1) != 1, the case linrec/impl/cuda/ops.py:96 copies
        (gx,) = torch.autograd.grad(y, x, g_strided)
        dx_t, _ = oracle.bwd(dy.numpy(), c.numpy(), y.detach().numpy())
        np.testing.assert_allclose(gx.numpy(), dx_t, rtol=1e-13)

    def test_errors(self):
        x = torch.randn(3, 5)
        with pytest.raises(RuntimeError):
            linrec_amd.linrec(x, torch.randn(3, 6))
        with pytest.raises(RuntimeError):
            linrec_amd.linrec(x, torch.randn(3, 5, dtype=torch.float64))
        with pytest.raises(RuntimeError):
            linrec_amd.linrec(x.to(torch.int32), x.to(torch.int32))
        with pytest.raises(RuntimeError):
            linrec_amd.linrec(torch.tensor(1.0), torch.tensor(1.0))

    def test_empty_tensors(self):
        for shape in [(0, 5), (4, 0), (0,)]:
            x = torch.randn(shape, requires_grad=True)
            y = linrec_amd.linrec(x, torch.randn(shape))
            assert y.shape == torch.Size(shape)
            y.sum().backward()
            assert x.grad.shape == torch.Size(shape)

    def test_aliases_of_the_reference_names(self):
        assert linrec_amd.linrec_pipe is linrec_amd.linrec_tile is linrec_amd.linrec_ref is linrec_amd.linrec

    def test_first_coefficient_is_never_used(self):
        x, c, _ = _rand((2, 6), torch.float32, 8)
        c2 = c.clone()
        c2[:, 0] = float("nan")
        assert torch.equal(linrec_amd.linrec(x, c2), linrec_amd.linrec(x, c))
        c3 = c.clone()
        c3[:, -1] = float("inf")
        assert torch.equal(linrec_amd.linrec(x, c3, True), linrec_amd.linrec(x, c, True))


def test_device_tensors_never_fall_back(monkeypatch):
    """With the library missing, the binding raises instead of computing something else."""
    monkeypatch.setattr(nat, "_lib", None)
    monkeypatch.setattr(nat, "LIB_PATH", "/nonexistent/liblinrec_hip.so")
    with pytest.raises(RuntimeError, match="missing"):
        nat.lib()


def test_torch_compile_traces_through_the_fake_impls():
    """torch.compile needs the fake (meta) functions and the autograd registration to agree with the
    real op (the reason the reference registers custom ops at all, linrec/impl/cuda/ops.py:105-118).
    aot_eager exercises tracing, functionalisation and the joint forward/backward graph without
    needing a code-generating backend."""
    x, c, dy = _rand((4, 19), torch.float64, 9)
    x.requires_grad_()
    c.requires_grad_()

    def f(a, b):
        return linrec_amd.linrec(a * 1.0, b, True).cumsum(-1)

    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)
    y1, y0 = compiled(x, c), f(x, c)
    assert torch.equal(y1, y0)
    g1 = torch.autograd.grad(y1, (x, c), dy)
    g0 = torch.autograd.grad(y0, (x, c), dy)
    assert torch.equal(g1[0], g0[0]) and torch.equal(g1[1], g0[1])


@pytest.mark.parametrize("reverse", [False, True])
def test_logc_and_dim_options(reverse):
    """The two extra options of the reference's CPU entry point (linrec/impl/python/ops.py:8-14):
    log-coefficients and a scan axis other than the last.  The gradient with respect to the
    logarithms is d_coeffs * exp(logc) (chain rule), checked by gradcheck."""
    x, c, dy = _rand((3, 8, 5), torch.float64, 10)
    want = oracle.fwd(x.transpose(1, 2).numpy(), c.transpose(1, 2).numpy(), reverse).transpose(0, 2, 1)
    got = linrec_amd.linrec(x, c, reverse, dim=1)
    assert got.shape == x.shape
    np.testing.assert_array_equal(got.numpy(), want)
    np.testing.assert_array_equal(linrec_amd.linrec(x, c, reverse, dim=-2).numpy(), want)
    logc = torch.log(c.abs() + 0.1)
    np.testing.assert_allclose(linrec_amd.linrec(x, logc, reverse, logc=True).numpy(),
                               oracle.fwd(x.numpy(), torch.exp(logc).numpy(), reverse), rtol=1e-14)
    a = x[:, :, 0].clone().requires_grad_()
    b = logc[:, :, 0].clone().requires_grad_()
    assert torch.autograd.gradcheck(lambda p, q: linrec_amd.linrec(p, q, reverse, logc=True, dim=0), (a, b))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sixteen_bit_types_plan_and_host_path(dtype):
    """16-bit storage: slots hold eight elements, at most two slots per lane, same families."""
    names = nat.kernel_table()
    p = nat.plan(torch.empty(512, 65536 + 8, dtype=dtype))
    assert p["family"] == nat.FAMILY_STREAM and p["vec"] == 8 and p["slots"] == 2
    assert names[p["kernel_id"]].startswith("f16_" if dtype == torch.float16 else "bf16_")
    p = nat.plan(torch.empty(1000, 4096, dtype=dtype))
    assert p["family"] == nat.FAMILY_TILE and p["waves"] * p["slots"] * 64 * 8 >= 4096 and p["slots"] <= 2
    p = nat.plan(torch.empty(16, 1 << 20, dtype=dtype))
    assert p["family"] == nat.FAMILY_DRIFT and p["vec"] == 8
    p = nat.plan(torch.empty(16, (1 << 20) + 4, dtype=dtype))    # rows that are not whole slots
    assert p["family"] == nat.FAMILY_TEAM
    # rows of whole slots whose last tile is a partial one: drift teams, the backward in 8 waves of two slots
    pfx = "f16_" if dtype == torch.float16 else "bf16_"
    p = nat.plan(torch.empty(16, (1 << 20) + 8, dtype=dtype))
    assert (p["family"], p["waves"], p["slots"], p["tiles_per_row"]) == (nat.FAMILY_DRIFT, 16, 2, 65) and names[p["kernel_id"]] == pfx + "drift_ragged_w16_s2_MODE_FWD_0"
    p = nat.plan(torch.empty(16, (1 << 20) + 8, dtype=dtype), False, True)
    assert (p["family"], p["waves"], p["slots"], p["tiles_per_row"]) == (nat.FAMILY_DRIFT, 8, 2, 129) and names[p["kernel_id"]] == pfx + "drift_ragged_w8_s2_MODE_BWD_1"
    p = nat.plan(torch.empty(256, 262144, dtype=dtype).t())
    assert p["family"] == nat.FAMILY_COLUMN and p["vec"] == 4
    p = nat.plan(torch.empty(9, 100, dtype=dtype)[:, 1:])  # base one element past a slot boundary
    assert p["vec"] == 8
    # host tensors: fp32 arithmetic with one final rounding
    x, c, dy = (t.to(dtype) for t in _rand((3, 50), torch.float32, 11))
    y = linrec_amd.linrec(x, c)
    want = oracle.fwd(x.float().numpy().astype(np.float64), c.float().numpy().astype(np.float64))
    assert y.dtype == dtype
    np.testing.assert_allclose(y.float().numpy(), want, rtol=2.0 ** -7, atol=1e-2)
    dx, dc = linrec_amd.linrec_bwd(dy, c, y)
    assert dx.dtype == dtype and dc.dtype == dtype


def test_workspace_need_follows_the_phase_of_the_bases():
    """Bases that disagree modulo 16 bytes run with element-sized slots, whose tiles are a quarter
    (an eighth) of the size: a row that fits one tile otherwise is then chained through a workspace."""
    lib = nat.lib()
    f16 = nat.DTYPES[torch.float16]
    assert lib.linrec_workspace_bytes_dtype(f16, 1, 6134, 6134, 1, 6, 0, None) == 0
    assert lib.linrec_workspace_bytes_dtype(f16, 1, 6134, 6134, 1, -1, 0, None) > 0
    assert lib.linrec_workspace_bytes(1, 3000, 3000, 1, 3, 0, None) == 0
    assert lib.linrec_workspace_bytes(1, 3000, 3000, 1, -1, 0, None) > 0
    assert nat._common_phase(torch.empty(8), torch.empty(8)) == 0
    buf = torch.empty(64)
    assert nat._common_phase(buf[1:9], buf[5:13]) == 1 and nat._common_phase(buf[1:9], buf[2:10]) == -1


def test_fake_functions_serve_device_tensors_without_storage():
    """Tracing hands the fake functions device tensors that have no memory behind them: they must
    answer from sizes and strides alone (no data pointer), with the strides the real op delivers."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(4, 100, device="cuda")
        y = torch.ops.linrec_amd.linrec_fwd(x, x, False)
        assert y.shape == x.shape and y.stride() == x.stride() and y.device == x.device
        xt = torch.empty(100, 4, device="cuda", dtype=torch.bfloat16).t()
        dx, dc = torch.ops.linrec_amd.linrec_bwd(xt, xt, xt, True)
        assert dx.stride() == xt.stride() and dc.stride() == xt.stride() and dx.dtype == torch.bfloat16
        odd = torch.empty(4, 3, 100, device="cuda")[::2]  # leading dims do not collapse: dense result
        assert torch.ops.linrec_amd.linrec_fwd(odd, odd, False).is_contiguous()
        # a batch of time-major matrices is read in place: results keep its strides
        tm = torch.empty(3, 400, 24, device="cuda").transpose(1, 2)
        assert nat.row_layout(tm) is None and nat.batched_layout(tm) == (3, 24, 400, 9600, 1, 24)
        assert nat.batched_layout(torch.empty(2, 3, 400, 24, device="cuda").transpose(-1, -2)) == (6, 24, 400, 9600, 1, 24)
        assert torch.ops.linrec_amd.linrec_fwd(tm, tm, False).stride() == tm.stride()
        dx, dc = torch.ops.linrec_amd.linrec_bwd(tm, tm, tm, False)
        assert dx.stride() == tm.stride() and dc.stride() == tm.stride()
        # not read in place: channels two elements apart, batches that share memory
        wide = torch.empty(3, 400, 48, device="cuda")[:, :, ::2].transpose(1, 2)
        shared = torch.empty(1, 400, 24, device="cuda").expand(3, 400, 24).transpose(1, 2)
        for t in (wide, shared):
            assert nat.batched_layout(t) is None and not nat.kept_layout(t)
            assert torch.ops.linrec_amd.linrec_fwd(t, t, False).is_contiguous()
    assert nat.batched_layout(torch.empty(3, 400, 24).transpose(1, 2)) is None  # host tensors take the dense path


def test_caches_of_the_binding_stay_bounded(monkeypatch):
    """One workspace per (device, stream) and one remembered workspace size per layout: both are kept
    for the most recently used few only, so a long-lived process with many streams and shapes does not
    grow without bound."""
    made = []

    def fake_zeros(size, dtype, device):
        made.append(size)
        return torch.empty(size, dtype=dtype)

    monkeypatch.setattr(nat.torch, "zeros", fake_zeros)
    monkeypatch.setattr(nat, "_workspaces", type(nat._workspaces)())
    dev = torch.device("cuda", 0)
    for stream in range(3 * nat._WS_MAX_KEPT):
        nat.workspace(dev, stream, 100)
        nat.workspace(dev, 0, 100)  # stream 0 stays in use, so it is never the one dropped
    assert len(nat._workspaces) == nat._WS_MAX_KEPT
    assert (0, 0) in nat._workspaces and (0, 3 * nat._WS_MAX_KEPT - 1) in nat._workspaces
    assert made.count(nat._WS_MIN_BYTES) == 3 * nat._WS_MAX_KEPT  # stream 0 was allocated once
    ws = nat.workspace(dev, 0, nat._WS_MIN_BYTES + 1)  # growing replaces the buffer
    assert ws.numel() == 2 * nat._WS_MIN_BYTES and len(nat._workspaces) == nat._WS_MAX_KEPT
    # a workspace handed out under graph capture is never dropped (the graph keeps writing to it), and is kept
    # alive when a later launch on its stream needs a larger one
    monkeypatch.setattr(nat, "_ws_pinned", set())
    monkeypatch.setattr(nat, "_ws_retired", [])
    monkeypatch.setattr(nat, "_capturing", lambda: True)
    captured = nat.workspace(dev, 1000, 100)
    monkeypatch.setattr(nat, "_capturing", lambda: False)
    for stream in range(2000, 2000 + 2 * nat._WS_MAX_KEPT):
        nat.workspace(dev, stream, 100)
    assert nat._workspaces[(0, 1000)] is captured and len(nat._workspaces) == nat._WS_MAX_KEPT + 1
    larger = nat.workspace(dev, 1000, nat._WS_MIN_BYTES + 1)
    assert larger is not captured and any(w is captured for w in nat._ws_retired)

    monkeypatch.setattr(nat, "_need_cache", type(nat._need_cache)())
    monkeypatch.setattr(nat, "_NEED_CACHE_MAX", 8)
    monkeypatch.setattr(nat, "workspace", lambda device, stream, need: torch.empty(need, dtype=torch.uint8))
    for L in range(4096, 4096 + 40 * 4, 4):
        t = torch.empty(600, L)
        nat._workspace_for(t, 0, nat.row_layout(t), False, None, 0)
    assert len(nat._need_cache) == 8
