"""The tooling around the kernels, on the GPU: tuning sweep, attribute report, standalone driver."""
import os
import subprocess

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_tuning_sweep_checks_every_geometry_against_the_sequential_path():
    from linrec_amd import tune
    def worst(r):  # a pass a geometry is not compiled for reports nan
        return max(d for d in (r["fwd_err_vs_sequential"], r["bwd_err_vs_sequential"]) if d == d)

    rows = tune.sweep((96, 20002), iters=3, warmup=1, sets=1)  # (rows that are not whole slots: no drift kernels)
    assert len(rows) > 10
    kinds = {r["geometry"].split()[0] for r in rows}
    assert {"table", "tile", "chain", "stream"} <= kinds
    for r in rows:
        assert worst(r) <= 1e-5, r  # every geometry within the parity bar of the float64 sequential loop
        assert r["fwd_us"] > 0 and r["bwd_us"] > 0
    # rows of whole tiles: the team kernels too, the forward-only geometries with an empty backward column
    rows = tune.sweep((48, 16 * 8192), iters=3, warmup=1, sets=1)
    by = {r["geometry"]: r for r in rows}
    assert {"sweep w8 s4", "drift w8 s4", "drift w8 s2", "drift w8 s2 x16"} <= set(by), sorted(by)
    assert by["drift w8 s4"]["bwd_kernel"] == "-" and by["drift w8 s2"]["bwd_kernel"].startswith("drift_w8_s2")
    assert all(worst(r) <= 1e-5 for r in rows)
    assert [r["geometry"] for r in tune.sweep((48, 16 * 8192), iters=2, warmup=1, sets=1, only="drift w8 s2 x")] == [
        "drift w8 s2 x16"]
    rows = tune.sweep((1024, 64), transposed=True, iters=3, warmup=1, sets=1)
    assert sum(r["geometry"].startswith("column") for r in rows) >= 4
    assert all(worst(r) <= 1e-5 for r in rows)
    # 16-bit storage: the same harness, bytes counted at two per element
    rows = tune.sweep((96, 20000), iters=3, warmup=1, sets=1, dtype=torch.bfloat16)
    assert {"table", "tile", "stream", "team"} <= {r["geometry"].split()[0] for r in rows}
    assert all(worst(r) <= 2.0 ** -7 for r in rows), rows  # one bf16 rounding of the results (and of the saved outputs)


@pytest.mark.parametrize("shape,transposed", [((96, 20000), False), ((48, 16 * 8192), False), ((3000, 50), False),
                                              ((1024, 64), True), ((4096, 2048), True), ((300, 4100), True)])
def test_every_tuning_candidate_matches_the_oracle(shape, transposed):
    """The harness' own list of candidates, each forced through the C ABI and held to the parity bar against the
    float64 oracle (the harness itself checks against the library's sequential host loop)."""
    from linrec_amd import _native as nat, tune
    from tests.util import check_close, make_inputs, truth
    x, c, dy = make_inputs(shape, "uniform", seed=5, transposed=transposed)
    for reverse in (False, True):
        y_t, dx_t, dc_t = truth(x, c, dy, reverse)
        xd, cd, dyd = (t.cuda() if not transposed else t.t().contiguous().cuda().t() for t in (x, c, dy))
        yd = torch.from_numpy(y_t).float().cuda()
        if transposed:
            yd = yd.t().contiguous().t()
        ran = set()
        for label, tun in tune.candidates(xd):
            for is_bwd in (False, True):
                try:
                    pl = nat.plan(xd, reverse, is_bwd, tun)
                except (RuntimeError, NotImplementedError):
                    continue  # not compiled for this layout or pass
                if tun is not None and pl["family"] != tun.family:
                    continue
                if not is_bwd:
                    got = nat.fwd(xd, cd, reverse, tun)
                    check_close(got, y_t, f"{label} forward {shape} reverse={reverse}")
                else:
                    gx, gc = nat.bwd(dyd, cd, yd, reverse, tun)
                    check_close(gx, dx_t, f"{label} d_inputs {shape} reverse={reverse}")
                    check_close(gc, dc_t, f"{label} d_coeffs {shape} reverse={reverse}")
                ran.add(label.split()[0])
        assert "table" in ran and len(ran) >= 2, ran
    assert nat.gave_up_count() == 0


def test_write_table_measures_a_crossover_and_keeps_the_rest(tmp_path):
    """`python -m linrec_amd.tune --write-table`: the file the planner is compiled with, one threshold measured
    again here, the others kept."""
    import re
    from linrec_amd import _native as nat, tune
    path = tmp_path / "plan_thresholds.inc"
    text = tune.write_table(str(path), only=["team_min_rows"])
    assert path.read_text() == text and text.startswith(tune.TABLE_HEADER)
    got = {m.group(1): int(m.group(2)) for m in re.finditer(r"^LINREC_THRESHOLD\((\w+), (-?\d+)\)", text, flags=re.M)}
    cur = nat.plan_thresholds()
    assert set(got) == set(cur)
    assert all(got[k] == cur[k] for k in cur if k != "team_min_rows")
    x = next(c for c in tune.CROSSOVERS if c.name == "team_min_rows")
    assert x.values[0] - 1 <= got["team_min_rows"] <= x.values[-1] + 1
    assert text.count(" us against ") == len(x.values) and text.count("value kept") == len(cur) - 1


def test_launch_model_reports_the_drift_launches_of_a_shape():
    from linrec_amd import _native as nat, tune
    rows = tune.launch_model((256, 65536), sets=1, iters=3, warmup=1)
    for what in ("forward", "backward"):
        mine = [r for r in rows if r["pass"] == what]
        assert mine[0]["launch"].startswith("scan kernel drift_") and mine[-1]["launch"].startswith("streaming kernel")
        models = [r for r in mine if r["launch"].startswith("memory-only model")]
        assert len(models) >= 2 and "as the kernel" in models[0]["launch"]
        assert all(r["us"] > 0 and 0 < r["first_end_us"] <= r["mean_end_us"] <= r["last_end_us"] for r in models)
    # the model moves what it claims: every input tile added up into every output tile
    x, c = torch.randn(16, 32768, device="cuda"), torch.randn(16, 32768, device="cuda")
    out = torch.full_like(x, float("nan"))
    nat.launch_model([x, c], [out], (16, 32768), 16, 2, 4, 1, 2)
    assert torch.equal(out, x + c)
    dy, o1, o2 = torch.randn_like(x), torch.full_like(x, float("nan")), torch.full_like(x, float("nan"))
    nat.launch_model([x, c, dy], [o1, o2], (16, 32768), 16, 1, 8, 2, 2)
    assert torch.equal(o1, x + c + dy) and torch.equal(o2, o1)
    with pytest.raises(NotImplementedError):
        nat.launch_model([x, c], [out], (16, 32768), 4, 4, 4, 1, 2)


def test_memory_probe_reports_every_launch_order():
    from linrec_amd import tune
    rows = tune.memory_probe((64, 16384), sets=1, iters=3, warmup=1)
    labels = [r["blocks in flight"] for r in rows]
    assert labels[0] == "address order" and labels[1].startswith("bits 14-15 held") and "bit 17 held" in labels
    assert all(r["2_in_1_out_GBps"] > 0 and r["3_in_2_out_GBps"] > 0 for r in rows)


def test_attrs_report_lists_every_kernel_without_scratch():
    from linrec_amd import tune, _native
    rep = tune.attrs_report()
    assert len(rep) == len(_native.kernel_table())
    assert all(r["scratch_bytes"] == 0 for r in rep)


@pytest.mark.parametrize("extra", [[], ["--reverse"], ["--family", "1", "--waves", "4", "--slots", "4", "--carry", "1",
                                                        "--tasks", "2"], ["--transposed"], ["--transposed", "--reverse"]])
def test_standalone_driver(extra):
    exe = os.path.join(ROOT, "linrec_amd", "lib", "linrec_driver")
    assert os.path.exists(exe), "build it with python linrec_amd/build.py"
    out = subprocess.run([exe, "--numseq", "24", "--seqlen", "30000", "--iters", "3", *extra], capture_output=True,
                         text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    line = [l for l in out.stdout.splitlines() if l.startswith("max abs difference")][0]
    errs = [float(tok.rstrip(",")) for tok in line.replace(",", " ").split() if "e-" in tok or "e+" in tok]
    # (fp32 against fp32 in another order of operations: values reach about 10, gradients of the coefficients about 30,
    # so one unit in the last place is 1e-6 to 4e-6; observed 1e-6 / 1e-6 / 3e-6 to 6e-6)
    assert len(errs) == 3 and max(errs) < 2e-5, out.stdout
    assert "look-backs given up 0" in out.stdout or "workspace 0 bytes" in out.stdout


@pytest.mark.parametrize("shape", [(16, 200000), (40, 8192 * 12), (300, 40000), (4096, 2048), (-500, 30000), (-9000, 700)])
def test_hip_graph_replay_matches_eager(shape):
    """Forward + backward captured in a HIP graph and replayed on changing inputs: the look-back
    workspace keeps its launch counter on the device and is never cleared by a memset, so replays need
    nothing from the host.  Every replay is checked against the eager result."""
    from linrec_amd import _native
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(1)
    if shape[0] < 0:  # a transposed view: 500 rows take the three launches of the segmented column scan,
        shape = (shape[1], -shape[0])  # 9000 rows the column block kernel
        x, c, dy = (f(shape, device=dev, generator=g).t() for f in (torch.randn, torch.rand, torch.randn))
        plan = _native.plan(x)
        assert (plan["family"], plan["carry"]) == ((_native.FAMILY_SEGMENT, 0) if shape[1] == 500 else (_native.FAMILY_COLUMN, 1))
    else:
        x = torch.randn(shape, device=dev, generator=g)
        c = torch.rand(shape, device=dev, generator=g)
        dy = torch.randn(shape, device=dev, generator=g)
    y, dx, dc = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    assert y.stride() == x.stride()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up on the capture stream: allocates that stream's workspace
            _native.fwd(x, c, False, out=y)
            _native.bwd(dy, c, y, False, out=(dx, dc))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _native.fwd(x, c, False, out=y)
        _native.bwd(dy, c, y, False, out=(dx, dc))
    for rep in range(4):
        x.normal_(generator=g)
        c.uniform_(generator=g)
        dy.normal_(generator=g)
        graph.replay()
        torch.cuda.synchronize()
        got = (y.clone(), dx.clone(), dc.clone())
        ye = _native.fwd(x, c, False)
        dxe, dce = _native.bwd(dy, c, ye, False)
        torch.cuda.synchronize()
        for a, b, name in zip(got, (ye, dxe, dce), ("outputs", "d_inputs", "d_coeffs")):
            assert torch.equal(a, b), (rep, name, (a - b).abs().max().item())
    assert _native.gave_up_count() == 0


def test_streaming_calibration_kernels_move_what_they_claim():
    """The memory-only kernels the benchmark quotes as ceilings: the copy copies, the mix kernel
    stores the sum of its input streams to every output stream and nothing else."""
    from linrec_amd import _native as nat
    dev = torch.device("cuda:0")
    n = 4096 * 37 + 8  # not a whole number of workgroups
    srcs = [torch.randn(n, device=dev) for _ in range(3)]
    guard = 64
    bufs = [torch.full((n + guard,), float("nan"), device=dev) for _ in range(2)]
    dsts = [b[:n] for b in bufs]
    nat.copy(srcs[0], dsts[0])
    assert torch.equal(dsts[0], srcs[0]) and torch.isnan(bufs[0][n:]).all()
    for reads in range(0, 4):
        for writes in range(0, 3):
            if reads + writes == 0:
                continue
            for b in bufs:
                b.fill_(float("nan"))
            nat.stream_mix(srcs[:reads], dsts[:writes])
            torch.cuda.synchronize()
            want = sum(srcs[:reads]) if reads else torch.zeros(n, device=dev)
            for w in range(2):
                if w < writes:
                    assert torch.allclose(dsts[w], want, rtol=0, atol=1e-6), (reads, writes, w)
                else:
                    assert torch.isnan(dsts[w]).all(), (reads, writes, w)
                assert torch.isnan(bufs[w][n:]).all()
    with pytest.raises(RuntimeError):
        nat.check(nat.lib().linrec_stream_mix_f32(1, 1, srcs[0].data_ptr(), None, None, dsts[0].data_ptr(), None, 6, None), "mix")
    # another launch order of the 16 KiB blocks: every block still taken exactly once
    m = 4096 * 256
    a, b = torch.randn(m, device=dev), torch.randn(m, device=dev)
    for hold in [(0, 1), (0, 8), (1, 3), (3, 2), (5, 3), (7, 1)]:
        out = torch.full((m + guard,), float("nan"), device=dev)
        nat.stream_mix([a, b], [out[:m]], hold)
        assert torch.equal(out[:m], a + b) and torch.isnan(out[m:]).all(), hold
    for bad_n, hold in [(4096 * 3, (0, 1)), (4096 * 4 + 4, (0, 1)), (4096 * 4, (1, 2)), (4096 * 4, (-1, 1))]:
        with pytest.raises(RuntimeError):
            nat.check(nat.lib().linrec_stream_mix_order_f32(1, 1, a.data_ptr(), None, None, b.data_ptr(), None, bad_n,
                                                            hold[0], hold[1], None), "mix order")


@pytest.mark.parametrize("transposed", [False, True, "batched"])
def test_torch_compile_inductor_with_the_device_op(transposed):
    """The operator inside a compiled graph on the device (what the reference registers custom ops
    for, linrec/impl/cuda/ops.py:105-118): the code-generating backend fuses the elementwise work
    around it, calls the HIP kernels through the registered op, and differentiates through the
    registered backward.  Strided (transposed) inputs check that the fake functions promise the
    strides the real op delivers; "batched" is (batch, time, channels) data scanned over dim 1."""
    import linrec_amd
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    shape = (48, 3000)
    dim = -1
    if transposed == "batched":
        mk, dim = (lambda f: f((3, 400, 24), generator=g).to(dev)), 1
    elif transposed:
        mk = lambda f: f(shape[::-1], generator=g).to(dev).t()
    else:
        mk = lambda f: f(shape, generator=g).to(dev)
    x, c, dy = mk(torch.randn), mk(torch.rand), mk(torch.randn)
    x.requires_grad_()
    c.requires_grad_()

    def f(a, b):
        return torch.tanh(linrec_amd.linrec(a * 2.0, torch.sigmoid(b), reverse=True, dim=dim)) + a

    torch._dynamo.reset()
    compiled = torch.compile(f, backend="inductor", fullgraph=True)
    y1 = compiled(x, c)
    g1 = torch.autograd.grad(y1, (x, c), dy)
    y0 = f(x, c)
    g0 = torch.autograd.grad(y0, (x, c), dy)
    torch.cuda.synchronize()
    assert torch.allclose(y1, y0, rtol=1e-5, atol=1e-5)
    for a, b in zip(g1, g0):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_opcheck_on_the_device(dtype):
    """torch.library's consistency checks (schema, fake function against the real result, autograd
    registration, functionalisation) with device tensors: dense, transposed, and a batch of transposed
    matrices."""
    import linrec_amd
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    for layout in ("dense", "transposed", "batched"):
        mk = {"dense": lambda f: f((6, 700), generator=g).to(dtype).to(dev),
              "transposed": lambda f: f((700, 6), generator=g).to(dtype).to(dev).t(),
              "batched": lambda f: f((2, 300, 8), generator=g).to(dtype).to(dev).transpose(1, 2)}[layout]
        x, c, dy = mk(torch.randn), mk(torch.rand), mk(torch.randn)
        torch.library.opcheck(torch.ops.linrec_amd.linrec_fwd.default, (x, c, False))
        torch.library.opcheck(torch.ops.linrec_amd.linrec_fwd.default,
                              (x.clone().requires_grad_(), c.clone().requires_grad_(), True))
        y = linrec_amd.linrec(x, c)
        torch.library.opcheck(torch.ops.linrec_amd.linrec_bwd.default, (dy, c, y, False))


def test_two_streams_run_chained_kernels_side_by_side():
    """Launches that overlap in time must not share a workspace: the binding keeps one per stream.
    Two streams run kernels that chain their tiles through a workspace (look-back, team, sweep) at
    the same time, many times over; every result must match the one computed alone."""
    from linrec_amd import _native as nat
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    shapes = [(3, 4096 * 300), (24, 8192 * 16), (20, 100003)]
    data = [(torch.randn(s, device=dev, generator=g), torch.rand(s, device=dev, generator=g)) for s in shapes]
    # and the segmented column scan, whose maps live in the same per-stream workspace
    data.append(tuple(f((50000, 96), device=dev, generator=g).t() for f in (torch.randn, torch.rand)))
    want = [nat.fwd(x, c) for x, c in data]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.empty_like(x) for x, _ in data] for _ in streams]
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
    for rep in range(10):
        for k, st in enumerate(streams):
            with torch.cuda.stream(st):
                for i, (x, c) in enumerate(data):
                    nat.fwd(x, c, out=outs[k][i])
    torch.cuda.synchronize()
    for k in range(2):
        for i in range(len(data)):
            assert torch.equal(outs[k][i], want[i]), (k, i)
    assert nat.gave_up_count() == 0
    assert len({ptr for (_, ptr) in nat._workspaces}) >= 3  # default stream and the two side streams
