"""GPU test of linrec_fwd_noalloc, the entry point for callers that cannot allocate device memory: through
the C ABI its results must equal linrec_fwd's bit for bit (same kernels, the library's static scratch
array in place of a caller-owned workspace), call after call on the same GPU, also when a later call is
smaller than the one before and so finds the previous call's descriptors in the array."""
import ctypes

import numpy as np
import pytest
import torch

from linrec_amd import _native as nat
from oracle import oracle

pytestmark = pytest.mark.gpu


def _pair(shape, seed, transposed=False):
    g = torch.Generator().manual_seed(seed)
    if transposed:
        x = torch.randn(shape[::-1], generator=g).cuda().t()
        c = torch.rand(shape[::-1], generator=g).cuda().t()
    else:
        x = torch.randn(shape, generator=g).cuda()
        c = torch.rand(shape, generator=g).cuda()
    return x, c


def _both(x, c, reverse):
    """(result of linrec_fwd with a workspace of its own, result of linrec_fwd_noalloc)"""
    lib = nat.lib()
    lay = nat.row_layout(x)
    assert lay is not None
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full_like(x, float("nan"))
    got = torch.full_like(x, float("nan"))
    need = lib.linrec_workspace_bytes_dtype(nat.DTYPES[x.dtype], *lay, 0, 0, None)
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=x.device)
    rc = lib.linrec_fwd(nat.DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), want.data_ptr(), *lay, int(reverse),
                        ws.data_ptr(), ws.numel(), None, stream)
    assert rc == 0, rc
    rc = lib.linrec_fwd_noalloc(nat.DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), got.data_ptr(), *lay, int(reverse),
                                None, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return want, got, need


def test_noalloc_forward_equals_forward_with_a_workspace_call_after_call():
    # each of these launches keeps state in the scratch: teams that go from row to row (16 rows), look-back
    # tiles (3 rows, then 1 row), one team per row (8 ragged rows), segments of a strided scan axis, teams along
    # a strided scan axis (4096 rows)
    cases = [((16, 131072), False, False), ((3, 40000), True, False), ((1, 9000), False, False),
             ((8, 70001), False, False), ((16, 65536), True, False), ((1024, 4096), False, True),
             ((4096, 2048), True, True), ((2, 20000), False, False)]
    used_scratch = 0
    for i, (shape, reverse, transposed) in enumerate(cases):
        print("noalloc case", i, shape, reverse, transposed, flush=True)
        x, c = _pair(shape, 100 + i, transposed)
        want, got, need = _both(x, c, reverse)
        used_scratch += need > 0
        assert not torch.isnan(got).any()
        assert torch.equal(want, got), (shape, (want - got).abs().max().item())
    assert used_scratch >= 7
    # the small last case also against the float64 recurrence (bar: 1e-5 normwise, as everywhere)
    truth = oracle.fwd(x.cpu().numpy(), c.cpu().numpy(), False, dtype=np.float64)
    assert oracle.error_report(got.cpu().numpy(), truth)["normwise"] <= 1e-5
    assert nat.gave_up_count() == 0
    # the waits of the launches on the static array are counted in its own header
    assert nat.lib().linrec_noalloc_gave_up_count() == 0


def test_noalloc_forward_of_16_bit_storage_and_kernels_without_scratch():
    lib = nat.lib()
    stream = torch.cuda.current_stream().cuda_stream
    for dtype, shape in ((torch.bfloat16, (16, 131072)), (torch.float16, (4, 50000)), (torch.float32, (64, 4096))):
        g = torch.Generator().manual_seed(7)
        x = torch.randn(shape, generator=g).to(dtype).cuda()
        c = torch.rand(shape, generator=g).to(dtype).cuda()
        lay = nat.row_layout(x)
        got = torch.full_like(x, float("nan"))
        assert lib.linrec_fwd_noalloc(nat.DTYPES[dtype], x.data_ptr(), c.data_ptr(), got.data_ptr(), *lay, 0, None,
                                      stream) == 0
        want = nat.fwd(x, c)
        torch.cuda.synchronize()
        assert torch.equal(want, got), (dtype, shape)
        # ... and against the float64 recurrence on the same rounded inputs: one rounding of the storage type
        truth = oracle.fwd(x.float().cpu().numpy(), c.float().cpu().numpy(), False, dtype=np.float64)
        ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 1e-5}[dtype]
        assert oracle.error_report(got.float().cpu().numpy(), truth)["normwise"] <= ulp, (dtype, shape)
    assert lib.linrec_noalloc_gave_up_count() == 0


def test_noalloc_forward_under_graph_capture_and_replay():
    """What the entry point is for: it is recorded into a HIP graph (after one call outside the capture, which looks
    up the static array's address) and replayed, with the program's own launches and synchronisations in between,
    and every replay must give the float64 recurrence's result."""
    lib = nat.lib()
    # (the last: bf16, the forward whose scanned tiles wait in 128 KB of LDS)
    for shape, reverse, dtype in (((16, 131072), False, torch.float32), ((3, 40000), True, torch.float32),
                                  ((32, 262144), False, torch.bfloat16)):
        x, c = (t.to(dtype) for t in _pair(shape, 11))
        if dtype == torch.bfloat16:
            assert nat.plan(x)["family"] == nat.FAMILY_DRIFT and nat.plan(x)["slots"] == 2
        lay = nat.row_layout(x)
        out = torch.full_like(x, float("nan"))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            assert lib.linrec_fwd_noalloc(nat.DTYPES[dtype], x.data_ptr(), c.data_ptr(), out.data_ptr(), *lay, int(reverse),
                                          None, side.cuda_stream) == 0  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = lib.linrec_fwd_noalloc(nat.DTYPES[dtype], x.data_ptr(), c.data_ptr(), out.data_ptr(), *lay, int(reverse),
                                        None, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        # (nothing the size of a workspace was allocated by the capture: the graph itself takes a few hundred KB)
        assert torch.cuda.mem_get_info()[0] >= free_before - (8 << 20)
        for rep in range(3):
            xs, cs = (t.to(dtype) for t in _pair(shape, 20 + rep))
            x.copy_(xs)
            c.copy_(cs)
            out.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            truth = oracle.fwd(x.float().cpu().numpy(), c.float().cpu().numpy(), reverse, dtype=np.float64)
            bar = 1e-5 if dtype == torch.float32 else 2.0 ** -8  # (one rounding of the storage type)
            assert oracle.error_report(out.float().cpu().numpy(), truth)["normwise"] <= bar, (shape, rep)
            nat.fwd(xs, cs, reverse)  # (the program's own eager work between the replays)
        del graph
    assert lib.linrec_noalloc_gave_up_count() == 0


def test_noalloc_takes_another_kernel_where_the_usual_choice_needs_more_scratch_than_there_is():
    """16384 timesteps x 4096 channels: linrec_fwd takes teams along the scan axis, whose per-step maps need
    17 MB of workspace; the entry point that allocates nothing serves the call with the kernels that need none
    instead of turning it down."""
    lib = nat.lib()
    x, c = _pair((4096, 16384), 5, transposed=True)
    lay = nat.row_layout(x)
    need = lib.linrec_workspace_bytes_dtype(nat.DTYPES[x.dtype], *lay, 0, 0, None)
    assert nat.plan(x)["family"] == nat.FAMILY_COLDRIFT and need > (4 << 20)
    got = torch.full_like(x, float("nan"))
    rc = lib.linrec_fwd_noalloc(nat.DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), got.data_ptr(), *lay, 0, None,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 63, 64, 2047, 4095], device=x.device)
    truth = oracle.fwd(x.index_select(0, rows).cpu().numpy(), c.index_select(0, rows).cpu().numpy(), False, dtype=np.float64)
    assert not torch.isnan(got).any()
    assert oracle.error_report(got.index_select(0, rows).cpu().numpy(), truth)["normwise"] <= 1e-5
    # a tuning that insists on the kernel that does not fit is turned down
    t = nat.Tuning(nat.FAMILY_COLDRIFT)
    assert lib.linrec_fwd_noalloc(nat.DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), got.data_ptr(), *lay, 0,
                                  ctypes.byref(t), torch.cuda.current_stream().cuda_stream) == -5


@pytest.mark.parametrize("shape", [(33000, 32768), (20001, 65536)])
def test_noalloc_serves_many_long_rows_with_one_workgroup_per_row(shape):
    """Tens of thousands of rows of 32768 elements: linrec_fwd takes teams that go from row to row, whose per-tile maps
    need more than the 4 MiB there are; the entry point that allocates nothing walks every row with one workgroup."""
    lib = nat.lib()
    x, c = _pair(shape, 6)
    lay = nat.row_layout(x)
    need = lib.linrec_workspace_bytes_dtype(nat.DTYPES[x.dtype], *lay, 0, 0, None)
    assert nat.plan(x)["family"] in (nat.FAMILY_DRIFT, nat.FAMILY_SWEEP) and need > (4 << 20)
    got = torch.full_like(x, float("nan"))
    rc = lib.linrec_fwd_noalloc(nat.DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), got.data_ptr(), *lay, 0, None,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    want = nat.fwd(x, c)
    torch.cuda.synchronize()
    assert not torch.isnan(got).any()
    pl = nat.Plan()
    assert lib.linrec_plan_noalloc(0, x.data_ptr(), *lay, 0, None, ctypes.byref(pl)) == 0
    assert pl.family == nat.FAMILY_STREAM and pl.workspace_bytes == 0
    rows = torch.tensor([0, 1, 255, 256, 9999, shape[0] - 1], device=x.device)
    truth = oracle.fwd(x.index_select(0, rows).cpu().numpy(), c.index_select(0, rows).cpu().numpy(), False, dtype=np.float64)
    assert oracle.error_report(got.index_select(0, rows).cpu().numpy(), truth)["normwise"] <= 1e-5
    assert oracle.error_report(want.index_select(0, rows).cpu().numpy(), truth)["normwise"] <= 1e-5
