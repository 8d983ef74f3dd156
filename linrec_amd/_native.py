"""ctypes binding of the C ABI declared in include/linrec_hip.h.

Takes the place of the reference's pybind11 module (linrec/impl/cuda/extension.cpp:36-72): it
passes data pointers, sizes, strides and the current HIP stream; outputs and the look-back
workspace are allocated here with torch so that they are stream-ordered like any other tensor.
There is no fallback: if the shared library is missing, every call raises.
"""
import collections
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblinrec_hip.so")

FAMILY_AUTO, FAMILY_TILE, FAMILY_COLUMN, FAMILY_NAIVE, FAMILY_STREAM, FAMILY_TEAM, FAMILY_SWEEP, FAMILY_GROUP = 0, 1, 2, 3, 4, 5, 6, 7
FAMILY_SEGMENT = 8
FAMILY_FLAT = 9
FAMILY_DRIFT = 10
FAMILY_COLDRIFT = 11


DTYPES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}  # LINREC_DTYPE_*


def _phase(t):
    """Misalignment of t's base address in elements, modulo one 16-byte slot."""
    size = t.element_size()
    return (t.data_ptr() // size) % (16 // size)


def _common_phase(*tensors):
    """The phase all tensors of a call share, or -1: the kernels then fall back to element-sized
    accesses, and the launch planner has to be asked about that case."""
    first = _phase(tensors[0])
    for t in tensors[1:]:
        if _phase(t) != first:
            return -1
    return first


class Tuning(ctypes.Structure):
    """linrec_tuning_t: per-call override of the built-in launch table."""
    _fields_ = [("family", ctypes.c_int32), ("waves", ctypes.c_int32),
                ("slots", ctypes.c_int32), ("carry", ctypes.c_int32), ("tasks", ctypes.c_int32)]

    def __init__(self, family=FAMILY_AUTO, waves=0, slots=0, carry=-1, tasks=0):
        super().__init__(family, waves, slots, carry, tasks)


class Plan(ctypes.Structure):
    """linrec_plan_t"""
    _fields_ = [("family", ctypes.c_int32), ("waves", ctypes.c_int32), ("slots", ctypes.c_int32),
                ("vec", ctypes.c_int32), ("carry", ctypes.c_int32), ("tiles_per_row", ctypes.c_int32),
                ("tasks", ctypes.c_int32), ("tail_rows", ctypes.c_int32), ("grid", ctypes.c_int64), ("block", ctypes.c_int32), ("kernel_id", ctypes.c_int32),
                ("workspace_bytes", ctypes.c_uint64)]

    def asdict(self):
        return {name: getattr(self, name) for name, _ in self._fields_}


class Call(ctypes.Structure):
    """linrec_call_t: the arguments of linrec_fwd_call / linrec_bwd_call in one block of memory."""
    _fields_ = [("dtype", ctypes.c_int32), ("reverse", ctypes.c_int32), ("numseq", ctypes.c_int64),
                ("seqlen", ctypes.c_int64), ("row_stride", ctypes.c_int64), ("elem_stride", ctypes.c_int64),
                ("in0", ctypes.c_void_p), ("coef", ctypes.c_void_p), ("aux", ctypes.c_void_p),
                ("out0", ctypes.c_void_p), ("out1", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("workspace_bytes", ctypes.c_uint64), ("stream", ctypes.c_void_p)]


_lib = None
_lib_lock = threading.Lock()


def _declare(lib):
    i64, i32, p, sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
    tun, plan = ctypes.POINTER(Tuning), ctypes.POINTER(Plan)
    sigs = {
        "linrec_hip_abi_version": (i32, []),
        "linrec_hip_error_string": (ctypes.c_char_p, [i32]),
        "linrec_fwd": (i32, [i32, p, p, p, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_bwd": (i32, [i32, p, p, p, p, p, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_plan": (i32, [i32, p, i64, i64, i64, i64, i32, i32, tun, plan]),
        "linrec_workspace_bytes_dtype": (sz, [i32, i64, i64, i64, i64, i32, i32, tun]),
        "linrec_fwd_f32": (i32, [p, p, p, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_bwd_f32": (i32, [p, p, p, p, p, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_workspace_bytes": (sz, [i64, i64, i64, i64, i32, i32, tun]),
        "linrec_workspace_bytes_for_tiles": (sz, [i64]),
        "linrec_plan_f32": (i32, [p, i64, i64, i64, i64, i32, i32, tun, plan]),
        "linrec_set_spin_limit": (i32, [i32]),
        "linrec_compute_units": (i32, []),
        "linrec_set_compute_units": (i32, [i32]),
        "linrec_fwd_noalloc": (i32, [i32, p, p, p, i64, i64, i64, i64, i32, tun, p]),
        "linrec_fwd_call": (i32, [ctypes.POINTER(Call)]),
        "linrec_bwd_call": (i32, [ctypes.POINTER(Call)]),
        "linrec_noalloc_gave_up_count": (i32, []),
        "linrec_plan_noalloc": (i32, [i32, p, i64, i64, i64, i64, i32, tun, plan]),
        "linrec_plan_threshold_count": (i32, []),
        "linrec_plan_threshold_name": (ctypes.c_char_p, [i32]),
        "linrec_plan_threshold_value": (i64, [i32]),
        "linrec_kernel_count": (i32, []),
        "linrec_kernel_name": (ctypes.c_char_p, [i32]),
        "linrec_kernel_attrs": (i32, [i32] + [ctypes.POINTER(ctypes.c_int)] * 4),
        "linrec_copy_f32": (i32, [p, p, i64, p]),
        "linrec_stream_mix_f32": (i32, [i32, i32, p, p, p, p, p, i64, p]),
        "linrec_stream_mix_order_f32": (i32, [i32, i32, p, p, p, p, p, i64, i32, i32, p]),
        "linrec_launch_model_f32": (i32, [i32, i32, p, p, p, p, p, i64, i64, i32, i32, i32, i32, i32, p, p]),
        "linrec_transpose": (i32, [i32, p, p, i64, i64, i64, p]),
        "linrec_fwd_batched": (i32, [i32, p, p, p, i64, i64, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_bwd_batched": (i32, [i32, p, p, p, p, p, i64, i64, i64, i64, i64, i64, i32, p, sz, tun, p]),
        "linrec_plan_batched": (i32, [i32, p, i64, i64, i64, i64, i64, i64, i32, i32, tun, ctypes.POINTER(Plan)]),
        "linrec_host_fwd_f32": (i32, [p, p, p, i64, i64, i64, i64, i32]),
        "linrec_host_fwd_f64": (i32, [p, p, p, i64, i64, i64, i64, i32]),
        "linrec_host_bwd_f32": (i32, [p, p, p, p, p, i64, i64, i64, i64, i32]),
        "linrec_host_bwd_f64": (i32, [p, p, p, p, p, i64, i64, i64, i64, i32]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype, fn.argtypes = res, args
    return sigs


EXPORTS = None


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib, EXPORTS
    if _lib is None:
        with _lib_lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is missing: build it with `python linrec_amd/build.py` "
                        "(needs hipcc; there is no fallback implementation for device tensors)")
                handle = ctypes.CDLL(LIB_PATH)
                EXPORTS = _declare(handle)
                _lib = handle
    return _lib


def check(code, what):
    if code:
        msg = lib().linrec_hip_error_string(code).decode()
        if code == -3:
            raise NotImplementedError(f"{what}: {msg}")
        raise RuntimeError(f"{what}: {msg} (code {code})")


# ---- tensor layout -----------------------------------------------------------------------------
def row_layout(t):
    """(numseq, seqlen, row_stride, elem_stride) if `t` is a set of uniformly strided rows along
    its last dim, else None.  Leading dims must collapse into one (as they do for any dense or
    row-padded tensor and for a transposed matrix), and no two elements may share an address
    (results are allocated with the same strides): rows of whole elements side by side, or elements
    of whole rows side by side."""
    if t.dim() == 0:
        return None
    L = t.size(-1)
    numseq = t.numel() // L if L else 0
    es = t.stride(-1) if L > 1 else 1
    sizes, strides = list(t.shape[:-1]), list(t.stride()[:-1])
    dims = [(n, s) for n, s in zip(sizes, strides) if n != 1]
    if not dims:
        return (numseq, L, max(L, 1), es) if es > 0 or L == 0 else None
    for (n0, s0), (n1, s1) in zip(dims[:-1], dims[1:]):
        if s0 != s1 * n1:
            return None
    rs = dims[-1][1]
    if L and not ((es > 0 and rs >= es * L) or (rs > 0 and es >= rs * numseq)):
        return None  # rows or elements overlap (expanded tensors and the like)
    return numseq, L, rs, es


def batched_layout(t):
    """(batches, rows_per_batch, seqlen, batch_stride, row_stride, elem_stride) for a device tensor that
    is a batch of matrices with a strided scan axis whose rows are not uniformly strided as a whole
    ((batch, time, channels) data seen as (batch, channels, time)), else None.  Leading dims must
    collapse into the one batch dim; no two elements may share an address."""
    if not t.is_cuda or t.dtype not in DTYPES or t.dim() < 3 or t.numel() == 0 or row_layout(t) is not None:
        return None
    L, es = t.size(-1), t.stride(-1)
    C, rs = t.size(-2), t.stride(-2)
    if L == 1 or es == 1 or C == 1 or rs != 1:
        return None  # (rows further apart than one element are left to the dense path)
    lead = [(n, st) for n, st in zip(t.shape[:-2], t.stride()[:-2]) if n != 1]
    if not lead:
        return None
    for (n0, s0), (n1, s1) in zip(lead[:-1], lead[1:]):
        if s0 != s1 * n1:
            return None
    B, bs = t.numel() // (L * C), lead[-1][1]
    extents = sorted([(bs, B), (rs, C), (es, L)])
    if extents[0][0] <= 0:
        return None
    for (s0, n0), (s1, _) in zip(extents[:-1], extents[1:]):
        if s1 < s0 * n0:
            return None  # dims overlap in memory
    return B, C, L, bs, rs, es


def kept_layout(t):
    """True if the kernels read `t` as it lies in memory (results then get its strides); False if it
    is first copied into dense rows."""
    return row_layout(t) is not None or batched_layout(t) is not None


def output_like(t, fake=False):
    """Allocation for results: same sizes and strides as `t` when it is a set of uniformly strided
    rows (so dense inputs get exactly torch.empty_like, linrec/impl/cuda/linrec_pipe.cu:31),
    contiguous otherwise.  `fake`: called for a tensor without storage (tracing); sizes and
    strides are what matters there."""
    if row_layout(t) is None:
        if batched_layout(t) is not None:
            return torch.empty_strided(t.size(), t.stride(), dtype=t.dtype, device=t.device)
        return torch.empty(t.size(), dtype=t.dtype, device=t.device)
    if t.numel() > 0:
        phase = _phase(t) if t.is_cuda and not fake else 0
        if phase == 0:
            return torch.empty_strided(t.size(), t.stride(), dtype=t.dtype, device=t.device)
        # A view that starts inside a 16-byte slot: give the result the same phase, so that the
        # kernels keep their 16-byte accesses (torch's allocations start on a slot boundary).
        span = 1 + sum((n - 1) * abs(st) for n, st in zip(t.size(), t.stride()))
        buf = torch.empty(span + phase, dtype=t.dtype, device=t.device)
        return buf.as_strided(t.size(), t.stride(), phase)
    return torch.empty(t.size(), dtype=t.dtype, device=t.device)


# ---- look-back workspace, one per (device, stream) ---------------------------------------------
_workspaces = collections.OrderedDict()  # (device index, stream handle) -> buffer, least recently used first
_ws_pinned = set()           # keys whose workspace a graph capture has been given: never dropped
_ws_retired = []             # buffers a captured graph may still write to, outgrown since
_ws_gave_up_of_dropped = {}  # device index -> waits that ran out, counted in workspaces since dropped
_ws_lock = threading.Lock()
_WS_MIN_BYTES = 1 << 20
_WS_MAX_KEPT = 16  # (device, stream) pairs whose workspace is kept; a process rarely launches from more


def _capturing():
    """True while the current stream is being captured into a graph."""
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def workspace(device, stream_ptr, nbytes):
    """Zero-initialised scratch owned by the kernels' look-back chain.  Kept per stream because two
    launches that overlap in time must not share descriptors; grown (and re-zeroed) on demand.
    A workspace handed out while its stream is being captured into a graph stays for good: the graph has
    its address baked in and every replay writes descriptors there, so such a buffer is neither dropped with
    the least recently used ones nor freed when a later launch on the stream needs a larger one."""
    key = (device.index, stream_ptr)
    with _ws_lock:
        capturing = _capturing()
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            size = max(_WS_MIN_BYTES, 1 << (int(nbytes) - 1).bit_length())
            if ws is not None and key in _ws_pinned:
                _ws_retired.append(ws)
                _ws_pinned.discard(key)
            ws = torch.zeros(size, dtype=torch.uint8, device=device)
            _workspaces[key] = ws
            # Streams come and go (their handles are even reused); the workspaces of the ones not
            # launched from for longest are dropped.  A dropped buffer goes back to torch's allocator,
            # which hands it out again in the order of the stream it was allocated on: the one its
            # kernels were queued on.
            if not capturing:
                droppable = [k for k in _workspaces if k not in _ws_pinned and k != key]
                while len(_workspaces) - len(_ws_pinned) > _WS_MAX_KEPT and droppable:
                    old = droppable.pop(0)
                    gone = _workspaces.pop(old)
                    # (what it counted is kept; reading it synchronises, which is allowed outside a capture)
                    if gone.is_cuda:
                        _ws_gave_up_of_dropped[old[0]] = _ws_gave_up_of_dropped.get(old[0], 0) + int(gone[:16].view(torch.int32)[1].item())
        if capturing:
            _ws_pinned.add(key)
        _workspaces.move_to_end(key)
        return ws


def _same_layout(ref, *others):
    return all(o.size() == ref.size() and o.stride() == ref.stride() for o in others)


def _as_transposed_matrices(t):
    """(batch, rows, cols) if `t`'s memory is `batch` dense row-major rows x cols matrices of which
    `t` shows the transposes (its scan axis is then the strided one), else None."""
    if not (t.is_cuda and t.dtype in DTYPES and t.numel()):
        return None
    if t.dim() >= 2 and t.transpose(-1, -2).is_contiguous():
        return t.numel() // (t.size(-1) * t.size(-2)), t.size(-1), t.size(-2)
    lay = row_layout(t)
    if lay is not None and lay[2] == 1 and lay[3] == lay[0]:
        return 1, lay[1], lay[0]  # leading dims collapse into the rows of one transposed matrix
    return None


def _transpose(src, dst, batch, rows, cols):
    def go(stream):
        check(lib().linrec_transpose(src.element_size(), src.data_ptr(), dst.data_ptr(), batch, rows, cols, stream),
              "linrec_transpose")
    _on_device(src, go)


def _dense(t):
    """`t`'s values in a dense row-major tensor (`t` itself if it is one)."""
    if t.is_contiguous():
        return t
    m = _as_transposed_matrices(t)
    if m is None:
        return t.contiguous()
    out = torch.empty(t.size(), dtype=t.dtype, device=t.device)
    _transpose(t, out, *m)
    return out


def _assign(dst, src):
    """dst[...] = src for a dense `src` of the same sizes."""
    m = _as_transposed_matrices(dst)
    if m is None or not src.is_contiguous() or src.dtype != dst.dtype or src.device != dst.device:
        dst.copy_(src)
    else:
        _transpose(src, dst, m[0], m[2], m[1])
    return dst


def _restride(t, like):
    """`t`'s values in the memory layout of `like`."""
    if like.is_contiguous():
        return _dense(t)
    out = torch.empty_strided(like.size(), like.stride(), dtype=t.dtype, device=t.device)
    out.copy_(t)
    return out


def plan(t, reverse=False, is_bwd=False, tuning=None):
    """The launch the library would make for a tensor of this layout (dict), or None if `t` would
    first be copied to a dense layout."""
    lay = row_layout(t)
    p = Plan()
    tun = ctypes.byref(tuning) if tuning is not None else None
    if lay is None:
        bl = batched_layout(t)
        if bl is None:
            return None
        check(lib().linrec_plan_batched(DTYPES[t.dtype], t.data_ptr(), *bl, int(reverse), int(is_bwd), tun,
                                        ctypes.byref(p)), "linrec_plan_batched")
        return p.asdict()
    check(lib().linrec_plan(DTYPES[t.dtype], t.data_ptr(), *lay, int(reverse), int(is_bwd), tun, ctypes.byref(p)),
          "linrec_plan")
    return p.asdict()


try:  # the stream handle without building a Stream object (a few microseconds per call)
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover
    def _raw_stream(index):
        return torch.cuda.current_stream(index).cuda_stream

_need_cache = collections.OrderedDict()  # (device, dtype, layout, phase, pass) -> workspace bytes, least recent first
_NEED_CACHE_MAX = 1024


def set_compute_units(cus):
    """Overrides the compute-unit count the planner sizes its launches by (0: ask the device again) and
    forgets the workspace sizes remembered for the count in force before (those of other threads' repeat calls
    are forgotten when those threads next look: the override is a testing aid).  Returns the previous override."""
    old = lib().linrec_set_compute_units(cus)
    if cus >= 0:
        _need_cache.clear()
        _repeat_table().clear()
    return old


def _workspace_for(t, phase, lay, is_bwd, tun, stream):
    """(pointer, bytes) of the workspace this call needs, (None, 0) for kernels without one.
    `phase`: common misalignment of all tensors of the call, -1 if they disagree."""
    key = (t.device.index, t.dtype, lay, phase, is_bwd) if tun is None else None
    need = _need_cache.get(key) if key is not None else None
    if need is None:
        need = lib().linrec_workspace_bytes_dtype(DTYPES[t.dtype], *lay, phase, is_bwd, tun)
        if key is not None:
            _need_cache[key] = need
            while len(_need_cache) > _NEED_CACHE_MAX:
                _need_cache.popitem(last=False)
    elif key is not None:
        try:
            _need_cache.move_to_end(key)
        except KeyError:  # another thread's insertion pushed it out meanwhile
            pass
    if not need:
        return None, 0
    ws = workspace(t.device, stream, need)
    return ws.data_ptr(), ws.numel()


def _on_device(t, fn):
    """Run fn(stream) with t's device current (the launch uses the current device)."""
    idx = t.device.index
    if torch.cuda.current_device() == idx:
        return fn(_raw_stream(idx))
    with torch.cuda.device(idx):
        return fn(_raw_stream(idx))


def _launch_fwd(x, c, y, lay, reverse, tuning):
    L = lib()
    tun = ctypes.byref(tuning) if tuning is not None else None
    if x.is_cuda:
        def go(stream):
            ws_ptr, ws_len = _workspace_for(x, _common_phase(x, c, y), lay, 0, tun, stream)
            check(L.linrec_fwd(DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), y.data_ptr(), *lay, int(reverse),
                               ws_ptr, ws_len, tun, stream), "linrec_fwd")
        _on_device(x, go)
    else:
        fn = L.linrec_host_fwd_f32 if x.dtype == torch.float32 else L.linrec_host_fwd_f64
        check(fn(x.data_ptr(), c.data_ptr(), y.data_ptr(), *lay, int(reverse)), "linrec_host_fwd")


def _launch_bwd(dy, c, y, dx, dc, lay, reverse, tuning):
    L = lib()
    tun = ctypes.byref(tuning) if tuning is not None else None
    if dy.is_cuda:
        def go(stream):
            ws_ptr, ws_len = _workspace_for(dy, _common_phase(dy, c, y, dx, dc), lay, 1, tun, stream)
            check(L.linrec_bwd(DTYPES[dy.dtype], dy.data_ptr(), c.data_ptr(), y.data_ptr(), dx.data_ptr(),
                               dc.data_ptr(), *lay, int(reverse), ws_ptr, ws_len, tun, stream), "linrec_bwd")
        _on_device(dy, go)
    else:
        fn = L.linrec_host_bwd_f32 if dy.dtype == torch.float32 else L.linrec_host_bwd_f64
        check(fn(dy.data_ptr(), c.data_ptr(), y.data_ptr(), dx.data_ptr(), dc.data_ptr(), *lay,
                 int(reverse)), "linrec_host_bwd")


def _batched_workspace(t, ptr_for_phase, bl, is_bwd, tun, stream):
    """Workspace of a batched launch, sized by the plan the library makes for it."""
    p = Plan()
    check(lib().linrec_plan_batched(DTYPES[t.dtype], ptr_for_phase, *bl, 0, is_bwd, tun, ctypes.byref(p)),
          "linrec_plan_batched")
    if not p.workspace_bytes:
        return None, 0
    ws = workspace(t.device, stream, p.workspace_bytes)
    return ws.data_ptr(), ws.numel()


def _launch_fwd_batched(x, c, y, bl, reverse, tuning):
    L = lib()
    tun = ctypes.byref(tuning) if tuning is not None else None

    def go(stream):
        # rows per lane depend on the common phase of the bases: plan with a pointer of that phase
        phase = _common_phase(x, c, y)
        probe = x.data_ptr() if phase >= 0 else x.data_ptr() | x.element_size()
        ws_ptr, ws_len = _batched_workspace(x, probe, bl, 0, tun, stream)
        check(L.linrec_fwd_batched(DTYPES[x.dtype], x.data_ptr(), c.data_ptr(), y.data_ptr(), *bl, int(reverse),
                                   ws_ptr, ws_len, tun, stream), "linrec_fwd_batched")
    _on_device(x, go)


def _launch_bwd_batched(dy, c, y, dx, dc, bl, reverse, tuning):
    L = lib()
    tun = ctypes.byref(tuning) if tuning is not None else None

    def go(stream):
        phase = _common_phase(dy, c, y, dx, dc)
        probe = dy.data_ptr() if phase >= 0 else dy.data_ptr() | dy.element_size()
        ws_ptr, ws_len = _batched_workspace(dy, probe, bl, 1, tun, stream)
        check(L.linrec_bwd_batched(DTYPES[dy.dtype], dy.data_ptr(), c.data_ptr(), y.data_ptr(), dx.data_ptr(),
                                   dc.data_ptr(), *bl, int(reverse), ws_ptr, ws_len, tun, stream), "linrec_bwd_batched")
    _on_device(dy, go)


def _validate(first, *rest, names):
    # same conditions as the reference's launcher (linrec/impl/cuda/linrec_pipe.cu:17-22)
    for t, name in zip(rest, names[1:]):
        if t.size() != first.size():
            raise RuntimeError(f"linrec: {name} has size {tuple(t.size())}, {names[0]} has {tuple(first.size())}")
        if t.device != first.device:
            raise RuntimeError(f"linrec: {name} is on {t.device}, {names[0]} on {first.device}")
        if t.dtype != first.dtype:
            raise RuntimeError(f"linrec: {name} has dtype {t.dtype}, {names[0]} has {first.dtype}")
    if first.dim() == 0:
        raise RuntimeError("linrec: tensors need at least one dimension (the scan runs over the last)")
    if first.is_cuda:
        if first.dtype not in DTYPES:
            raise RuntimeError(f"linrec: device tensors must be float32, float16 or bfloat16, got {first.dtype}")
    elif first.dtype not in (torch.float32, torch.float64, torch.float16, torch.bfloat16):
        raise RuntimeError(f"linrec: host tensors must be a floating-point type, got {first.dtype}")


def gave_up_count(device=None):
    """Waits for another workgroup that hit the poll limit, summed over this process's workspaces on
    `device` (synchronises).  The results are valid whatever the count (a wave whose wait runs out computes
    what it was waiting for from the row's own data); non-zero says that launches were slow."""
    want = None if device is None else torch.device(device).index
    with _ws_lock:
        items = list(_workspaces.items())
        total = sum(n for idx, n in _ws_gave_up_of_dropped.items() if want in (None, idx))
    for key, ws in items:
        if want in (None, key[0]):
            total += int(ws[:16].view(torch.int32)[1].item())
    return total


# Scan axis strided, few rows, and the rows not adjacent in memory (say every other row of a transposed
# matrix): the only kernel that reads such a layout gives every lane a row and walks the scan axis
# step by step, which leaves the chip idle (about 70 ns per step however few the rows).  Below this
# many rows the tensors are re-laid out with rows on the unit-stride axis, scanned there, and the
# results copied back into the caller's layout (the reference makes the same kind of copy for
# d_outputs, linrec/impl/cuda/ops.py:96).  Adjacent rows need none of this: the library cuts their
# scan axis into segments (LINREC_FAMILY_SEGMENT).
_STRIDED_AXIS_MIN_ROWS = 8192

_RELAYOUT_UNIT_ROW_STRIDE = False  # tests and measurements: re-lay out adjacent rows as well


def _few_rows_on_strided_axis(t, lay, tuning):
    if not (t.is_cuda and tuning is None and lay[3] != 1 and lay[1] > 1 and lay[0] < _STRIDED_AXIS_MIN_ROWS):
        return False
    return _RELAYOUT_UNIT_ROW_STRIDE or (lay[2] != 1 and lay[0] != 1)


# ---- repeat calls ------------------------------------------------------------------------------
# A call on device tensors whose sizes, strides, types and devices have been seen before (on this thread) skips
# everything that only depends on those: validation, the layout, the workspace size; what is left is the
# pointers (which must be 16-byte aligned, as the results then are), the stream and one library call that takes
# its arguments in one block of memory.  On a 64 x 4096 tensor, whose kernel takes 3 us, this halves the time
# the host needs per launch.  Everything else takes the general path below.
_repeat = threading.local()
_REPEAT_MAX = 256


def _repeat_table():
    table = getattr(_repeat, "table", None)
    if table is None:
        table = _repeat.table = {}
    return table


def _remember(table, key, lay, t, is_bwd, reverse):
    """What a repeat of the call `key` needs: (Call, reference to it, workspace bytes), or None if calls of
    this kind take the general path."""
    entry = None
    if lay is not None:
        call = Call(dtype=DTYPES[t.dtype], reverse=int(bool(reverse)), numseq=lay[0], seqlen=lay[1], row_stride=lay[2],
                    elem_stride=lay[3])
        need = lib().linrec_workspace_bytes_dtype(DTYPES[t.dtype], *lay, 0, int(is_bwd), None)
        entry = (call, ctypes.byref(call), int(need))
    if len(table) >= _REPEAT_MAX:
        table.clear()
    table[key] = entry
    return entry


def _repeat_launch(entry, fn, t, what):
    call, ref, need = entry
    idx = t.device.index
    if torch.cuda.current_device() == idx:
        stream = _raw_stream(idx)
        if need:
            ws = workspace(t.device, stream, need)
            call.workspace, call.workspace_bytes = ws.data_ptr(), ws.numel()
        call.stream = stream
        rc = fn(ref)
    else:
        with torch.cuda.device(idx):
            stream = _raw_stream(idx)
            if need:
                ws = workspace(t.device, stream, need)
                call.workspace, call.workspace_bytes = ws.data_ptr(), ws.numel()
            call.stream = stream
            rc = fn(ref)
    if rc:
        check(rc, what)


def _plain_rows(t, lay, *same):
    """The layout if a call on `t` (and tensors `same`, which must lie in memory like it) can be repeated
    from remembered arguments, else None."""
    if lay is None or not t.is_cuda or t.dtype not in DTYPES or not t.numel() or _few_rows_on_strided_axis(t, lay, None):
        return None
    return lay if _same_layout(t, *same) else None


def fwd(inputs, coeffs, reverse=False, tuning=None, out=None):
    """outputs = linrec(inputs, coeffs) over the last dim (linrec/impl/cuda/linrec_pipe.cu:16-92).
    `out`, if given, must have the layout the result would be allocated with."""
    if tuning is None and inputs.is_cuda:
        shape, stride = inputs.shape, inputs.stride()
        key = (inputs.dtype, inputs.device, shape, stride, coeffs.dtype, coeffs.device, coeffs.shape, coeffs.stride(), reverse)
        table = _repeat_table()
        entry = table.get(key, False)
        if entry is False:
            _validate(inputs, coeffs, names=("inputs", "coeffs"))
            entry = _remember(table, key, _plain_rows(inputs, row_layout(inputs), coeffs), inputs, False, reverse)
        if entry is not None:
            px, pc = inputs.data_ptr(), coeffs.data_ptr()
            if not (px | pc) & 15:
                if out is None:
                    res = torch.empty_strided(shape, stride, dtype=inputs.dtype, device=inputs.device)
                elif out.shape == shape and out.stride() == stride and out.dtype == inputs.dtype and out.device == inputs.device:
                    res = out
                else:
                    raise RuntimeError("linrec: `out` does not have the layout of the (canonicalised) inputs")
                po = res.data_ptr()
                if not po & 15:
                    call = entry[0]
                    call.in0, call.coef, call.out0 = px, pc, po
                    _repeat_launch(entry, lib().linrec_fwd_call, inputs, "linrec_fwd")
                    return res
    return _fwd_general(inputs, coeffs, reverse, tuning, out)


def bwd(d_outputs, coeffs, outputs, reverse=False, tuning=None, out=None):
    """(d_inputs, d_coeffs) (linrec/impl/cuda/linrec_pipe.cu:96-174).  The three tensors are brought
    to one memory layout first (the reference instead requires equal strides, linrec_pipe.cu:98)."""
    if tuning is None and outputs.is_cuda:
        shape, stride = outputs.shape, outputs.stride()
        key = (outputs.dtype, outputs.device, shape, stride, coeffs.dtype, coeffs.device, coeffs.shape, coeffs.stride(),
               d_outputs.dtype, d_outputs.device, d_outputs.shape, d_outputs.stride(), reverse, True)
        table = _repeat_table()
        entry = table.get(key, False)
        if entry is False:
            _validate(outputs, coeffs, d_outputs, names=("outputs", "coeffs", "d_outputs"))
            entry = _remember(table, key, _plain_rows(outputs, row_layout(outputs), coeffs, d_outputs), outputs, True, reverse)
        if entry is not None:
            pd, pc, py = d_outputs.data_ptr(), coeffs.data_ptr(), outputs.data_ptr()
            if not (pd | pc | py) & 15:
                if out is None:
                    dx = torch.empty_strided(shape, stride, dtype=outputs.dtype, device=outputs.device)
                    dc = torch.empty_strided(shape, stride, dtype=outputs.dtype, device=outputs.device)
                else:
                    dx, dc = out
                    if not (_same_layout(outputs, dx, dc) and dx.dtype == outputs.dtype == dc.dtype
                            and dx.device == outputs.device == dc.device):
                        raise RuntimeError("linrec: `out` tensors do not have the layout of the (canonicalised) outputs")
                p0, p1 = dx.data_ptr(), dc.data_ptr()
                if not (p0 | p1) & 15:
                    call = entry[0]
                    call.in0, call.coef, call.aux, call.out0, call.out1 = pd, pc, py, p0, p1
                    _repeat_launch(entry, lib().linrec_bwd_call, outputs, "linrec_bwd")
                    return dx, dc
    return _bwd_general(d_outputs, coeffs, outputs, reverse, tuning, out)


def _fwd_general(inputs, coeffs, reverse=False, tuning=None, out=None):
    _validate(inputs, coeffs, names=("inputs", "coeffs"))
    if not inputs.is_cuda and inputs.dtype in (torch.float16, torch.bfloat16):
        # host tensors in a 16-bit type: fp32 arithmetic, one rounding at the end, as on the device
        res = fwd(inputs.float(), coeffs.float(), reverse).to(inputs.dtype)
        return res if out is None else out.copy_(res)
    lay = row_layout(inputs)
    bl = batched_layout(inputs) if lay is None else None
    if lay is None and bl is None:
        inputs = _dense(inputs)
        lay = row_layout(inputs)
    if not _same_layout(inputs, coeffs):
        coeffs = _restride(coeffs, inputs)
    outputs = output_like(inputs) if out is None else out
    if not _same_layout(inputs, outputs) or outputs.dtype != inputs.dtype or outputs.device != inputs.device:
        raise RuntimeError("linrec: `out` does not have the layout of the (canonicalised) inputs")
    if inputs.numel():
        if bl is not None:
            _launch_fwd_batched(inputs, coeffs, outputs, bl, reverse, tuning)
        elif _few_rows_on_strided_axis(inputs, lay, tuning):
            _assign(outputs, fwd(_dense(inputs), _dense(coeffs), reverse))
        else:
            _launch_fwd(inputs, coeffs, outputs, lay, reverse, tuning)
    return outputs


def _bwd_general(d_outputs, coeffs, outputs, reverse=False, tuning=None, out=None):
    _validate(outputs, coeffs, d_outputs, names=("outputs", "coeffs", "d_outputs"))
    if not outputs.is_cuda and outputs.dtype in (torch.float16, torch.bfloat16):
        dx, dc = bwd(d_outputs.float(), coeffs.float(), outputs.float(), reverse)
        dx, dc = dx.to(outputs.dtype), dc.to(outputs.dtype)
        return (dx, dc) if out is None else (out[0].copy_(dx), out[1].copy_(dc))
    lay = row_layout(outputs)
    bl = batched_layout(outputs) if lay is None else None
    if lay is None and bl is None:
        outputs = _dense(outputs)
        lay = row_layout(outputs)
    if not _same_layout(outputs, coeffs):
        coeffs = _restride(coeffs, outputs)
    if not _same_layout(outputs, d_outputs):
        d_outputs = _restride(d_outputs, outputs)
    d_inputs, d_coeffs = (output_like(outputs), output_like(outputs)) if out is None else out
    if not _same_layout(outputs, d_inputs, d_coeffs):
        raise RuntimeError("linrec: `out` tensors do not have the layout of the (canonicalised) outputs")
    if outputs.numel():
        if bl is not None:
            _launch_bwd_batched(d_outputs, coeffs, outputs, d_inputs, d_coeffs, bl, reverse, tuning)
        elif _few_rows_on_strided_axis(outputs, lay, tuning):
            dx, dc = bwd(_dense(d_outputs), _dense(coeffs), _dense(outputs), reverse)
            _assign(d_inputs, dx)
            _assign(d_coeffs, dc)
        else:
            _launch_bwd(d_outputs, coeffs, outputs, d_inputs, d_coeffs, lay, reverse, tuning)
    return d_inputs, d_coeffs


def kernel_table():
    """Names of all compiled kernels (role of _C.config_list, linrec/impl/cuda/extension.cpp:38-39)."""
    L = lib()
    return [L.linrec_kernel_name(i).decode() for i in range(L.linrec_kernel_count())]


def plan_thresholds():
    """{name: value} of the planner's generated crossover thresholds (csrc/plan_thresholds.inc as compiled in)."""
    L = lib()
    return {L.linrec_plan_threshold_name(i).decode(): int(L.linrec_plan_threshold_value(i))
            for i in range(L.linrec_plan_threshold_count())}


def kernel_attrs(kernel_id):
    """Registers / LDS / scratch of one kernel (role of linrec_pipe_attrs, linrec_pipe.cu:177-212)."""
    vals = [ctypes.c_int() for _ in range(4)]
    check(lib().linrec_kernel_attrs(kernel_id, *[ctypes.byref(v) for v in vals]), "linrec_kernel_attrs")
    return dict(zip(("num_regs", "lds_bytes", "scratch_bytes", "max_threads"), (v.value for v in vals)))


def copy(src, dst):
    """Streaming copy with the scan kernels' access pattern (bandwidth ceiling measurement)."""
    assert src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()
    assert src.dtype == torch.float32 and dst.dtype == torch.float32 and src.numel() == dst.numel()
    with torch.cuda.device(src.device):
        check(lib().linrec_copy_f32(src.data_ptr(), dst.data_ptr(), src.numel(),
                                    torch.cuda.current_stream(src.device).cuda_stream), "linrec_copy_f32")


def stream_mix(srcs, dsts, hold=(0, 0)):
    """Sum of the float32 streams `srcs` (0-3 dense tensors) stored to each of `dsts` (0-2): the
    memory system's rate for that mix of read and write streams, no scan attached.  `hold` = (lo, bits):
    the launch takes its 16 KiB blocks in an order that keeps those bits of the block index (address bits
    14 + lo and up) the same among the blocks in flight (needs a power of two of whole blocks)."""
    ts = list(srcs) + list(dsts)
    assert ts and all(t.is_cuda and t.is_contiguous() and t.dtype == torch.float32 for t in ts)
    n = ts[0].numel()
    assert all(t.numel() == n for t in ts) and n % 4 == 0
    ps = [t.data_ptr() for t in srcs] + [None] * (3 - len(srcs))
    pd = [t.data_ptr() for t in dsts] + [None] * (2 - len(dsts))
    with torch.cuda.device(ts[0].device):
        check(lib().linrec_stream_mix_order_f32(len(srcs), len(dsts), *ps, *pd, n, int(hold[0]), int(hold[1]),
                                                torch.cuda.current_stream(ts[0].device).cuda_stream),
              "linrec_stream_mix_order_f32")


def launch_model(srcs, dsts, shape, waves, slots, team, ahead=1, late=2, stamps=None):
    """Memory-only model of a drift launch over dense float32 tensors of `shape` = (rows, length): the drift
    kernels' workgroups, teams, tiles and order of accesses without scan or exchange (linrec_launch_model_f32).
    `stamps`: int64 device tensor of 2 x workgroups words for every workgroup's start and end (100 MHz clock)."""
    ts = list(srcs) + list(dsts)
    assert ts and all(t.is_cuda and t.is_contiguous() and t.dtype == torch.float32 and t.numel() == shape[0] * shape[1] for t in ts)
    ps = [t.data_ptr() for t in srcs] + [None] * (3 - len(srcs))
    pd = [t.data_ptr() for t in dsts] + [None] * (2 - len(dsts))
    with torch.cuda.device(ts[0].device):
        check(lib().linrec_launch_model_f32(len(srcs), len(dsts), *ps, *pd, shape[0], shape[1], waves, slots, team, ahead, late,
                                            None if stamps is None else stamps.data_ptr(),
                                            torch.cuda.current_stream(ts[0].device).cuda_stream), "linrec_launch_model_f32")
