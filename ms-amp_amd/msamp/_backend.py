"""ctypes binding of libmsamp_hip.so: the only door from the Python host layer to the HIP kernels.

Plays the role the reference gives to TransformerEngineWrapper and the msamp_adamw extension
(msamp/common/utils/transformer_engine_wrapper.py:63-176, msamp/optim/adamw.cu:157-162).
There is no CPU or eager fallback: if the library cannot be loaded, or an operand is not on
the GPU, the call raises.
"""

import ctypes
import os

import torch
import torch.distributed as _dist

_LIB_NAME = 'libmsamp_hip.so'
_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'lib', _LIB_NAME)

DT_F32, DT_F16, DT_BF16, DT_E4M3, DT_E5M2 = 2, 3, 4, 5, 6
FLAG_NAN_TO_INF = 1
FLAG_TWO_PASS = 2
FLAG_NO_SPECULATION = 4
WORKSPACE_BYTES = 16384
ADAMW_CHUNK = 16384

_TORCH_TO_DT = {torch.float32: DT_F32, torch.float16: DT_F16, torch.bfloat16: DT_BF16}

_lib = None
_workspaces = {}

_vp, _i, _f, _d, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_double, ctypes.c_size_t

_SIGNATURES = {
    'msamp_hip_version': ([], _i),
    'msamp_last_error': ([], ctypes.c_char_p),
    'msamp_check_async_error': ([_vp, _vp], _i),
    'msamp_set_spin_limit': ([ctypes.c_uint32], None),
    'msamp_amax': ([_vp, _i, _sz, _vp, _vp, _vp], _i),
    'msamp_compute_scaling_factor': ([_vp, _vp, _i, _vp, _i, _f, _i, _vp], _i),
    'msamp_cast_to_fp8': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _i, _vp], _i),
    'msamp_cast_to_fp8_intime': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp], _i),
    'msamp_cast_to_fp8_intime_static': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _i, _i, _i, _vp], _i),
    'msamp_cast_scaled_to_fp8': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp], _i),
    'msamp_add_to_fp8': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _i, _vp, _vp], _i),
    'msamp_cast_from_fp8': ([_vp, _i, _sz, _vp, _vp, _i, _vp], _i),
    'msamp_cast_transpose': ([_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp], _i),
    'msamp_cast_transpose_intime': ([_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp], _i),
    'msamp_fp8_transpose': ([_vp, _i, _i, _vp, _vp], _i),
    'msamp_scale_cast': ([_vp, _i, _sz, _vp, _vp, _i, _vp], _i),
    'msamp_scale_update': ([_vp, _vp, _vp, _vp, _i, _i, _f, _i, _vp], _i),
    'msamp_cast_to_fp8_gated': ([_vp, _i, _sz, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp], _i),
    'msamp_cast_transpose_gated': ([_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp], _i),
    'msamp_fp8_gemm': ([_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _vp], _i),
    'msamp_fp8_gemm_kmajor': ([_vp, _i, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp, _i, _vp], _i),
    'msamp_fp8_gemm_cast': ([_vp, _i, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp], _i),
    'msamp_mfma_probe': ([_vp, _vp, _i, _i, _i, _vp, _vp], _i),
    'msamp_set_small_tile_limit': ([_i], None),
    'msamp_scale_update_groups': ([_vp, _i, _i, _vp], _i),
    'msamp_fp8_norms': ([_vp, _i, _vp, _i, _i, _i, _vp], _i),
    'msamp_bucket_amax': ([_vp, _i, _vp, _i, _i, _i, _vp], _i),
    'msamp_bucket_amax_speculative': ([_vp, _i, _vp, _i, _i, _i, _i, _vp], _i),
    'msamp_bucket_cast': ([_vp, _i, _vp, _i, _i, _i, _f, _f, _i, _vp], _i),
    'msamp_adamw_fp8_stage1': ([_vp, _vp, _sz, _vp, _i, _f, _vp, _f, _vp, _i, _f, _vp, _f, _f, _i, _f, _i, _vp], _i),
    'msamp_adamw_fp8_stage2': ([_vp, _sz, _vp, _i, _f, _f, _f, _vp, _i, _f, _f, _f, _vp], _i),
    'msamp_adamw_fp8_fused': ([_vp, _i, _vp, _i, _i, _i, _d, _d, _d, _d, _d, _i, _i, _i, _i, _i, _vp, _i, _vp], _i),
    'msamp_fp8_gemm_set_walk': ([_i, _i, _i, _i, _i, _i], _i),
    'msamp_fp8_gemm_get_walk': ([_i, _i, _i, _i, _i], _i),
    'msamp_fp8_gemm_tune': ([_vp, _i, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _i, _vp, _vp], _i),
    'msamp_adamw_f32': ([_vp, _vp, _i, _sz, _vp, _vp, _d, _d, _d, _d, _d, _i, _i, _i, _i, _vp], _i),
    'msamp_adamw_plain_fused': ([_vp, _i, _vp, _i, _i, _i, _d, _d, _d, _d, _d, _i, _i, _i, _i, _i, _vp], _i),
    'msamp_adamw_fp8_fused_shift': ([_vp, _vp, _vp, _i, _vp, _i, ctypes.c_longlong, _i, _i, _d, _d, _d, _d, _d, _i, _i, _i, _i, _i, _vp, _vp], _i),
    'msamp_adamw_fp8_fused_speculative': ([_vp, _vp, _vp, _i, _vp, _i, _i, _i, _d, _d, _d, _d, _d, _i, _i, _i, _i, _i, _vp], _i),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path():
    """Path the library is loaded from (env MSAMP_HIP_LIB overrides the in-tree build)."""
    return os.environ.get('MSAMP_HIP_LIB', _LIB_PATH)


def load():
    """Load the shared library once and declare the argument types of every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f'{_LIB_NAME} not found at {path}: build it with `make -C ms-amp_amd/csrc` '
            '(hipcc, --offload-arch=gfx950). There is no fallback implementation.'
        )
    lib = ctypes.CDLL(path)
    for name, (argtypes, restype) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    _lib = lib
    return lib


def _check(rc, what):
    if rc != 0:
        msg = load().msamp_last_error().decode(errors='replace')
        raise RuntimeError(f'{what} failed with code {rc}: {msg}')


def _gpu(t, what):
    if not t.is_cuda:
        raise ValueError(f'{what} is not in GPU memory; the FP8 kernels only run on the HIP device.')
    return t


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    """Raw handle of torch's current stream on the current device."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _dt(t):
    try:
        return _TORCH_TO_DT[t.dtype]
    except KeyError:
        raise TypeError(f'unsupported tensor dtype {t.dtype}') from None


def workspace(device):
    """Scratch words of the two-pass kernels: one buffer per device and stream, since calls that share a buffer
    must be ordered on one stream (the current stream is the one every entry point is given)."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(), _stream())
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.zeros(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


# ---- failures of the kernels whose workgroups wait for each other ------------------------------------------
ERR_TIMEOUT = -5
WS_ERROR_BYTE = 32    # byte offset of the sticky error word in a workspace
_force_two_pass = False
_pending_error_reads = {}
_static_workspace_streams = set()    # (device index, raw stream) pairs that ran msamp_cast_to_fp8_intime_static


class WaitExpiredError(RuntimeError):
    """A one-pass in-time cast or a fused GEMM + cast gave up waiting for its other workgroups."""


def _two_pass_only():
    return _force_two_pass or _shared_device()


def check_async_error(block=True):
    """Report a bounded wait that ran out in one of the kernels whose workgroups wait for each other (the one-pass
    in-time cast, the fused GEMM + cast).  Such a failure cannot be seen by the call that enqueued the kernel; the
    kernel leaves a sticky word in the workspace instead.

    block=True reads the word of every workspace of this process now (synchronises their streams' work up to here),
    including the library's own workspace on every device where cast_to_fp8_intime_static was called.
    block=False never waits: it looks at the copies of the words requested by the previous call -- if they have
    arrived -- and requests new ones, so a training loop that calls it once per step learns of a failure a step or
    two late without ever synchronising (the library's own workspace has no tensor to copy from and is left to the
    blocking form).  Either way a failure raises WaitExpiredError, after switching this process to the two-pass
    kernels for good (same results, no waiting).  The tensors and metas the failed kernel wrote are invalid, and so
    is whatever was computed from them since: go back to the last good state (a checkpoint)."""
    global _force_two_pass
    lib = load()
    failed = None
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        return    # nothing here can be recorded into a graph, and the waiting kernels stay out of captured streams anyway
    if block:
        for dev, stream in sorted(_static_workspace_streams):
            with torch.cuda.device(dev):
                rc = lib.msamp_check_async_error(None, stream)
            if rc == ERR_TIMEOUT:
                failed = lib.msamp_last_error().decode(errors='replace')
            elif rc != 0:
                _check(rc, 'msamp_check_async_error')
    for key, ws in list(_workspaces.items()):
        if not ws.is_cuda:
            continue
        if block:
            with torch.cuda.device(ws.device):
                rc = lib.msamp_check_async_error(_ptr(ws), key[2])
            if rc == ERR_TIMEOUT:
                failed = lib.msamp_last_error().decode(errors='replace')
            elif rc != 0:
                _check(rc, 'msamp_check_async_error')
            continue
        entry = _pending_error_reads.get(key)
        if entry is None:
            # the word is sticky, so it may be read at any time: on a stream of its own, where the copy does not stand
            # between two kernels of the stream that does the work
            with torch.cuda.device(ws.device):
                side = torch.cuda.Stream()
            entry = {'host': torch.zeros(1, dtype=torch.int32, pin_memory=True), 'event': torch.cuda.Event(), 'in_flight': False,
                     'stream': side}
            _pending_error_reads[key] = entry
        if entry['in_flight'] and entry['event'].query():
            entry['in_flight'] = False
            code = int(entry['host'].item())
            if code != 0:
                failed = f'a kernel whose workgroups wait for each other gave up waiting (code {code})'
                ws[WS_ERROR_BYTE:WS_ERROR_BYTE + 4].zero_()
        if not entry['in_flight']:
            with torch.cuda.stream(entry['stream']):
                entry['host'].copy_(ws[WS_ERROR_BYTE:WS_ERROR_BYTE + 4].view(torch.int32), non_blocking=True)
                entry['event'].record()
            entry['in_flight'] = True
    if failed is not None:
        _force_two_pass = True
        # copies of the words requested before they were cleared still carry the old code: forget them, so that
        # the failure is reported once
        _pending_error_reads.clear()
        raise WaitExpiredError(failed + '; the tensors and metas it wrote are invalid, and so is everything computed from '
                               'them since. The process now uses the two-pass kernels only: restore the last good state '
                               'and go on from there.')


def set_spin_limit(polls):
    """Polls after which a waiting kernel gives up (default 2**20); 0 = give up at once, for tests of that path."""
    load().msamp_set_spin_limit(int(polls))


# ---- scaling ------------------------------------------------------------------------------------
def amax(x, amax_cell):
    """amax_cell[0] = max|x| (NaN propagates)."""
    lib = load()
    _gpu(x, 'input')
    _check(lib.msamp_amax(_ptr(x), _dt(x), x.numel(), _ptr(amax_cell), _ptr(workspace(x.device)), _stream()), 'msamp_amax')


def compute_scaling_factor(amax_t, scale_t, fp_max, margin):
    """Element-wise pow-2 scale rule on float32 GPU tensors; returns a new tensor shaped like amax."""
    lib = load()
    _gpu(amax_t, 'amax')
    a = amax_t.to(torch.float32).contiguous()
    s = scale_t.to(device=a.device, dtype=torch.float32).contiguous()
    if s.numel() not in (1, a.numel()):
        raise ValueError('scale must have one element or as many as amax')
    out = torch.empty_like(a)
    _check(
        lib.msamp_compute_scaling_factor(_ptr(a), _ptr(s), s.numel(), _ptr(out), a.numel(), fp_max, margin, _stream()),
        'msamp_compute_scaling_factor'
    )
    return out


def scale_update(scales, amaxs, fp_max, margin, counters=None, want_mask=True):
    """In-place window update of flattened metas.  `counters` (int32 on the GPU) are bumped, or reset where
    the current amax was not finite; returns the uint8 mask of those entries if asked for."""
    lib = load()
    _gpu(scales, 'scales')
    n, window = amaxs.shape
    if counters is not None:
        _gpu(counters, 'counters')
    bad = torch.empty(n, dtype=torch.uint8, device=scales.device) if want_mask else None
    _check(
        lib.msamp_scale_update(_ptr(scales), _ptr(amaxs), _ptr(bad), _ptr(counters), n, window, fp_max, margin, _stream()),
        'msamp_scale_update'
    )
    return bad


MAX_SCALE_GROUPS = 4


class _ScaleGroup(ctypes.Structure):
    """msamp_scale_group."""
    _fields_ = [('scales', ctypes.c_void_p), ('amaxs', ctypes.c_void_p), ('bad', ctypes.c_void_p),
                ('counters', ctypes.c_void_p), ('n', ctypes.c_int32), ('window', ctypes.c_int32),
                ('fp_max', ctypes.c_float), ('reserved', ctypes.c_int32)]


def scale_update_groups(groups, margin):
    """scale_update for several (scales, amaxs, fp_max, counters) groups in one launch (counters may be None)."""
    lib = load()
    for start in range(0, len(groups), MAX_SCALE_GROUPS):
        part = groups[start:start + MAX_SCALE_GROUPS]
        table = (_ScaleGroup * len(part))()
        for row, (scales, amaxs, fp_max, counters) in zip(table, part):
            _gpu(scales, 'scales')
            _gpu(amaxs, 'amaxs')
            if counters is not None:
                _gpu(counters, 'counters')
            row.scales, row.amaxs, row.bad, row.counters = _ptr(scales), _ptr(amaxs), None, _ptr(counters)
            row.n, row.window = amaxs.shape
            row.fp_max = fp_max
        _check(lib.msamp_scale_update_groups(table, len(part), margin, _stream()), 'msamp_scale_update_groups')


# ---- casts --------------------------------------------------------------------------------------
def cast_to_fp8(x, scale, amax_cell, scale_inv, fp8_dt):
    lib = load()
    _gpu(x, 'input')
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _check(
        lib.msamp_cast_to_fp8(_ptr(x), _dt(x), x.numel(), _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), fp8_dt, _stream()),
        'msamp_cast_to_fp8'
    )
    return out


_world_seen = (None, False)


def _default_group():
    """The default process group, or None while torch.distributed is not initialised."""
    return _dist.GroupMember.WORLD if _dist.is_available() else None


def _shared_device():
    """True when other kernels may hold part of the GPU for long (a process group with peers keeps RCCL kernels
    resident beside the compute stream): kernels whose workgroups wait for each other then stay off.  The answer
    is kept per default process group, so a cast pays one attribute read for it."""
    global _world_seen
    world = _default_group()
    if world is None:
        return False
    if world is not _world_seen[0]:
        _world_seen = (world, _dist.get_world_size() > 1)
    return _world_seen[1]


def cast_to_fp8_intime(x, scale, amax_cell, scale_inv, fp8_dt, margin=0, nan_to_inf=False, two_pass=False, speculate=True):
    """amax, scale rule, quantize and reciprocal in one call.  `two_pass` keeps the call off the
    one-pass kernel whose workgroups wait for each other; `speculate=False` keeps the kernels from
    writing the output with the old scale before the new one is known (same results either way)."""
    lib = load()
    _gpu(x, 'input')
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _check(
        lib.msamp_cast_to_fp8_intime(
            _ptr(x), _dt(x), x.numel(), _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), fp8_dt, margin,
            (FLAG_NAN_TO_INF if nan_to_inf else 0) | (FLAG_TWO_PASS if two_pass or _two_pass_only() else 0) |
            (0 if speculate else FLAG_NO_SPECULATION),
            _ptr(workspace(x.device)),
            _stream()
        ), 'msamp_cast_to_fp8_intime'
    )
    return out


STATIC_MAX_ELEMS = 1 << 32


def cast_to_fp8_intime_static(x, scale, amax_cell, scale_inv, out, fp8_dt, margin=0, nan_to_inf=False, two_pass=False):
    """cast_to_fp8_intime into the caller's `out`, with the library's own static workspace: the call allocates
    nothing (for callers that cannot allocate).  Calls on one GPU must not overlap in time."""
    lib = load()
    _gpu(x, 'input')
    _gpu(out, 'output')
    if out.dtype != torch.uint8 or out.numel() != x.numel() or not out.is_contiguous():
        raise ValueError('out must be a contiguous uint8 tensor with as many elements as the input')
    _static_workspace_streams.add((x.device.index if x.device.index is not None else torch.cuda.current_device(), _stream()))
    _check(
        lib.msamp_cast_to_fp8_intime_static(
            _ptr(x), _dt(x), x.numel(), _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), fp8_dt, margin,
            (FLAG_NAN_TO_INF if nan_to_inf else 0) | (FLAG_TWO_PASS if two_pass or _two_pass_only() else 0), _stream()
        ), 'msamp_cast_to_fp8_intime_static'
    )
    return out


def cast_to_fp8_gated(x, scale, amax_cell, scale_inv, fp8_dt, counter, window, margin=0, nan_to_inf=False):
    """In-time cast while counter < window, delayed cast afterwards; the test runs on the GPU."""
    lib = load()
    _gpu(x, 'input')
    _gpu(counter, 'warm-up counter')
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _check(
        lib.msamp_cast_to_fp8_gated(
            _ptr(x), _dt(x), x.numel(), _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), fp8_dt, margin,
            (FLAG_NAN_TO_INF if nan_to_inf else 0) | (FLAG_TWO_PASS if _two_pass_only() else 0), _ptr(counter), window,
            _ptr(workspace(x.device)), _stream()
        ), 'msamp_cast_to_fp8_gated'
    )
    return out


def cast_scaled_to_fp8(x, amax, old_scale_inv, scale, scale_inv, fp8_dt, margin=0, amax_out=None, counter_out=None):
    """Requantize a scaled 16/32-bit payload whose amax is known; writes scale and scale_inv, and, if
    given, copies the amax window to `amax_out` and zeroes `counter_out` (the rest of a fresh meta)."""
    lib = load()
    _gpu(x, 'input')
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    window = amax_out.numel() if amax_out is not None else 0
    if window > amax.numel():
        raise ValueError('amax_out is longer than the source amax window')
    _check(
        lib.msamp_cast_scaled_to_fp8(
            _ptr(x), _dt(x), x.numel(), _ptr(amax), _ptr(old_scale_inv), _ptr(scale), _ptr(scale_inv), _ptr(amax_out),
            window, _ptr(counter_out), _ptr(out), fp8_dt, margin, _stream()
        ), 'msamp_cast_scaled_to_fp8'
    )
    return out


def add_to_fp8(q, fp8_dt, scale, scale_inv, amax_cell, other):
    """In place: q <- in-time cast of (dequant(q) in other's dtype + other); rewrites scale, scale_inv, amax."""
    lib = load()
    _gpu(q, 'fp8 tensor')
    _gpu(other, 'other')
    _check(
        lib.msamp_add_to_fp8(
            _ptr(q), fp8_dt, q.numel(), _ptr(scale), _ptr(scale_inv), _ptr(amax_cell), _ptr(other), _dt(other),
            _ptr(workspace(q.device)), _stream()
        ), 'msamp_add_to_fp8'
    )
    return q


def cast_from_fp8(q, scale_inv, fp8_dt, out_dtype):
    lib = load()
    _gpu(q, 'input')
    out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
    _check(
        lib.msamp_cast_from_fp8(_ptr(q), fp8_dt, q.numel(), _ptr(scale_inv), _ptr(out), _TORCH_TO_DT[out_dtype], _stream()),
        'msamp_cast_from_fp8'
    )
    return out


def cast_transpose(x, scale, amax_cell, scale_inv, fp8_dt, in_time=False, margin=0, nan_to_inf=False):
    lib = load()
    _gpu(x, 'input')
    rows, cols = x.shape
    out = torch.empty((rows, cols), dtype=torch.uint8, device=x.device)
    out_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device)
    if in_time:
        rc = lib.msamp_cast_transpose_intime(
            _ptr(x), _dt(x), rows, cols, _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), _ptr(out_t), fp8_dt,
            margin, FLAG_NAN_TO_INF if nan_to_inf else 0, _ptr(workspace(x.device)), _stream()
        )
    else:
        rc = lib.msamp_cast_transpose(
            _ptr(x), _dt(x), rows, cols, _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), _ptr(out_t), fp8_dt,
            _stream()
        )
    _check(rc, 'msamp_cast_transpose')
    return out, out_t


def cast_transpose_gated(x, scale, amax_cell, scale_inv, fp8_dt, counter, window, margin=0, nan_to_inf=False):
    lib = load()
    _gpu(x, 'input')
    _gpu(counter, 'warm-up counter')
    rows, cols = x.shape
    out = torch.empty((rows, cols), dtype=torch.uint8, device=x.device)
    out_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device)
    _check(
        lib.msamp_cast_transpose_gated(
            _ptr(x), _dt(x), rows, cols, _ptr(scale), _ptr(amax_cell), _ptr(scale_inv), _ptr(out), _ptr(out_t), fp8_dt,
            margin, FLAG_NAN_TO_INF if nan_to_inf else 0, _ptr(counter), window, _ptr(workspace(x.device)), _stream()
        ), 'msamp_cast_transpose_gated'
    )
    return out, out_t


def fp8_transpose(q):
    lib = load()
    _gpu(q, 'input')
    rows, cols = q.shape
    out = torch.empty((cols, rows), dtype=torch.uint8, device=q.device)
    _check(lib.msamp_fp8_transpose(_ptr(q), rows, cols, _ptr(out), _stream()), 'msamp_fp8_transpose')
    return out


def scale_cast(x, scale, out_dtype):
    """out = out_dtype(float(x) * scale) with IEEE overflow."""
    lib = load()
    _gpu(x, 'input')
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    _check(
        lib.msamp_scale_cast(_ptr(x), _dt(x), x.numel(), _ptr(scale), _ptr(out), _TORCH_TO_DT[out_dtype], _stream()),
        'msamp_scale_cast'
    )
    return out


# ---- GEMM ---------------------------------------------------------------------------------------
def gemm_kmajor_supported(m, n, k, a_kmajor, b_kmajor):
    """Shapes the kernel reads K-major operands for (see msamp_fp8_gemm_kmajor)."""
    if b_kmajor and not a_kmajor:
        return False
    return k % 128 == 0 and k >= 256 and (not a_kmajor or m % 256 == 0) and (not b_kmajor or n % 256 == 0) and \
        m * k < 2**32 and n * k < 2**32


# ---- tile walks of the large GEMM, timed at first use ---------------------------------------------------------------
_tune_walks = os.environ.get('MSAMP_GEMM_TUNE', '1') != '0'
_walk_seen = set()
_TUNE_MIN_TILES = 512    # two rounds of 256 x 256 tiles on 256 compute units: below that the library does not time anything


def tune_gemm_walks(on=True):
    """Whether a GEMM problem (sizes and operand layouts) seen for the first time has its tile walk timed: the product of
    that call is computed some forty times over, and the fastest of the walks is used from then on (same bits whichever).
    On by default; the environment variable MSAMP_GEMM_TUNE=0 switches it off from the start."""
    global _tune_walks
    _tune_walks = bool(on)


def forget_gemm_walks():
    """Drop every walk registered so far (the next call of each problem times again if tuning is on)."""
    lib = load()
    for m, n, k, a_kmajor, b_kmajor in _walk_seen:
        lib.msamp_fp8_gemm_set_walk(m, n, k, int(a_kmajor), int(b_kmajor), -1)
    _walk_seen.clear()


def gemm_walks():
    """{(m, n, k, a_kmajor, b_kmajor): walk} of the problems whose timing registered a walk other than the rule's."""
    lib = load()
    found = {key: lib.msamp_fp8_gemm_get_walk(key[0], key[1], key[2], int(key[3]), int(key[4])) for key in _walk_seen}
    return {key: walk for key, walk in found.items() if walk >= 0}


def _tune_walk(lib, a, a_dt, a_scale_inv, a_kmajor, b, b_dt, b_scale_inv, b_kmajor, out, m, n, k, bias):
    """Times the walks of a problem not seen before on the operands given, writing the product to `out`; False (nothing
    done) if the problem has been seen, is too small to matter, or the stream is being captured."""
    key = (m, n, k, bool(a_kmajor), bool(b_kmajor))
    if key in _walk_seen or ((n + 255) // 256) * ((m + 255) // 256) < _TUNE_MIN_TILES or k < 512 or k % 128:
        return False
    if torch.cuda.is_current_stream_capturing():
        return False
    _walk_seen.add(key)
    _check(
        lib.msamp_fp8_gemm_tune(
            _ptr(a), a_dt, _ptr(a_scale_inv), 1 if a_kmajor else 0, _ptr(b), b_dt, _ptr(b_scale_inv), 1 if b_kmajor else 0,
            _ptr(out), _dt(out), m, n, k, _ptr(bias), _dt(bias) if bias is not None else DT_F32, None, _stream()
        ), 'msamp_fp8_gemm_tune'
    )
    return True


def fp8_gemm(a, a_dt, a_scale_inv, b, b_dt, b_scale_inv, out, accumulate=False, bias=None, a_kmajor=False, b_kmajor=False):
    """out[N,M] (+)= (b[N,K] . a[M,K]^T) * a_scale_inv * b_scale_inv (+ bias[M]).
    With a_kmajor / b_kmajor the tensor handed over is the transpose, [K,M] / [K,N]."""
    lib = load()
    _gpu(a, 'mat_a')
    _gpu(b, 'mat_b')
    if _tune_walks and not accumulate and a.dim() == 2 and b.dim() == 2 and (a_kmajor or not b_kmajor):
        k, m = a.shape if a_kmajor else a.shape[::-1]
        kb, n = b.shape if b_kmajor else b.shape[::-1]
        if kb == k and tuple(out.shape) == (n, m) and out.is_contiguous() and \
                _tune_walk(lib, a, a_dt, a_scale_inv, a_kmajor, b, b_dt, b_scale_inv, b_kmajor, out, m, n, k, bias):
            return out
    if a_kmajor or b_kmajor:
        k, m = a.shape if a_kmajor else a.shape[::-1]
        kb, n = b.shape if b_kmajor else b.shape[::-1]
        if kb != k or tuple(out.shape) != (n, m):
            raise ValueError(f'shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}, out {tuple(out.shape)}')
        _check(
            lib.msamp_fp8_gemm_kmajor(
                _ptr(a), a_dt, _ptr(a_scale_inv), 1 if a_kmajor else 0, _ptr(b), b_dt, _ptr(b_scale_inv),
                1 if b_kmajor else 0, _ptr(out), _dt(out), m, n, k, 1 if accumulate else 0, _ptr(bias),
                _dt(bias) if bias is not None else DT_F32, _stream()
            ), 'msamp_fp8_gemm_kmajor'
        )
        return out
    m, k = a.shape
    n = b.shape[0]
    if b.shape[1] != k or tuple(out.shape) != (n, m):
        raise ValueError(f'shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}, out {tuple(out.shape)}')
    _check(
        lib.msamp_fp8_gemm(
            _ptr(a), a_dt, _ptr(a_scale_inv), _ptr(b), b_dt, _ptr(b_scale_inv), _ptr(out), _dt(out), m, n, k,
            1 if accumulate else 0, _ptr(bias), _dt(bias) if bias is not None else DT_F32, _stream()
        ), 'msamp_fp8_gemm'
    )
    return out


NOT_FUSED = 1


def fp8_gemm_cast(a, a_dt, a_scale_inv, b, b_dt, b_scale_inv, hp_dtype, q_dt, scale, amax_cell, scale_inv, margin=0,
                  nan_to_inf=False, a_kmajor=False, b_kmajor=False, hp_out=None, accumulate=False, speculate=True):
    """The product of fp8_gemm, rounded to hp_dtype and cast on to FP8 with in-time scaling (amax_cell[0], scale and
    scale_inv are updated), without a second trip over the product.  Small problems (at most one tile per compute unit)
    take one launch and never store the product; any other problem stores it in `hp_out` (allocated here if not given;
    with `accumulate` it must be given and the product is added to what it holds) together with the codes for the scale in
    force, and reads it again only when the scale rule arrives at another scale.  Returns the uint8 payload [N, M], or
    None when neither form applies to this problem (nothing has been touched then): take fp8_gemm and cast_to_fp8_intime
    instead."""
    lib = load()
    _gpu(a, 'mat_a')
    _gpu(b, 'mat_b')
    k, m = a.shape if a_kmajor else a.shape[::-1]
    kb, n = b.shape if b_kmajor else b.shape[::-1]
    if kb != k:
        raise ValueError(f'shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}')
    if hp_dtype not in _TORCH_TO_DT:
        raise TypeError(f'unsupported intermediate dtype {hp_dtype}')
    if accumulate and hp_out is None:
        raise ValueError('accumulate needs hp_out')
    if hp_out is not None and (hp_out.dtype != hp_dtype or tuple(hp_out.shape) != (n, m) or not hp_out.is_contiguous()):
        raise ValueError(f'hp_out must be a contiguous {hp_dtype} tensor of shape {(n, m)}')
    if hp_out is None and speculate and m % 256 == 0 and n % 256 == 0 and (n // 256) * (m // 256) > 0:
        hp_out = torch.empty(n, m, dtype=hp_dtype, device=a.device)
    if _tune_walks and (a_kmajor or not b_kmajor):
        # (the product into a scratch buffer of its own: hp_out may hold a sum that is being added to)
        key = (m, n, k, bool(a_kmajor), bool(b_kmajor))
        if key not in _walk_seen and ((n + 255) // 256) * ((m + 255) // 256) >= _TUNE_MIN_TILES and \
                not torch.cuda.is_current_stream_capturing():
            _tune_walk(lib, a, a_dt, a_scale_inv, a_kmajor, b, b_dt, b_scale_inv, b_kmajor,
                       torch.empty(n, m, dtype=hp_dtype, device=a.device), m, n, k, None)
    out = torch.empty(n, m, dtype=torch.uint8, device=a.device)
    rc = lib.msamp_fp8_gemm_cast(
        _ptr(a), a_dt, _ptr(a_scale_inv), 1 if a_kmajor else 0, _ptr(b), b_dt, _ptr(b_scale_inv), 1 if b_kmajor else 0,
        _ptr(hp_out), _TORCH_TO_DT[hp_dtype], 1 if accumulate else 0, _ptr(out), q_dt, _ptr(scale), _ptr(amax_cell),
        _ptr(scale_inv), m, n, k, margin,
        (FLAG_NAN_TO_INF if nan_to_inf else 0) | (FLAG_TWO_PASS if _two_pass_only() else 0) |
        (0 if speculate else FLAG_NO_SPECULATION), _ptr(workspace(a.device)), _stream()
    )
    if rc == NOT_FUSED:
        return None
    _check(rc, 'msamp_fp8_gemm_cast')
    return out


def set_small_tile_limit(big_tiles):
    """Row-major GEMMs of at most this many 256 x 256 output tiles run 128 x 128 tiles (default 128, 0 = never)."""
    load().msamp_set_small_tile_limit(int(big_tiles))


def mfma_probe(seed, sink, iters, workgroups, distinct_operands=False):
    """Launch the register-only FP8 MFMA loop (calibration aid); returns the floating-point operations of the launch.
    seed: at least 4096 bytes of FP8 codes on the device, sink: one float32 on the device.  distinct_operands: eight X
    and eight Y fragments taken in turn instead of one pair for every MFMA."""
    assert seed.is_cuda and seed.is_contiguous() and seed.numel() * seed.element_size() >= 4096
    assert sink.is_cuda and sink.dtype == torch.float32
    flop = ctypes.c_double(0.0)
    _check(load().msamp_mfma_probe(_ptr(seed), _ptr(sink), int(iters), int(workgroups), 1 if distinct_operands else 0,
                                   ctypes.byref(flop), _stream()), 'msamp_mfma_probe')
    return flop.value


# ---- gradient buckets -----------------------------------------------------------------------------
BUCKET_CHUNK = 16384
BUCKET_ITEM_WORDS = 7    # int64 words per msamp_bucket_item (56 bytes)


_CHUNK_MAPS = {}


def chunk_map(numels, device):
    """[(item, chunk)] rows, one per workgroup of BUCKET_CHUNK elements, as an int32 device tensor.  The map
    depends on the sizes only, so the last few are kept per device."""
    import numpy as np
    key = (str(device), tuple(int(n) for n in numels))
    hit = _CHUNK_MAPS.get(key)
    if hit is not None:
        return hit
    chunks = [(n + BUCKET_CHUNK - 1) // BUCKET_CHUNK for n in key[1]]
    item_idx = np.repeat(np.arange(len(chunks), dtype=np.int32), chunks)
    chunk_idx = np.concatenate([np.arange(c, dtype=np.int32) for c in chunks]) if sum(chunks) else np.zeros(0, np.int32)
    block_map = torch.from_numpy(np.stack([item_idx, chunk_idx], axis=1).copy()).to(device)
    if len(_CHUNK_MAPS) >= 32:
        _CHUNK_MAPS.pop(next(iter(_CHUNK_MAPS)))
    _CHUNK_MAPS[key] = block_map
    return block_map


def bucket_tables(srcs, dsts, amaxs, scales, scale_invs):
    """Device descriptor table and block map for quantizing `srcs` into `dsts` (views of one flat buffer)."""
    import numpy as np
    rows = [(s.data_ptr(), d.data_ptr(), a.data_ptr(), sc.data_ptr(), si.data_ptr(), s.numel(), 0)
            for s, d, a, sc, si in zip(srcs, dsts, amaxs, scales, scale_invs)]
    device = srcs[0].device
    items = torch.from_numpy(np.asarray(rows, dtype=np.int64).reshape(len(rows), BUCKET_ITEM_WORDS)).to(device)
    return items, chunk_map([s.numel() for s in srcs], device)


def bucket_amax(items, block_map, in_dt, nan_to_inf=True, speculate_fp8_dt=None):
    """amax[0] of every item of the table.  With speculate_fp8_dt the pass also writes every item's codes with the
    scale the item has now; bucket_cast then redoes only the items whose scale came out different."""
    lib = load()
    _gpu(items, 'descriptor table')
    flags = FLAG_NAN_TO_INF if nan_to_inf else 0
    if speculate_fp8_dt is not None:
        _check(
            lib.msamp_bucket_amax_speculative(_ptr(items), items.shape[0], _ptr(block_map), block_map.shape[0], in_dt,
                                              speculate_fp8_dt, flags, _stream()), 'msamp_bucket_amax_speculative'
        )
        return
    _check(
        lib.msamp_bucket_amax(_ptr(items), items.shape[0], _ptr(block_map), block_map.shape[0], in_dt, flags, _stream()),
        'msamp_bucket_amax'
    )


def bucket_cast(items, block_map, in_dt, fp8_dt, pre_scale, scale_inv_div=1.0, margin=0):
    """scale = rule(amax[0]) * pre_scale, scale_inv = (1/scale) / scale_inv_div, FP8 codes of every item into its place."""
    lib = load()
    _gpu(items, 'descriptor table')
    _check(
        lib.msamp_bucket_cast(_ptr(items), items.shape[0], _ptr(block_map), block_map.shape[0], in_dt, fp8_dt, pre_scale,
                              scale_inv_div, margin, _stream()), 'msamp_bucket_cast'
    )


NORM_ITEM_WORDS = 5    # int64 words per msamp_norm_item (40 bytes)


_NORM_TABLES = {}


def fp8_norms(values, scale_invs, fp8_dt, norm_type):
    """Per-tensor p-norms (p = 1, 2 or inf) of FP8 payloads times their scale_inv, as one float32 vector.  The
    descriptor table is kept per set of payload and scale_inv addresses (a training loop asks for the same gradients'
    norms every step), the result is a fresh tensor every time."""
    import numpy as np
    kind = {1.0: 1, 2.0: 2, float('inf'): 0}[float(norm_type)]
    lib = load()
    sig = (tuple(v.data_ptr() for v in values), tuple(si.data_ptr() for si in scale_invs), tuple(v.numel() for v in values))
    cached = _NORM_TABLES.get(sig)
    if cached is None:
        for v in values:
            _gpu(v, 'fp8 tensor')
            if not v.is_contiguous():
                raise ValueError('fp8 tensors must be contiguous')
        device = values[0].device
        result = torch.empty(len(values), dtype=torch.float32, device=device)
        rows = [(v.data_ptr(), si.data_ptr(), result.data_ptr() + 4 * i, v.numel(), 0) for i, (v, si) in enumerate(zip(values, scale_invs))]
        items = torch.from_numpy(np.asarray(rows, dtype=np.int64).reshape(len(rows), NORM_ITEM_WORDS)).to(device)
        cached = (items, chunk_map(sig[2], device), result)
        if len(_NORM_TABLES) >= 8:
            _NORM_TABLES.pop(next(iter(_NORM_TABLES)))
        _NORM_TABLES[sig] = cached
    items, block_map, result = cached
    _check(
        lib.msamp_fp8_norms(_ptr(items), len(values), _ptr(block_map), block_map.shape[0], fp8_dt, kind, _stream()),
        'msamp_fp8_norms'
    )
    return result.clone()


# ---- AdamW --------------------------------------------------------------------------------------
_STATE_DT = {torch.float32: DT_F32, torch.float16: DT_F16}


def state_dt(tensor, qtype_value=None):
    """Library code of an optimizer-state payload (uint8 payloads need the qtype to tell the format)."""
    if tensor.dtype == torch.uint8:
        return qtype_value if qtype_value is not None else DT_E4M3
    return _STATE_DT[tensor.dtype]


def adamw_stage1(param, grad, exp_avg, exp_avg_dt, exp_avg_factor, exp_avg_amax, beta1, exp_avg_sq, exp_avg_sq_dt,
                 exp_avg_sq_factor, exp_avg_sq_amax, beta2, eps, step, lr, bias_correction):
    lib = load()
    _gpu(param, 'param')
    _check(
        lib.msamp_adamw_fp8_stage1(
            _ptr(param), _ptr(grad), param.numel(), _ptr(exp_avg), exp_avg_dt, exp_avg_factor, _ptr(exp_avg_amax), beta1,
            _ptr(exp_avg_sq), exp_avg_sq_dt, exp_avg_sq_factor, _ptr(exp_avg_sq_amax), beta2, eps, step, lr,
            1 if bias_correction else 0, _stream()
        ), 'msamp_adamw_fp8_stage1'
    )


def adamw_stage2(grad, exp_avg, exp_avg_dt, old_factor, new_factor, beta1, exp_avg_sq, exp_avg_sq_dt, old_sq_factor,
                 new_sq_factor, beta2):
    lib = load()
    _gpu(grad, 'grad')
    _check(
        lib.msamp_adamw_fp8_stage2(
            _ptr(grad), grad.numel(), _ptr(exp_avg), exp_avg_dt, old_factor, new_factor, beta1, _ptr(exp_avg_sq),
            exp_avg_sq_dt, old_sq_factor, new_sq_factor, beta2, _stream()
        ), 'msamp_adamw_fp8_stage2'
    )


ADAMW_DESC_WORDS = 19    # int64 words per msamp_adamw_tensor (152 bytes)
ADAMW_BUFFER_WORDS = 4    # int64 words per msamp_adamw_buffers (weight, exp_avg, exp_avg_sq, reserved)


# chunks per cache-resident group of the fused AdamW step; 0 = one group (the kernels are compute-bound, so
# splitting the launch only costs occupancy)
ADAMW_GROUP_BLOCKS = int(os.environ.get('MSAMP_ADAMW_GROUP_BLOCKS', 0))


def adamw_fused(desc, n_tensors, block_map, n_blocks, weight_dt, grad_dt, lr, beta1, beta2, eps, weight_decay, step,
                bias_correction, adam_mode, maximize, tensor_scale, blocks_per_tensor=None, group_blocks=None):
    """blocks_per_tensor: host-side sequence of chunk counts (one per tensor) enabling cache-sized groups."""
    lib = load()
    _gpu(desc, 'descriptor table')
    bpt = None
    if blocks_per_tensor is not None:
        bpt = (ctypes.c_int32 * n_tensors)(*blocks_per_tensor)
    gb = ADAMW_GROUP_BLOCKS if group_blocks is None else group_blocks
    _check(
        lib.msamp_adamw_fp8_fused(
            _ptr(desc), n_tensors, _ptr(block_map), n_blocks, weight_dt, grad_dt, lr, beta1, beta2, eps, weight_decay,
            step, 1 if bias_correction else 0, 1 if adam_mode else 0, 1 if maximize else 0, 1 if tensor_scale else 0,
            ctypes.cast(bpt, ctypes.c_void_p) if bpt is not None else None, gb if bpt is not None else 0, _stream()
        ), 'msamp_adamw_fp8_fused'
    )


def hp_dt(tensor):
    """Library code of a float32 / float16 / bfloat16 tensor's element type."""
    return _dt(tensor)


def adamw_f32(param, grad, exp_avg, exp_avg_sq, lr, beta1, beta2, eps, weight_decay, step, bias_correction, adam_mode,
              maximize):
    """One AdamW / Adam step of a float32 parameter with float32 moments, in place, in one pass; `grad` may be float32,
    float16 or bfloat16."""
    lib = load()
    for t, what in ((param, 'param'), (grad, 'grad'), (exp_avg, 'exp_avg'), (exp_avg_sq, 'exp_avg_sq')):
        _gpu(t, what)
        if not t.is_contiguous() or t.numel() != param.numel():
            raise ValueError(f'adamw_f32: {what} must be contiguous and of the parameter\'s size')
    if any(t.dtype != torch.float32 for t in (param, exp_avg, exp_avg_sq)):
        raise TypeError('adamw_f32: param, exp_avg and exp_avg_sq must be float32')
    _check(
        lib.msamp_adamw_f32(
            _ptr(param), _ptr(grad), _dt(grad), param.numel(), _ptr(exp_avg), _ptr(exp_avg_sq), lr, beta1, beta2, eps,
            weight_decay, step, 1 if bias_correction else 0, 1 if adam_mode else 0, 1 if maximize else 0, _stream()
        ), 'msamp_adamw_f32'
    )


def adamw_plain_fused(desc, n_tensors, param_dt, grad_dt, lr, beta1, beta2, eps, weight_decay, step, bias_correction,
                      adam_mode, maximize, tensor_scale, block_map=None, n_blocks=0):
    """Both stages of the step for n_tensors high-precision parameters with E4M3 / scaled-fp16 moments.  `desc`: int64
    device tensor [n_tensors, ADAMW_DESC_WORDS] with the parameter, gradient, moment payloads, moment metas and numel
    columns filled in.  Without `block_map`: one launch, one workgroup per tensor (small tensors); with it (int32 device
    tensor of {tensor, chunk} pairs over chunks of ADAMW_CHUNK elements): three launches, any size, payloads aligned for
    four elements."""
    lib = load()
    _gpu(desc, 'descriptor table')
    if desc.dtype != torch.int64 or desc.numel() != n_tensors * ADAMW_DESC_WORDS or not desc.is_contiguous():
        raise ValueError('desc must be a contiguous int64 tensor of n_tensors x %d words' % ADAMW_DESC_WORDS)
    if block_map is not None:
        _gpu(block_map, 'block map')
        if block_map.dtype != torch.int32 or block_map.numel() != 2 * n_blocks or not block_map.is_contiguous():
            raise ValueError('block_map must be a contiguous int32 tensor of n_blocks pairs')
    _check(
        lib.msamp_adamw_plain_fused(
            _ptr(desc), n_tensors, _ptr(block_map) if block_map is not None else None, n_blocks, param_dt, grad_dt, lr, beta1,
            beta2, eps, weight_decay, step, 1 if bias_correction else 0, 1 if adam_mode else 0, 1 if maximize else 0,
            1 if tensor_scale else 0, _stream()
        ), 'msamp_adamw_plain_fused'
    )


def adamw_fused_speculative(desc, outputs, redo, n_tensors, block_map, n_blocks, weight_dt, grad_dt, lr, beta1, beta2, eps,
                            weight_decay, step, bias_correction, adam_mode, maximize, tensor_scale):
    """The fused step in one pass into separate buffers.  `outputs`: int64 device tensor [n_tensors, ADAMW_BUFFER_WORDS]
    of output pointers; `redo`: int32 device tensor [n_tensors], set by the call where a tensor took the second round.
    On return every tensor's new payloads are in its output buffers; the inputs still hold the old state."""
    lib = load()
    _gpu(desc, 'descriptor table')
    _gpu(outputs, 'output table')
    _gpu(redo, 'redo flags')
    if outputs.dtype != torch.int64 or outputs.numel() != n_tensors * ADAMW_BUFFER_WORDS or not outputs.is_contiguous():
        raise ValueError('outputs must be a contiguous int64 tensor of n_tensors x %d words' % ADAMW_BUFFER_WORDS)
    if redo.dtype != torch.int32 or redo.numel() != n_tensors or not redo.is_contiguous():
        raise ValueError('redo must be a contiguous int32 tensor of n_tensors flags')
    _check(
        lib.msamp_adamw_fp8_fused_speculative(
            _ptr(desc), _ptr(outputs), _ptr(redo), n_tensors, _ptr(block_map), n_blocks, weight_dt, grad_dt, lr, beta1, beta2,
            eps, weight_decay, step, 1 if bias_correction else 0, 1 if adam_mode else 0, 1 if maximize else 0,
            1 if tensor_scale else 0, _stream()
        ), 'msamp_adamw_fp8_fused_speculative'
    )


ADAMW_POST_WORDS = 8


def adamw_shift_sync_bytes(n_tensors, n_blocks):
    """Size of the `sync` buffer of adamw_fused_shift (MSAMP_ADAMW_SYNC_BYTES)."""
    return n_tensors * ADAMW_POST_WORDS * 8 + n_blocks * 136


def adamw_fused_shift(desc, redo, sync, n_tensors, block_map, n_blocks, shift_elems, weight_dt, grad_dt, lr, beta1, beta2, eps,
                      weight_decay, step, bias_correction, adam_mode, maximize, tensor_scale):
    """The fused step in one pass inside shifting arenas: every tensor's new payloads land `shift_elems` elements away
    from the old ones (see msamp_adamw_fp8_fused_shift for the layout this needs).  `redo`: int32 device tensor
    [n_tensors], set by the call where a tensor took the second round; `sync`: uint8 device tensor of
    adamw_shift_sync_bytes(n_tensors, n_blocks) bytes, zeroed once, the kernels' own."""
    lib = load()
    _gpu(desc, 'descriptor table')
    _gpu(redo, 'redo flags')
    if redo.dtype != torch.int32 or redo.numel() != n_tensors or not redo.is_contiguous():
        raise ValueError('redo must be a contiguous int32 tensor of n_tensors flags')
    _gpu(sync, 'sync buffer')
    if sync.numel() * sync.element_size() < adamw_shift_sync_bytes(n_tensors, n_blocks) or not sync.is_contiguous():
        raise ValueError('sync must be a contiguous buffer of at least %d bytes' % adamw_shift_sync_bytes(n_tensors, n_blocks))
    _check(
        lib.msamp_adamw_fp8_fused_shift(
            _ptr(desc), _ptr(redo), _ptr(sync), n_tensors, _ptr(block_map), n_blocks, int(shift_elems), weight_dt, grad_dt, lr,
            beta1, beta2, eps, weight_decay, step, 1 if bias_correction else 0, 1 if adam_mode else 0, 1 if maximize else 0,
            1 if tensor_scale else 0, _ptr(workspace(desc.device)), _stream()
        ), 'msamp_adamw_fp8_fused_shift'
    )
