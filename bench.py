"""Benchmark of the FP8 hot path on one MI355X.

Headline workload (config 4 of the baseline): every FP8Linear GEMM of one Llama-7B-shaped transformer layer,
forward and backward, at 16384 tokens -- QKV [12288,4096], O [4096,4096], gate and up [11008,4096], down
[4096,11008] -- through the msamp API in steady-state delayed scaling (amax history 16): per layer the input
cast to E4M3, the weight cast, y = x W^T, the cast of dy to E5M2, dx = dy W and dW = dy^T x (W, x and dy are
read K-major in place, no transposed copies), the in-time E4M3 cast of dW; once per step the amax-window
update.  A step is one such pass over the five layers; `value` is the fifteen GEMMs' 2*M*N*K flops divided by
the whole step time, inputs resident in HBM.

`roofline` is the GEMM kernel alone: the flops of the GEMM launches bracketed by HIP events inside the timed
region (every fourth step), divided by their summed duration, against the dense-FP8 MFMA peak.

Beside it: the same step at config 2 (one FP8Linear 8192 x 4096 x 4096), a per-shape GEMM sweep over the
Llama-7B (config 4) and Llama-70B (config 5) projections x {forward, dgrad, wgrad}, the cast+amax and fused
FP8-AdamW kernels against the HBM roofline, and the CPU oracle timed on the host cores.

Prints one JSON line.  Synthetic data, random weights.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, 'ms-amp_amd')):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
FP8_PEAK_TFLOPS = 5000.0
GEMM_EVENT_STRIDE = 4
SCALING_WARMUP_STEPS = 17    # one more than the amax window: afterwards the casts use delayed scaling

# (name, out_features, in_features) of the projections of one layer
LLAMA_7B = {'tokens': 16384, 'proj': (('qkv', 12288, 4096), ('o', 4096, 4096), ('gate', 11008, 4096),
                                       ('up', 11008, 4096), ('down', 4096, 11008))}
LLAMA_70B = {'tokens': 16384, 'proj': (('qkv', 10240, 8192), ('o', 8192, 8192), ('gate', 28672, 8192),
                                        ('up', 28672, 8192), ('down', 8192, 28672))}
# not a BASELINE configuration: a Llama-3-8B layer (MLP width 14336), shapes on which the tile-walk rules were not measured
LLAMA3_8B = {'tokens': 16384, 'proj': (('qkv', 6144, 4096), ('o', 4096, 4096), ('gate', 14336, 4096), ('up', 14336, 4096),
                                       ('down', 4096, 14336))}
CONFIG_2 = {'tokens': 8192, 'proj': (('linear', 4096, 4096), )}


def _events():
    import torch
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def _time_gpu(fn, iters, warm=3, settle_ms=0.0, batches=1):
    """Average duration of one call, from HIP events around a batch of `iters` back-to-back calls on the
    current stream (what a kernel sustains once the launch queue is primed).  `settle_ms`: keep warming up until that
    much wall time has passed (clocks, allocator pools and library heuristics settled); `batches`: time that many
    batches and return the median one (a stall in one batch -- an allocation inside a library call -- does not
    become the figure)."""
    import torch
    t0 = time.perf_counter()
    n = 0
    while n < warm or (time.perf_counter() - t0) * 1e3 < settle_ms:
        fn()
        n += 1
        if settle_ms and n % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    times = []
    for _ in range(batches):
        s, e = _events()
        s.record()
        for _ in range(iters):
            fn()
        e.record()
        e.synchronize()
        times.append(s.elapsed_time(e) / iters)
    return sorted(times)[len(times) // 2]


# ---- synthetic inputs (bench-local: the GPU legs import nothing from tests/ or oracle/) ---------------------------
def c1_input(seed=0, n_rows=4096, n_cols=4096):
    """Config 1: fp32 N(0,1) with 0.1 % of the entries (uniformly chosen) multiplied by 100.  On the CPU."""
    import torch
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n_rows, n_cols, generator=g)
    idx = torch.randperm(x.numel(), generator=g)[:x.numel() // 1000]
    x.view(-1)[idx] *= 100
    return x


def new_meta(window=1):
    """Device-side (scale, scale_inv, amax) as the C ABI wants them."""
    import torch
    return torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(window, device='cuda')


def fp8_randn(shape, std, fp8_dt, seed):
    """N(0, std) drawn on the GPU in bf16 and cast to FP8 in-time; returns (payload, scale_inv)."""
    import torch
    from msamp import _backend
    g = torch.Generator(device='cuda').manual_seed(seed)
    x = torch.randn(shape, device='cuda', dtype=torch.bfloat16, generator=g)
    if std != 1.0:
        x *= std
    s, si, am = new_meta()
    q = _backend.cast_to_fp8_intime(x, s, am, si, fp8_dt)
    return q, si


# ---- FP8Linear steps through the msamp API -------------------------------------------------------------------
def bench_layer(cfg, steps, warmup, micro_batches=1, in_time=False):
    """Forward + backward of every projection of `cfg` as FP8Linear modules, then the amax-window update.  With
    in_time the metas are held in their warm-up phase (the counters of the amax windows are put back to zero after
    every update: two more tiny launches per step), so that every activation cast is an in-time one (amax, scale and
    cast of the same tensor) as in the first sixteen steps of a run.  With
    micro_batches > 1 every projection runs that many forward + backward passes before its gradient is dropped: from
    the second on, the weight-gradient GEMM adds into the dequantized FP8 gradient of the passes before and the sum
    is cast to E4M3 again (gradient accumulation)."""
    import torch
    import msamp    # noqa: F401
    from msamp import _backend
    from msamp.common.dtype import Dtypes
    from msamp.nn import LinearReplacer, model_state
    from msamp.optim import LBAdamW
    import msamp.operators.gemm.gemm as gemm_mod

    tokens = cfg['tokens']
    g = torch.Generator(device='cuda').manual_seed(0)
    layers = torch.nn.ModuleList()
    inputs, ograds = {}, []
    flops = 0.0
    for _, d_out, d_in in cfg['proj']:
        lin = torch.nn.Linear(d_in, d_out, bias=False, device='cuda', dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(torch.randn(d_out, d_in, device='cuda', generator=g) * 0.02)
        layers.append(lin)
        if d_in not in inputs:
            inputs[d_in] = torch.randn(tokens, d_in, device='cuda', generator=g).bfloat16().requires_grad_(True)
        ograds.append((torch.randn(tokens, d_out, device='cuda', generator=g) * 1e-3).bfloat16())
        flops += 3 * 2.0 * tokens * d_in * d_out
    model_state.clear()
    model = LinearReplacer.replace(layers, Dtypes.kbfloat16)
    opt = LBAdamW(model.parameters())    # only its scaling-factor update runs here

    gemm_events = []
    real_gemm, real_gemm_cast = _backend.fp8_gemm, _backend.fp8_gemm_cast

    class _Timed:
        enabled = False

        @staticmethod
        def _flops(a, out, a_kmajor):
            return 2.0 * out.numel() * (a.shape[0] if a_kmajor else a.shape[1])

        @staticmethod
        def fp8_gemm(a, a_dt, a_si, b, b_dt, b_si, out, accumulate=False, bias=None, a_kmajor=False, b_kmajor=False):
            if not _Timed.enabled:
                return real_gemm(a, a_dt, a_si, b, b_dt, b_si, out, accumulate, bias, a_kmajor=a_kmajor, b_kmajor=b_kmajor)
            s, e = _events()
            s.record()
            real_gemm(a, a_dt, a_si, b, b_dt, b_si, out, accumulate, bias, a_kmajor=a_kmajor, b_kmajor=b_kmajor)
            e.record()
            gemm_events.append((s, e, _Timed._flops(a, out, a_kmajor)))
            return out

        @staticmethod
        def fp8_gemm_cast(a, *args, **kwargs):
            # the weight-gradient GEMM with its cast to E4M3 fused in: one launch, timed as the GEMM it is
            if not _Timed.enabled:
                return real_gemm_cast(a, *args, **kwargs)
            s, e = _events()
            s.record()
            out = real_gemm_cast(a, *args, **kwargs)
            e.record()
            if out is not None:
                gemm_events.append((s, e, _Timed._flops(a, out, kwargs.get('a_kmajor', False))))
            return out

        def __getattr__(self, name):
            return getattr(_backend, name)

    gemm_mod._backend = _Timed()

    def step():
        for lin, dy in zip(model, ograds):
            x = inputs[lin.in_features]
            for _ in range(micro_batches):
                lin(x).backward(dy)
                x.grad = None
            lin.weight.grad = None
        opt._update_scaling_factors()
        if in_time:
            for name in ('input', 'ograd'):
                model_state.flattened_scaling_metas[name]['amax_counters'].zero_()

    try:
        for _ in range(SCALING_WARMUP_STEPS):    # untimed set-up: fill the amax windows
            step()
        assert model[0].scaling_metas['input'].is_in_time_scaling() == in_time
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            # an event pair costs the stream a few microseconds: bracket the GEMMs of every fourth step only
            _Timed.enabled = i % GEMM_EVENT_STRIDE == 0
            step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    finally:
        _Timed.enabled = False
        gemm_mod._backend = _backend
        model_state.clear()

    ms_per_step = dt / steps * 1e3
    gemm_ms_total = sum(s.elapsed_time(e) for s, e, _ in gemm_events)
    gemm_flops_total = sum(f for _, _, f in gemm_events)
    return {
        'ms_per_step': ms_per_step,
        'step_tflops': micro_batches * flops / (ms_per_step * 1e-3) / 1e12,
        'gemm_tflops': gemm_flops_total / (gemm_ms_total * 1e-3) / 1e12,
        'gemm_avg_launch_ms': gemm_ms_total / len(gemm_events),
        'gemm_avg_launch_flops': gemm_flops_total / len(gemm_events),
        'gemm_launches': len(gemm_events),
        'gemms_per_step': 3 * len(cfg['proj']) * micro_batches,
    }


# ---- GEMM sweep: one row per projection and pass, straight through the C ABI -------------------------------------
def bench_gemm_sweep(cfg, iters=10, accumulate_row=None, vendor=True):
    """Forward (E4M3 x E4M3), dgrad (W K-major, dy E5M2) and wgrad (x and dy K-major) of every projection, bf16
    out, operands drawn as the configs describe them and cast to FP8 by the library."""
    import torch
    from msamp import _backend
    E4, E5 = _backend.DT_E4M3, _backend.DT_E5M2
    tokens = cfg['tokens']
    rows, seen = [], {}
    acts = {}
    for name, d_out, d_in in cfg['proj']:
        if (d_out, d_in) in seen:    # gate and up: same problem, measured once, counted twice in the aggregate
            for r in seen[(d_out, d_in)]:
                rows.append(dict(r, proj=name))
            continue
        if d_in not in acts:
            acts[d_in] = fp8_randn((tokens, d_in), 1.0, E4, seed=d_in)
        x, x_si = acts[d_in]
        w, w_si = fp8_randn((d_out, d_in), 0.02, E4, seed=d_out + 1)
        dy, dy_si = fp8_randn((tokens, d_out), 1e-3, E5, seed=d_out + 2)
        y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
        dx = torch.empty(tokens, d_in, dtype=torch.bfloat16, device='cuda')
        dw = torch.empty(d_out, d_in, dtype=torch.bfloat16, device='cuda')
        passes = [
            ('fwd', lambda: _backend.fp8_gemm(w, E4, w_si, x, E4, x_si, y), (d_out, tokens, d_in)),
            ('dgrad', lambda: _backend.fp8_gemm(w, E4, w_si, dy, E5, dy_si, dx, a_kmajor=True), (d_in, tokens, d_out)),
            ('wgrad', lambda: _backend.fp8_gemm(x, E4, x_si, dy, E5, dy_si, dw, a_kmajor=True, b_kmajor=True),
             (d_in, d_out, tokens)),
        ]
        if accumulate_row == name:
            passes.append(('wgrad_accumulate',
                           lambda: _backend.fp8_gemm(x, E4, x_si, dy, E5, dy_si, dw, accumulate=True, a_kmajor=True, b_kmajor=True),
                           (d_in, d_out, tokens)))
        # For scale: the vendor library (hipBLASLt through torch._scaled_mm) on the same problem sizes and the same
        # bytes, E4M3 x E4M3 into bf16 with K-contiguous operands (the transposed copies it needs for dgrad and wgrad are
        # made outside the timed region).
        dy4 = fp8_randn((tokens, d_out), 1e-3, E4, seed=d_out + 2)[0] if vendor else None
        vendor_ops = {'fwd': (x, w), 'dgrad': (dy4, lambda: w.t().contiguous()), 'wgrad': (lambda: dy4.t().contiguous(),
                                                                                    lambda: x.t().contiguous())}
        mine = []
        for pname, fn, (m, n, k) in passes:
            ms = _time_gpu(fn, iters, settle_ms=30.0, batches=3)
            fl = 2.0 * m * n * k
            tf = fl / (ms * 1e-3) / 1e12
            row = {'proj': name, 'pass': pname, 'm': m, 'n': n, 'k': k, 'ms': round(ms, 4), 'tflops': round(tf, 1),
                   'frac_mfma': round(tf / FP8_PEAK_TFLOPS, 4)}
            if vendor and pname in vendor_ops:
                vms = _time_vendor(*vendor_ops[pname], iters)
                if vms is not None:
                    row['hipblaslt_ms'] = round(vms, 4)
                    row['hipblaslt_tflops'] = round(fl / (vms * 1e-3) / 1e12, 1)
            mine.append(row)
        seen[(d_out, d_in)] = mine
        rows.extend(mine)
        del w, dy, dy4, y, dx, dw
    core = [r for r in rows if r['pass'] in ('fwd', 'dgrad', 'wgrad')]
    fl = sum(2.0 * r['m'] * r['n'] * r['k'] for r in core)
    ms = sum(r['ms'] for r in core)
    agg = fl / (ms * 1e-3) / 1e12
    aggregate = {'flops': fl, 'ms': round(ms, 3), 'tflops': round(agg, 1), 'frac_mfma': round(agg / FP8_PEAK_TFLOPS, 4),
                 'gemms': len(core)}
    if core and all('hipblaslt_ms' in r for r in core):
        vms = sum(r['hipblaslt_ms'] for r in core)
        aggregate['hipblaslt_ms'] = round(vms, 3)
        aggregate['hipblaslt_tflops'] = round(fl / (vms * 1e-3) / 1e12, 1)
    return {'rows': rows, 'aggregate': aggregate}


def bench_small_gemms(iters=50):
    """The three GEMMs of layers too small to fill the chip with 256 x 256 tiles (64 of them per output and fewer):
    the library's pick (128 x 128 tiles), the large tile forced, and hipBLASLt on the forward problem."""
    import torch
    from msamp import _backend
    E4, E5 = _backend.DT_E4M3, _backend.DT_E5M2
    rows = []
    for tokens, d_out, d_in in ((2048, 2048, 4096), (1024, 4096, 4096)):
        x, x_si = fp8_randn((tokens, d_in), 1.0, E4, seed=tokens)
        w, w_si = fp8_randn((d_out, d_in), 0.02, E4, seed=d_out + 1)
        dy, dy_si = fp8_randn((tokens, d_out), 1e-3, E5, seed=d_out + 2)
        y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
        dx = torch.empty(tokens, d_in, dtype=torch.bfloat16, device='cuda')
        dw = torch.empty(d_out, d_in, dtype=torch.bfloat16, device='cuda')
        passes = [
            ('fwd', lambda: _backend.fp8_gemm(w, E4, w_si, x, E4, x_si, y), (d_out, tokens, d_in)),
            ('dgrad', lambda: _backend.fp8_gemm(w, E4, w_si, dy, E5, dy_si, dx, a_kmajor=True), (d_in, tokens, d_out)),
            ('wgrad', lambda: _backend.fp8_gemm(x, E4, x_si, dy, E5, dy_si, dw, a_kmajor=True, b_kmajor=True), (d_in, d_out, tokens)),
        ]
        for pname, fn, (m, n, k) in passes:
            fl = 2.0 * m * n * k
            ms = _time_gpu(fn, iters)
            try:
                _backend.set_small_tile_limit(0)
                ms_large = _time_gpu(fn, iters)
            finally:
                _backend.set_small_tile_limit(128)
            row = {'tokens': tokens, 'pass': pname, 'm': m, 'n': n, 'k': k, 'ms': round(ms, 4), 'tflops': round(fl / ms / 1e9, 1),
                   'frac_mfma': round(fl / ms / 1e9 / FP8_PEAK_TFLOPS, 4),
                   'large_tile_ms': round(ms_large, 4), 'large_tile_tflops': round(fl / ms_large / 1e9, 1)}
            if pname == 'fwd':
                vms = _time_vendor(x, w, iters)
                if vms is not None:
                    row['hipblaslt_ms'] = round(vms, 4)
                    row['hipblaslt_tflops'] = round(fl / vms / 1e9, 1)
            rows.append(row)
    return rows


def _time_vendor(rows_op, cols_op, iters):
    """torch._scaled_mm (hipBLASLt) on FP8 payloads: out[n, m] = rows_op[n, k] . cols_op[m, k]^T, unit scales, bf16 out.
    Operands are uint8 payloads or callables that make them; None if this build of torch does not take the call."""
    import torch
    try:
        a = (rows_op() if callable(rows_op) else rows_op).view(torch.float8_e4m3fn)
        b = (cols_op() if callable(cols_op) else cols_op).view(torch.float8_e4m3fn)
        one = torch.ones((), device='cuda')
        fn = lambda: torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        fn()
        torch.cuda.synchronize()
        return _time_gpu(fn, iters, settle_ms=30.0, batches=3)
    except (RuntimeError, AttributeError, TypeError):
        return None


# ---- cast group ----------------------------------------------------------------------------------------------
def bench_cast(iters=20):
    """cast+amax throughput: C1 (fp32 [4096,4096], in-time, E4M3 / E5M2, dequantize), steady-state delayed cast of
    bf16 [8192,4096], and the in-time cast of one Llama-70B MLP weight (bf16 [28672,8192], N(0,0.01) with 0.01 %
    outliers x 50) and of the whole layer's 855 638 016 weight elements.  Rows marked `cache_resident` run one working
    set of at most 96 MiB over and over, which the 256 MiB memory-side cache then serves: their fraction of the HBM
    peak is reached out of that cache.  The `_cold` rows walk through enough distinct buffers that nothing of an
    input is left in any cache when its turn comes again (how a training step meets its activations); `_miss` rows
    alternate two inputs whose amax differ by a factor of two, so that the scale the kernel speculates on is wrong every
    time; `_fresh_meta` rows use a new meta per call (nothing to speculate on: the input is read twice)."""
    import torch
    from msamp import _backend
    out = {}
    E4, E5 = _backend.DT_E4M3, _backend.DT_E5M2

    def row(name, ms, nbytes, resident=False):
        out[name] = {'ms': ms, 'GBps': nbytes / ms / 1e6}
        if resident:
            out[name]['cache_resident'] = True

    def in_turn(items, call):
        turn = {'i': 0}

        def fn():
            turn['i'] = (turn['i'] + 1) % len(items)
            call(items[turn['i']])
        return fn

    x = c1_input(0).cuda()
    n1 = x.numel()
    s, si, am = new_meta()
    row('c1_intime_fp32_e4m3', _time_gpu(lambda: _backend.cast_to_fp8_intime(x, s, am[0:1], si, E4), iters), n1 * 5, resident=True)
    row('c1_intime_fp32_e5m2', _time_gpu(lambda: _backend.cast_to_fp8_intime(x, s, am[0:1], si, E5), iters), n1 * 5, resident=True)
    q = _backend.cast_to_fp8_intime(x, s, am[0:1], si, E4)
    row('c1_dequant_e4m3_fp32', _time_gpu(lambda: _backend.cast_from_fp8(q, si, E4, torch.float32), iters), n1 * 5, resident=True)
    # eight distinct 64 MiB inputs in turn (512 MiB, twice the memory-side cache)
    xs = [x] + [torch.randn_like(x) for _ in range(7)]
    row('c1_intime_fp32_e4m3_cold', _time_gpu(in_turn(xs, lambda t: _backend.cast_to_fp8_intime(t, s, am[0:1], si, E4)), 2 * len(xs), warm=len(xs)), n1 * 5)
    # the guess wrong every time: x and 2x in turn on one meta (each call finds the other's scale)
    pair = [x, x * 2]
    row('c1_intime_fp32_e4m3_miss', _time_gpu(in_turn(pair, lambda t: _backend.cast_to_fp8_intime(t, s, am[0:1], si, E4)), iters, warm=4), n1 * 5,
        resident=True)
    metas = [new_meta() for _ in range(iters + 4)]
    row('c1_intime_fp32_e4m3_fresh_meta',
        _time_gpu(in_turn(metas, lambda m: _backend.cast_to_fp8_intime(x, m[0], m[2][0:1], m[1], E4)), iters, warm=3), n1 * 5, resident=True)
    qs = [_backend.cast_to_fp8_intime(t, s, am[0:1], si, E4) for t in xs] + [torch.randint(0, 120, x.shape, dtype=torch.uint8, device='cuda')
                                                                             for _ in range(8)]
    row('c1_dequant_e4m3_fp32_cold', _time_gpu(in_turn(qs, lambda t: _backend.cast_from_fp8(t, si, E4, torch.float32)), 2 * len(qs), warm=len(qs)),
        n1 * 5)
    del x, q, xs, qs, pair
    a = torch.randn(8192, 4096, device='cuda').bfloat16()
    n2 = a.numel()
    row('c2_delayed_bf16_e4m3', _time_gpu(lambda: _backend.cast_to_fp8(a, s, am[0:1], si, E4), iters), n2 * 3, resident=True)
    row('c2_cast_transpose_bf16_e5m2', _time_gpu(lambda: _backend.cast_transpose(a, s, am[0:1], si, E5), iters), n2 * 4, resident=True)
    qa = _backend.cast_to_fp8(a, s, am[0:1], si, E4)
    row('c2_fp8_transpose', _time_gpu(lambda: _backend.fp8_transpose(qa), iters), n2 * 2, resident=True)
    # the same three over eight distinct 64 MiB activations (and sixteen 32 MiB payloads) in turn
    acts = [a] + [torch.randn(8192, 4096, device='cuda').bfloat16() for _ in range(7)]
    row('c2_delayed_bf16_e4m3_cold', _time_gpu(in_turn(acts, lambda t: _backend.cast_to_fp8(t, s, am[0:1], si, E4)), 2 * len(acts), warm=len(acts)),
        n2 * 3)
    row('c2_cast_transpose_bf16_e5m2_cold',
        _time_gpu(in_turn(acts, lambda t: _backend.cast_transpose(t, s, am[0:1], si, E5)), 2 * len(acts), warm=len(acts)), n2 * 4)
    pays = [_backend.cast_to_fp8(t, s, am[0:1], si, E4) for t in acts] + [torch.randint(0, 120, (8192, 4096), dtype=torch.uint8, device='cuda')
                                                                           for _ in range(8)]
    row('c2_fp8_transpose_cold', _time_gpu(in_turn(pays, lambda t: _backend.fp8_transpose(t)), 2 * len(pays), warm=len(pays)), n2 * 2)
    del a, qa, acts, pays

    def c5_weight(d_out, d_in, seed):
        g = torch.Generator(device='cuda').manual_seed(seed)
        w = torch.randn(d_out, d_in, device='cuda', generator=g) * 0.01
        idx = torch.randint(0, w.numel(), (w.numel() // 10000, ), device='cuda', generator=g)
        w.view(-1)[idx] *= 50
        return w.bfloat16()

    weights = [c5_weight(d_out, d_in, 100 + i) for i, (_, d_out, d_in) in enumerate(LLAMA_70B['proj'])]
    wmetas = [new_meta() for _ in weights]
    w = weights[2]    # gate: [28672, 8192], 234 881 024 elements
    row('c5_intime_bf16_e4m3_235M', _time_gpu(lambda: _backend.cast_to_fp8_intime(w, s, am[0:1], si, E4), max(iters // 2, 5)), w.numel() * 3)
    pair = [w, w * 2]
    row('c5_intime_bf16_e4m3_235M_miss', _time_gpu(in_turn(pair, lambda t: _backend.cast_to_fp8_intime(t, s, am[0:1], si, E4)), 6, warm=2),
        w.numel() * 3)
    del pair
    row('c5_intime_bf16_e4m3_235M_fresh_meta',
        _time_gpu(in_turn(metas, lambda m: _backend.cast_to_fp8_intime(w, m[0], m[2][0:1], m[1], E4)), 6, warm=2), w.numel() * 3)

    def layer_cast():
        for wt, (ws, wsi, wam) in zip(weights, wmetas):
            _backend.cast_to_fp8_intime(wt, ws, wam[0:1], wsi, E4)

    n_layer = sum(wt.numel() for wt in weights)
    row('c5_intime_bf16_e4m3_layer_856M', _time_gpu(layer_cast, 5, warm=2), n_layer * 3)
    del w, weights
    # what a plain copy reaches on this box (the practical ceiling of the streaming kernels above): 256 MiB of
    # fp32 through the library's scale_cast at scale 1, read once, written once
    src = torch.ones(64 * 1024 * 1024, device='cuda')
    one = torch.ones((), device='cuda')
    row('copy_fp32_256MiB', _time_gpu(lambda: _backend.scale_cast(src, one, torch.float32), max(iters // 2, 5)), src.numel() * 8)
    return out


def bench_grad_side(iters=10):
    """The reducer's compute steps on one bucket of 32 bf16 gradients of [4096,1024] (amax, scales, quantize
    into the flat E4M3 buffer: 2 B read + 1 B written per element when the scales of the round before hold, the
    input read a second time otherwise), and the per-tensor 2-norms of 64 such FP8 gradients (1 B read per element)."""
    import torch
    from msamp import _backend
    from msamp.nn import GradientBucket
    n = 4096 * 1024
    grads = [(torch.randn(n, device='cuda') * 1e-3).bfloat16() for _ in range(32)]
    bucket = GradientBucket([n] * len(grads))
    out = {}
    ms = _time_gpu(lambda: bucket.quantize(grads, world_size=8), iters)
    out['bucket_quantize_32x4M_bf16'] = {'ms': ms, 'GBps': n * len(grads) * 3 / ms / 1e6}
    # the same through the two C entry points alone, tables built once (what the launches cost without the Python around them)
    import math
    items, block_map = bucket._get_tables(grads)
    in_dt = _backend._dt(grads[0])

    def two_calls():
        _backend.bucket_amax(items, block_map, in_dt, nan_to_inf=True, speculate_fp8_dt=int(bucket.qtype))
        _backend.bucket_cast(items, block_map, in_dt, int(bucket.qtype), 1.0 / math.sqrt(8), 8.0)

    ms = _time_gpu(two_calls, iters)
    out['bucket_quantize_32x4M_bf16_entry_points_only'] = {'ms': ms, 'GBps': n * len(grads) * 3 / ms / 1e6}
    # beside it: without the codes going out during the amax pass (input read twice)
    bucket = GradientBucket([n] * len(grads), speculate=False)
    ms = _time_gpu(lambda: bucket.quantize(grads, world_size=8), iters)
    out['bucket_quantize_32x4M_bf16_two_reads'] = {'ms': ms, 'GBps': n * len(grads) * 3 / ms / 1e6}
    del grads, bucket
    qs = [torch.randint(0, 120, (n,), dtype=torch.uint8, device='cuda') for _ in range(64)]
    sis = [torch.ones((), device='cuda') for _ in qs]
    ms = _time_gpu(lambda: _backend.fp8_norms(qs, sis, _backend.DT_E4M3, 2.0), iters)
    out['fp8_l2_norms_64x4M_e4m3'] = {'ms': ms, 'GBps': n * len(qs) / ms / 1e6}
    return out


def bench_adam(iters=10, total_params=1_000_000_000):
    """Fused LBAdamW step over 1.0e9 parameters held as [4096,1024] tensors (last one truncated): E4M3 weights, E5M2
    grads, E4M3 exp_avg, scaled-fp16 exp_avg_sq.  Timed through msamp.optim.LBAdamW.step() itself (239
    ScalingParameters with FP8 gradients) in its three forms -- in place (default), one pass inside shifting arenas
    (one_pass='shift'), one pass between two sets of buffers (one_pass='double') -- and, for the arena form, through
    the C entry point alone on the tables the optimizer built, which shows what the Python around it costs."""
    import torch
    import msamp    # noqa: F401
    from msamp import _backend
    from msamp.common.dtype import Dtypes
    from msamp.nn import ScalingParameter
    from msamp.optim import LBAdamW
    per = 4096 * 1024
    sizes = [per] * (total_params // per)
    if total_params % per:
        sizes.append(total_params % per)
    g = torch.Generator(device='cuda').manual_seed(3)
    params = []
    for n in sizes:
        shape = (4096, 1024) if n == per else (n, )
        w = torch.randn(shape, device='cuda', generator=g) * 0.02
        p = ScalingParameter(w.cast(Dtypes.kfloat8_e4m3))
        p.grad = (torch.randn(shape, device='cuda', generator=g) * 1e-3).cast(Dtypes.kfloat8_e5m2)
        params.append(p)
        del w
    hyper = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    out = {'params': total_params, 'tensors': len(sizes)}

    def redone(opt):
        return sum(int(plan.redo.sum().item()) for plan in opt._plans.values() if plan.redo is not None)

    for mode, name in ((None, 'in_place'), ('shift', 'shift'), ('double', 'double')):
        opt = LBAdamW(params, one_pass=mode, **hyper)
        # The one-pass forms pay for every tensor whose power-of-two scales move (that tensor is done again).  Two
        # figures: after 40 steps the moments are still travelling from zero to where this (constant) gradient takes
        # them and their scales move every few steps -- and since all 239 tensors hold data of one distribution they
        # move in the same steps; after 150 more the state has settled and no scale moves, which is the long-run case.
        ms_moving = _time_gpu(opt.step, iters, warm=40)
        moving_redone = redone(opt)
        ms = _time_gpu(opt.step, 3 * iters, warm=150)    # (long enough that the first step's host time does not show)
        row = {'ms': ms, 'ms_while_scales_move': ms_moving, 'extra_bytes_per_param': opt.extra_bytes() / total_params}
        if mode is not None:
            row['tensors_redone_in_last_step'] = redone(opt)
            row['tensors_redone_while_scales_move'] = moving_redone
        # host time of one step (the launches are asynchronous: this is what the CPU spends per step)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            opt.step()
        row['host_ms_per_step'] = (time.perf_counter() - t0) / 5 * 1e3
        torch.cuda.synchronize()
        if mode == 'shift':
            # the same step through the C entry point alone, on the optimizer's own tables (the payloads end up where
            # they started: an even number of calls)
            plan = next(iter(opt._plans.values()))
            wq, gq = int(Dtypes.kfloat8_e4m3), int(Dtypes.kfloat8_e5m2)
            state = {'phase': plan.phase, 't': opt.state[params[0]]['step']}

            def entry():
                state['t'] += 1
                ph = state['phase']
                shift = (-plan.slack if ph == 0 else plan.slack) * _backend.ADAMW_CHUNK
                _backend.adamw_fused_shift(plan.desc[('shift', ph)], plan.redo, plan.sync, len(params), plan.block_map, plan.n_blocks,
                                           shift, wq, gq, 3e-4, 0.9, 0.95, 1e-8, 0.1, state['t'], True, False, False, True)
                state['phase'] = 1 - ph

            row['entry_point_ms'] = _time_gpu(entry, 3 * iters, warm=2)
            assert state['phase'] == plan.phase
            row['slack_chunks'] = plan.slack
        out[name] = row
        del opt
        torch.cuda.empty_cache()
    del params
    torch.cuda.empty_cache()
    # float32 moments (the reference's opt_level O1 keeps them so): 16 float32 parameters of 4096 x 4096 with float32
    # gradients, stepped by the one-pass kernel and by the reference's chain of element-wise calls; 28 B/param (read p, g,
    # m, v; write p, m, v)
    plain = [torch.nn.Parameter(torch.randn(4096, 4096, device='cuda', generator=g) * 0.02) for _ in range(16)]
    for p in plain:
        p.grad = torch.randn(4096, 4096, device='cuda', generator=g) * 1e-3
    n_plain = sum(p.numel() for p in plain)
    opt = LBAdamW(plain, exp_avg_dtype=torch.float32, exp_avg_sq_dtype=torch.float32, **hyper)
    row = {'params': n_plain, 'ms': _time_gpu(opt.step, iters, warm=3)}
    kernel_step = LBAdamW._f32_step
    LBAdamW._f32_step = lambda self, *a, **k: False
    try:
        row['ms_as_torch_calls'] = _time_gpu(opt.step, iters, warm=3)
    finally:
        LBAdamW._f32_step = kernel_step
    row['hbm_frac'] = n_plain * 28 / (row['ms'] * 1e-3) / 8e12
    out['float32_moments'] = row
    del opt, plain
    # what a model keeps in high precision beside its FP8 weights: 64 bfloat16 vectors of 4096 .. 11008 elements with E4M3 /
    # scaled-float16 moments.  One launch for all of them against the reference's recipe tensor by tensor (two stages and
    # two reads of the amaxs by the host per tensor); wall time, since the recipe is bound by the host
    small = [torch.nn.Parameter(torch.randn(4096 if i % 2 else 11008, device='cuda', generator=g).bfloat16()) for i in range(64)]
    for p in small:
        p.grad = (torch.randn(p.shape, device='cuda', generator=g) * 1e-3).bfloat16()
    opt = LBAdamW(small, **hyper)

    def wall_ms(n=20):
        for _ in range(3):
            opt.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            opt.step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    row = {'tensors': len(small), 'wall_ms': wall_ms()}
    fusable = LBAdamW._plain_fusable
    LBAdamW._plain_fusable = classmethod(lambda cls, *a: False)
    opt._groups = None
    try:
        row['wall_ms_tensor_by_tensor'] = wall_ms()
    finally:
        LBAdamW._plain_fusable = fusable
    out['small_plain_parameters'] = row
    del opt, small
    # an embedding kept in bfloat16 (32000 x 4096) with E4M3 / scaled-float16 moments: the same step chunk by chunk in
    # three launches (19 B/param: read p, g, m, v, write p; read g, m, v, write m, v) against the recipe tensor by tensor
    emb = torch.nn.Parameter((torch.randn(32000, 4096, device='cuda', generator=g) * 0.02).bfloat16())
    emb.grad = (torch.randn(32000, 4096, device='cuda', generator=g) * 1e-3).bfloat16()
    opt = LBAdamW([emb], **hyper)
    row = {'params': emb.numel(), 'ms': _time_gpu(opt.step, iters, warm=3)}
    row['hbm_frac'] = emb.numel() * 19 / (row['ms'] * 1e-3) / 8e12
    LBAdamW._plain_fusable = classmethod(lambda cls, *a: False)
    opt._groups = None
    try:
        row['ms_tensor_by_tensor'] = _time_gpu(opt.step, iters, warm=3)
    finally:
        LBAdamW._plain_fusable = fusable
    out['plain_embedding'] = row
    return out


# ---- CPU baseline: the oracle on the host cores --------------------------------------------------------------
def cpu_baseline():
    """The oracle (PyTorch CPU restatement of the reference math) on a bounded sample, all host cores: the
    config-1 cast at full size, the config-3 AdamW step on 16 of its [4096,1024] tensors, the config-5 cast of one
    [28672,8192] weight, and the GEMM definition (fp32 matmul of dequantized operands) on a slice of config 2."""
    import torch
    from oracle import adamw as oadam, cast as ocast, fp8
    # the box sets OMP_NUM_THREADS to its CPU share; never spread over more threads than that
    cores = min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', '16') or 16))
    torch.set_num_threads(cores)

    def med(fn, runs=5, warm=2):
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(runs):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    x = c1_input(0)
    t = med(lambda: ocast.cast_to_fp8(x, ocast.new_meta(), fp8.E4M3, in_time=True))
    cast_gbps = x.numel() * 5 / t / 1e9
    del x

    n = 4096 * 1024
    n_tensors = 16

    def adam_inputs(seed):
        g = torch.Generator().manual_seed(seed)

        def quant(v, fmt):
            meta = ocast.new_meta()
            return ocast.cast_to_fp8(v, meta, fmt, in_time=True), meta

        w, wm = quant(0.02 * torch.randn(n, generator=g), fp8.E4M3)
        gq, gm = quant(1e-3 * torch.randn(n, generator=g), fp8.E5M2)
        m, mm = quant((1e-4 * torch.randn(n, generator=g)).abs(), fp8.E4M3)
        vm = ocast.new_meta()
        v = ocast.cast_to_fp16((1e-4 * torch.randn(n, generator=g)).abs(), vm, in_time=True)
        return dict(w=w, wm=wm, g=gq, gm=gm, m=m, mm=mm, v=v, vm=vm)

    tens = [adam_inputs(i) for i in range(n_tensors)]

    def adam():
        for d in tens:
            oadam.step_tensor(d['w'], d['wm'], fp8.E4M3, d['g'], d['gm']['scale_inv'], fp8.E5M2, d['m'], d['mm'], d['v'], d['vm'],
                              lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=2)

    ta = med(adam, runs=3, warm=1)
    adam_gps = n_tensors * n / ta / 1e9
    del tens

    g = torch.Generator().manual_seed(5)
    w5 = torch.randn(28672, 8192, generator=g) * 0.01
    idx = torch.randint(0, w5.numel(), (w5.numel() // 10000, ), generator=g)
    w5.view(-1)[idx] *= 50
    w5 = w5.bfloat16()
    t5 = med(lambda: ocast.cast_to_fp8(w5, ocast.new_meta(), fp8.E4M3, in_time=True), runs=3, warm=1)
    c5_gbps = w5.numel() * 3 / t5 / 1e9
    del w5

    # GEMM definition (fp32 matmul of dequantized operands) on 1024 of the 8192 token rows of config 2
    a = fp8.decode(fp8.encode(torch.randn(4096, 4096) * 0.02 * 64, fp8.E4M3), fp8.E4M3)
    b = fp8.decode(fp8.encode(torch.randn(1024, 4096), fp8.E4M3), fp8.E4M3)
    tg = med(lambda: b @ a.t(), runs=5, warm=1)
    gemm_tflops = 2.0 * 1024 * 4096 * 4096 / tg / 1e12
    return {
        'value': gemm_tflops, 'unit': 'TFLOP/s', 'cores': cores, 'threads': torch.get_num_threads(), 'kind': 'port',
        'sample': 'gemm: fp32 matmul of dequantized operands, 1024 of the 8192 token rows of the config-2 forward GEMM; '
                  'cast: full config-1 tensor fp32[4096,4096] in-time E4M3 (median of 5) and one config-5 weight '
                  'bf16[28672,8192] (median of 3); adam: 16 of the 239 config-3 tensors [4096,1024] (median of 3)',
        'cast_amax': {'value': cast_gbps, 'unit': 'GB/s (5 B/elt, config 1)'},
        'cast_amax_c5': {'value': c5_gbps, 'unit': 'GB/s (3 B/elt, config 5 weight)'},
        'fp8_adam': {'value': adam_gps, 'unit': 'Gparams/s', 'tensors': n_tensors},
    }


def bench_power(seconds=2.0):
    """Socket power and shader clock, sampled from the amdgpu driver's sysfs files at 20 Hz by a host thread, while
    (a) nothing runs, (b) the FP8 GEMMs of the Llama-70B gate projection [16384 x 28672 x 8192] and of the Llama-7B QKV
    projection [16384 x 12288 x 4096] and (c) a register-only FP8 MFMA loop (msamp_mfma_probe) each run back to back for
    `seconds`.  Reported so that a GEMM rate can be read
    against what the matrix pipes sustain under the device's power limit, not only against the nominal peak."""
    import glob
    import threading
    import torch
    from msamp import _backend as be

    def first(pattern):
        hits = sorted(glob.glob(pattern))
        return hits[0] if hits else None

    hwmon = '/sys/class/drm/card*/device/hwmon/hwmon*/'
    power = first(hwmon + 'power1_average') or first(hwmon + 'power1_input')
    cap = first(hwmon + 'power1_cap')
    dpm = first('/sys/class/drm/card*/device/pp_dpm_sclk')

    def read(path):
        try:
            with open(path) as f:
                return f.read().strip()
        except (OSError, TypeError):
            return None

    def clock_now():
        for line in (read(dpm) or '').splitlines():
            if line.endswith('*'):
                return float(line.split()[1].lower().replace('mhz', ''))
        return None

    def sample_while(fn, duration):
        fn()
        torch.cuda.synchronize()
        watts, mhz, stop = [], [], threading.Event()

        def sampler():
            while not stop.is_set():
                p, c = read(power), clock_now()
                if p is not None and p.isdigit():
                    watts.append(int(p) / 1e6)
                if c is not None:
                    mhz.append(c)
                time.sleep(0.05)

        th = threading.Thread(target=sampler)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        th.start()
        t0, calls = time.perf_counter(), 0
        e0.record()
        while time.perf_counter() - t0 < duration:
            for _ in range(20):
                fn()
            calls += 20
            torch.cuda.synchronize()
        e1.record()
        e1.synchronize()
        stop.set()
        th.join()

        def mmm(v):
            # the first quarter second holds the ramp from idle
            v = v[5:] if len(v) > 10 else v
            return {'min': round(min(v)), 'mean': round(sum(v) / len(v)), 'max': round(max(v))} if v else None

        return e0.elapsed_time(e1) / calls, {'samples': len(watts), 'power_W': mmm(watts), 'sclk_MHz': mmm(mhz)}

    out = {'sources': {'power': power, 'clock': dpm}, 'power_cap_W': None}
    if read(cap) and read(cap).isdigit():
        out['power_cap_W'] = int(read(cap)) / 1e6
    _, out['idle'] = sample_while(lambda: None, 1.0)

    tokens, d_out, d_in = 16384, 28672, 8192
    g = torch.Generator(device='cuda').manual_seed(1)

    def quantized(shape, std):
        x = (torch.randn(shape, device='cuda', generator=g) * std).bfloat16()
        s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
        return be.cast_to_fp8_intime(x, s, am, si, be.DT_E4M3), si

    x, xs = quantized((tokens, d_in), 1.0)
    w, ws = quantized((d_out, d_in), 0.02)
    y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
    ms, row = sample_while(lambda: be.fp8_gemm(w, be.DT_E4M3, ws, x, be.DT_E4M3, xs, y), seconds)
    row.update({'ms_per_call': round(ms, 4), 'TFLOPs': round(2.0 * tokens * d_out * d_in / ms / 1e9, 1)})
    out['fp8_gemm_16384x28672x8192'] = row
    # the vendor library on the same operands (hipBLASLt through torch._scaled_mm, its output allocated once): what it
    # draws and at which clock, for the comparison of the two kernels' energy per flop
    try:
        x8, w8 = x.view(torch.float8_e4m3fn), w.view(torch.float8_e4m3fn)
        one = torch.ones((), device='cuda')
        vendor = lambda: torch._scaled_mm(x8, w8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16, out=y)    # noqa: E731
        vendor()
        ms, row = sample_while(vendor, seconds)
        row.update({'ms_per_call': round(ms, 4), 'TFLOPs': round(2.0 * tokens * d_out * d_in / ms / 1e9, 1)})
        out['hipblaslt_16384x28672x8192'] = row
    except (RuntimeError, AttributeError, TypeError) as exc:
        out['hipblaslt_16384x28672x8192'] = {'skipped': str(exc)[:200]}
    del x, w, y

    # the forward GEMM of the Llama-7B QKV projection: K = 4096, where the time outside the K loop weighs most
    d_out, d_in = 12288, 4096
    x, xs = quantized((tokens, d_in), 1.0)
    w, ws = quantized((d_out, d_in), 0.02)
    y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
    ms, row = sample_while(lambda: be.fp8_gemm(w, be.DT_E4M3, ws, x, be.DT_E4M3, xs, y), seconds)
    row.update({'ms_per_call': round(ms, 4), 'TFLOPs': round(2.0 * tokens * d_out * d_in / ms / 1e9, 1)})
    out['fp8_gemm_16384x12288x4096'] = row
    del x, w, y

    seed = quantized((4096, ), 1.0)[0]
    sink = torch.zeros(1, device='cuda')
    flop = [0.0]

    for key, distinct in (('register_only_fp8_mfma_loop', False), ('register_only_fp8_mfma_loop_8x8_operands', True)):
        def probe():
            flop[0] = be.mfma_probe(seed, sink, 20000, 1024, distinct_operands=distinct)

        ms, row = sample_while(probe, seconds)
        row.update({'ms_per_call': round(ms, 4), 'TFLOPs': round(flop[0] / ms / 1e9, 1)})
        out[key] = row
    return out


def pmc_calibration_copy():
    """One plain copy of known size -- scale_cast fp32 -> fp32 at scale 1 over 64 Mi elements: 256 MiB read,
    256 MiB written -- so that a `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` run of this program holds a
    dispatch of known traffic to scale the counters by.  Untimed."""
    import torch
    from msamp import _backend
    src = torch.ones(64 * 1024 * 1024, device='cuda')
    _backend.scale_cast(src, torch.ones((), device='cuda'), torch.float32)
    torch.cuda.synchronize()


def measured_gemm_traffic():
    """(HBM bytes per GEMM launch of the headline step, where the figure comes from): the last rocprofv3 --pmc
    measurement on file under profiles/ -- a static figure, not taken in this run -- or (None, None)."""
    name = 'fp8_gemm_hbm_traffic.json'
    try:
        with open(os.path.join(ROOT, 'profiles', name)) as f:
            return json.load(f)['traffic_bytes_per_launch'], 'profiles/%s (static: measured with rocprofv3 --pmc, not in this run)' % name
    except (OSError, KeyError, ValueError):
        return None, None


def _round_kernels(d):
    out = {}
    for k, v in d.items():
        out[k] = {'ms': round(v['ms'], 4), 'GBps': round(v['GBps'], 1), 'frac_hbm': round(v['GBps'] / HBM_PEAK_GBS, 4)}
        if v.get('cache_resident'):
            out[k]['cache_resident'] = True
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--skip-cpu', action='store_true', help='leave out the CPU-oracle baseline')
    ap.add_argument('--skip-extra', action='store_true', help='leave out the sweep, cast and Adam kernel sections')
    ap.add_argument('--only', choices=('gemm_c2', 'gemm_c4', 'gemm_c5', 'gemm_llama3_8b', 'gemm_small', 'cast', 'adam', 'grad_side', 'power'), default=None,
                    help='run one kernel section alone (after the calibration copy), for profiling')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)', file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print('bench.py needs the GPU', file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    pmc_calibration_copy()
    if args.only:
        if args.only == 'gemm_c2':
            out = bench_gemm_sweep(CONFIG_2, iters=6)
        elif args.only == 'gemm_c4':
            out = bench_gemm_sweep(LLAMA_7B, iters=3, accumulate_row='gate')
        elif args.only == 'gemm_c5':
            out = bench_gemm_sweep(LLAMA_70B, iters=3)
        elif args.only == 'gemm_llama3_8b':
            out = bench_gemm_sweep(LLAMA3_8B, iters=3)
        elif args.only == 'cast':
            out = _round_kernels(bench_cast())
        elif args.only == 'grad_side':
            out = _round_kernels(bench_grad_side())
        elif args.only == 'power':
            out = bench_power()
        elif args.only == 'gemm_small':
            out = bench_small_gemms()
        else:
            out = bench_adam()
        from msamp import _backend as _be
        walks = {'%dx%dx%d%s%s' % (k[0], k[1], k[2], ' aT' if k[3] else '', ' bT' if k[4] else ''): w
                 for k, w in sorted(_be.gemm_walks().items())}
        print(json.dumps({'only': args.only, 'result': out, 'gemm_walks_timed_at_first_use': walks}))
        return

    lin = bench_layer(LLAMA_7B, args.steps, args.warmup)
    traffic, traffic_source = measured_gemm_traffic()
    result = {
        'metric': 'FP8 GEMM TFLOPS, cast+amax GB/s, FP8-Adam Gparams/s on 1 MI355X',
        'value': lin['step_tflops'],
        'unit': 'TFLOP/s (15 GEMMs of one Llama-7B layer of FP8Linear fwd+bwd / whole step incl. casts and window update)',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': lin['ms_per_step'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'fp8 (e4m3 x e4m3 / e4m3 x e5m2), fp32 accumulate',
        'data': 'synthetic',
        'config': {'workload': 'config 4: Llama-7B layer, every FP8Linear GEMM fwd+bwd at 16384 tokens (QKV [12288,4096], '
                               'O [4096,4096], gate/up [11008,4096], down [4096,11008]); x, dy bf16, W bf16 payload, delayed '
                               'scaling (history 16) after %d untimed scaling warm-up steps, outputs bf16, dW -> E4M3'
                               % SCALING_WARMUP_STEPS},
        'roofline': {
            'kernel': 'fp8_gemm_dma_kernel (flop-weighted over the 15 GEMM launches of the config-4 step)',
            'bound': 'mfma', 'achieved': lin['gemm_tflops'], 'peak': FP8_PEAK_TFLOPS, 'unit': 'TFLOP/s',
            'frac': lin['gemm_tflops'] / FP8_PEAK_TFLOPS, 'traffic': traffic, 'traffic_source': traffic_source,
            'avg_launch_ms': lin['gemm_avg_launch_ms'], 'avg_launch_flops': lin['gemm_avg_launch_flops'],
            'launches': lin['gemm_launches'],
        },
    }
    if not args.skip_extra:
        torch.cuda.empty_cache()
        c2 = bench_layer(CONFIG_2, max(args.steps, 200), args.warmup)
        result['c2_step'] = {
            'workload': 'config 2: single FP8Linear fwd+bwd, x bf16[8192,4096], W bf16[4096,4096], dy bf16[8192,4096]',
            'ms_per_step': round(c2['ms_per_step'], 4), 'step_tflops': round(c2['step_tflops'], 1),
            'gemm_tflops': round(c2['gemm_tflops'], 1), 'gemm_frac_mfma': round(c2['gemm_tflops'] / FP8_PEAK_TFLOPS, 4),
            'gemm_avg_launch_ms': round(c2['gemm_avg_launch_ms'], 4), 'gemm_launches': c2['gemm_launches'],
        }
        torch.cuda.empty_cache()
        acc = bench_layer(LLAMA_7B, max(args.steps // 4, 20), 2, micro_batches=2)
        result['c4_grad_accumulation_step'] = {
            'workload': 'config 4 with two micro-batches per step: the second weight-gradient GEMM of every projection adds '
                        'into the dequantized E4M3 gradient of the first and the sum is cast to E4M3 again',
            'ms_per_step': round(acc['ms_per_step'], 4), 'step_tflops': round(acc['step_tflops'], 1),
            'gemm_tflops': round(acc['gemm_tflops'], 1), 'gemm_frac_mfma': round(acc['gemm_tflops'] / FP8_PEAK_TFLOPS, 4),
            'gemm_launches': acc['gemm_launches'], 'gemms_per_step': acc['gemms_per_step'],
        }
        torch.cuda.empty_cache()
        warm = bench_layer(LLAMA_7B, max(args.steps // 4, 20), 2, in_time=True)
        result['c4_in_time_step'] = {
            'workload': 'config 4 with every meta held in its warm-up phase: the activation and gradient casts are in-time '
                        '(amax, scale, cast of the same tensor) as in the first 16 steps of a run',
            'ms_per_step': round(warm['ms_per_step'], 4), 'step_tflops': round(warm['step_tflops'], 1),
            'gemm_tflops': round(warm['gemm_tflops'], 1), 'gemm_frac_mfma': round(warm['gemm_tflops'] / FP8_PEAK_TFLOPS, 4),
        }
        torch.cuda.empty_cache()
        result['gemm_sweep'] = {'c4_llama7b': bench_gemm_sweep(LLAMA_7B, accumulate_row='gate')}
        torch.cuda.empty_cache()
        result['gemm_sweep']['c5_llama70b'] = bench_gemm_sweep(LLAMA_70B, iters=5)
        result['gemm_sweep']['small_layers'] = bench_small_gemms()
        torch.cuda.empty_cache()
        cast = bench_cast()
        torch.cuda.empty_cache()
        adam = bench_adam()
        total_bytes = adam['params'] * 9
        torch.cuda.empty_cache()
        grad_side = bench_grad_side()
        torch.cuda.empty_cache()
        # the top-level cast figure: the config-5 weight (704 MB: nothing of it stays in a cache between calls)
        result['cast_amax_GBps'] = cast['c5_intime_bf16_e4m3_235M']['GBps']
        result['cast_amax_GBps_what'] = 'in-time cast bf16 -> E4M3 of one Llama-70B MLP weight [28672,8192], 3 B/elt, from HBM'

        def adam_row(r):
            row = {'ms': round(r['ms'], 3), 'Gparams_per_s': round(adam['params'] / r['ms'] / 1e6, 1),
                   'GBps': round(total_bytes / r['ms'] / 1e6, 1), 'frac_hbm': round(total_bytes / r['ms'] / 1e6 / HBM_PEAK_GBS, 4),
                   'extra_bytes_per_param': round(r['extra_bytes_per_param'], 3), 'host_ms_per_step': round(r['host_ms_per_step'], 3),
                   'while_scales_move': {'ms': round(r['ms_while_scales_move'], 3),
                                         'frac_hbm': round(total_bytes / r['ms_while_scales_move'] / 1e6 / HBM_PEAK_GBS, 4)}}
            for k in ('tensors_redone_in_last_step', 'slack_chunks'):
                if k in r:
                    row[k] = r[k]
            if 'tensors_redone_while_scales_move' in r:
                row['while_scales_move']['tensors_redone_in_last_step'] = r['tensors_redone_while_scales_move']
            if 'entry_point_ms' in r:
                row['entry_point_alone'] = {'ms': round(r['entry_point_ms'], 3),
                                            'frac_hbm': round(total_bytes / r['entry_point_ms'] / 1e6 / HBM_PEAK_GBS, 4)}
            return row

        best = min(('shift', 'double', 'in_place'), key=lambda k: adam[k]['ms'] if adam[k]['extra_bytes_per_param'] <= 0.5 else 1e9)
        result['fp8_adam_Gparams_per_s'] = adam['params'] / adam[best]['ms'] / 1e6
        result['fp8_adam_what'] = 'LBAdamW.step() through the msamp API, %s form, settled state' % best
        fused = adam_row(adam[best])
        fused.update({
            'params': adam['params'], 'tensors': adam['tensors'],
            'mode': 'LBAdamW.step() through the msamp API (239 ScalingParameters, FP8 gradients), form %r: the fastest one '
                    'that holds at most 0.5 extra bytes per parameter; settled state (no scale moves); 9 B/param algorithmic'
                    % best,
            'through_api': {'in_place (default: every payload keeps its address, two passes)': adam_row(adam['in_place']),
                            "one_pass='shift' (arenas of the optimizer's own, one pass)": adam_row(adam['shift']),
                            "one_pass='double' (second set of payload buffers, one pass)": adam_row(adam['double'])},
        })
        torch.cuda.empty_cache()
        result['power_and_clock'] = bench_power()
        result['kernels'] = {
            'cast': _round_kernels(cast),
            'fused_adamw': fused,
            'adamw_other_parameters': {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in adam[k].items()}
                                       for k in ('float32_moments', 'small_plain_parameters', 'plain_embedding')},
            'grad_side': _round_kernels(grad_side),
        }
    # the tile walks that timing at first use registered in place of the rules' (m, n, k, a K-major, b K-major -> walk)
    from msamp import _backend as _be
    result['gemm_walks_timed_at_first_use'] = {'%dx%dx%d%s%s' % (k[0], k[1], k[2], ' aT' if k[3] else '', ' bT' if k[4] else ''): w
                                               for k, w in sorted(_be.gemm_walks().items())}
    if not args.skip_cpu:
        result['cpu_baseline'] = cpu_baseline()
    print(json.dumps(result))


if __name__ == '__main__':
    main()
