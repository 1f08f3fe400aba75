"""Benchmark of the FP8 hot path on one MI355X.

A step is one forward + backward of a single FP8Linear at x[8192,4096] (bf16), W[4096,4096] (bf16
payload), dy[8192,4096] (bf16) in steady-state delayed scaling (amax history 16): input cast to E4M3,
weight cast, y = x W^T, cast of dy to E5M2, dx = dy W and dW = dy^T x (the kernel reads W, x and dy
K-major in place, so no transposed copies are made), the in-time E4M3 cast of dW and the amax-window
update.  `value` is the three GEMMs'
2*M*N*K flops divided by the whole step time (inputs resident in HBM).  Beside it: the GEMM kernel's
own roofline (HIP events around the GEMM launches of every fourth step inside the timed region), the cast+amax and fused
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
GEMM_EVENT_STRIDE = 4
FP8_PEAK_TFLOPS = 5000.0


def _events():
    import torch
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def bench_fp8linear(steps, warmup):
    import torch
    import msamp    # noqa: F401
    from msamp import _backend
    from msamp.common.dtype import Dtypes
    from msamp.nn import LinearReplacer, model_state
    from msamp.optim import LBAdamW
    import msamp.operators.gemm.gemm as gemm_mod

    tokens, d_in, d_out = 8192, 4096, 4096
    g = torch.Generator(device='cuda').manual_seed(0)
    x = torch.randn(tokens, d_in, device='cuda', generator=g).bfloat16().requires_grad_(True)
    dy = (torch.randn(tokens, d_out, device='cuda', generator=g) * 1e-3).bfloat16()
    lin = torch.nn.Linear(d_in, d_out, bias=False).cuda()
    with torch.no_grad():
        lin.weight.copy_(torch.randn(d_out, d_in, device='cuda', generator=g) * 0.02)
    model_state.clear()
    model = LinearReplacer.replace(lin.bfloat16(), Dtypes.kbfloat16)
    opt = LBAdamW(model.parameters())    # only its scaling-factor update runs here

    gemm_events = []
    real_gemm = _backend.fp8_gemm
    real_gemm_cast = _backend.fp8_gemm_cast

    class _Timed:
        enabled = False

        @staticmethod
        def fp8_gemm(*args, **kwargs):
            if not _Timed.enabled:
                return real_gemm(*args, **kwargs)
            s, e = _events()
            s.record()
            out = real_gemm(*args, **kwargs)
            e.record()
            gemm_events.append((s, e))
            return out

        @staticmethod
        def fp8_gemm_cast(*args, **kwargs):
            # the weight-gradient GEMM with its cast to E4M3 fused in: one launch, timed as the GEMM it is
            if not _Timed.enabled:
                return real_gemm_cast(*args, **kwargs)
            s, e = _events()
            s.record()
            out = real_gemm_cast(*args, **kwargs)
            e.record()
            if out is not None:
                gemm_events.append((s, e))
            return out

        def __getattr__(self, name):
            return getattr(_backend, name)

    gemm_mod._backend = _Timed()

    def step():
        y = model(x)
        y.backward(dy)
        opt._update_scaling_factors()
        model.weight.grad = None
        x.grad = None

    for _ in range(max(warmup, 17)):    # >= 17 steps: past the 16-step warm-up, casts are single-pass
        step()
    assert not model.scaling_metas['input'].is_in_time_scaling()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        # an event pair costs the stream a few microseconds: bracket the GEMMs of every fourth step only
        _Timed.enabled = i % GEMM_EVENT_STRIDE == 0
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    _Timed.enabled = False
    gemm_mod._backend = _backend

    flops_per_gemm = 2.0 * tokens * d_in * d_out
    ms_per_step = dt / steps * 1e3
    gemm_ms = sum(s.elapsed_time(e) for s, e in gemm_events) / len(gemm_events)
    return {
        'ms_per_step': ms_per_step,
        'step_tflops': 3 * flops_per_gemm / (ms_per_step * 1e-3) / 1e12,
        'gemm_ms': gemm_ms,
        'gemm_tflops': flops_per_gemm / (gemm_ms * 1e-3) / 1e12,
        'gemm_launches': len(gemm_events),
    }


def _time_gpu(fn, iters, warm=3):
    """Average duration of one call, from HIP events around a batch of `iters` back-to-back calls on the
    current stream (what a kernel sustains once the launch queue is primed)."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    s, e = _events()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) / iters


def bench_cast(iters=20):
    """cast+amax throughput: C1 (fp32 [4096,4096], in-time, E4M3), steady-state delayed cast of bf16
    [8192,4096], and the in-time cast of one Llama-70B MLP weight (bf16 [28672,8192])."""
    import torch
    from msamp import _backend
    from tests.gpu_util import c1_input, make_meta
    out = {}
    x = c1_input(0).cuda()
    s, si, am = make_meta()
    ms = _time_gpu(lambda: _backend.cast_to_fp8_intime(x, s, am[0:1], si, _backend.DT_E4M3), iters)
    out['c1_intime_fp32_e4m3'] = {'ms': ms, 'GBps': x.numel() * 5 / ms / 1e6}
    ms = _time_gpu(lambda: _backend.cast_to_fp8_intime(x, s, am[0:1], si, _backend.DT_E5M2), iters)
    out['c1_intime_fp32_e5m2'] = {'ms': ms, 'GBps': x.numel() * 5 / ms / 1e6}
    q = _backend.cast_to_fp8_intime(x, s, am[0:1], si, _backend.DT_E4M3)
    ms = _time_gpu(lambda: _backend.cast_from_fp8(q, si, _backend.DT_E4M3, torch.float32), iters)
    out['c1_dequant_e4m3_fp32'] = {'ms': ms, 'GBps': x.numel() * 5 / ms / 1e6}
    # the same cast with nothing in the caches: eight distinct 64 MiB inputs in turn (512 MiB, twice the 256 MiB
    # memory-side cache), which is how a training step meets its activations
    xs = [x] + [torch.randn_like(x) for _ in range(7)]
    turn = {'i': 0}

    def cold_cast():
        turn['i'] = (turn['i'] + 1) % len(xs)
        _backend.cast_to_fp8_intime(xs[turn['i']], s, am[0:1], si, _backend.DT_E4M3)

    ms = _time_gpu(cold_cast, 2 * len(xs), warm=len(xs))
    out['c1_intime_fp32_e4m3_cold'] = {'ms': ms, 'GBps': x.numel() * 5 / ms / 1e6}
    del x, q, xs
    a = torch.randn(8192, 4096, device='cuda').bfloat16()
    ms = _time_gpu(lambda: _backend.cast_to_fp8(a, s, am[0:1], si, _backend.DT_E4M3), iters)
    out['c2_delayed_bf16_e4m3'] = {'ms': ms, 'GBps': a.numel() * 3 / ms / 1e6}
    ms = _time_gpu(lambda: _backend.cast_transpose(a, s, am[0:1], si, _backend.DT_E5M2), iters)
    out['c2_cast_transpose_bf16_e5m2'] = {'ms': ms, 'GBps': a.numel() * 4 / ms / 1e6}
    qa = _backend.cast_to_fp8(a, s, am[0:1], si, _backend.DT_E4M3)
    ms = _time_gpu(lambda: _backend.fp8_transpose(qa), iters)
    out['c2_fp8_transpose'] = {'ms': ms, 'GBps': a.numel() * 2 / ms / 1e6}
    del a, qa
    w = (torch.randn(28672, 8192, device='cuda') * 0.01).bfloat16()
    ms = _time_gpu(lambda: _backend.cast_to_fp8_intime(w, s, am[0:1], si, _backend.DT_E4M3), max(iters // 2, 5))
    out['c5_intime_bf16_e4m3_235M'] = {'ms': ms, 'GBps': w.numel() * 3 / ms / 1e6}
    del w
    # what a plain copy reaches on this box (the practical ceiling of the streaming kernels above): 256 MiB of
    # fp32 through the library's scale_cast at scale 1, read once, written once
    src = torch.ones(64 * 1024 * 1024, device='cuda')
    one = torch.ones((), device='cuda')
    ms = _time_gpu(lambda: _backend.scale_cast(src, one, torch.float32), max(iters // 2, 5))
    out['copy_fp32_256MiB'] = {'ms': ms, 'GBps': src.numel() * 8 / ms / 1e6}
    return out


def bench_grad_side(iters=10):
    """The reducer's compute steps on one bucket of 32 bf16 gradients of [4096,1024] (amax, scales, quantize
    into the flat E4M3 buffer: 2 B read twice + 1 B written per element), and the per-tensor 2-norms of 64
    such FP8 gradients (1 B read per element)."""
    import torch
    from msamp import _backend
    from msamp.nn import GradientBucket
    n = 4096 * 1024
    grads = [(torch.randn(n, device='cuda') * 1e-3).bfloat16() for _ in range(32)]
    bucket = GradientBucket([n] * len(grads))
    out = {}
    ms = _time_gpu(lambda: bucket.quantize(grads, world_size=8), iters)
    out['bucket_quantize_32x4M_bf16'] = {'ms': ms, 'GBps': n * len(grads) * 5 / ms / 1e6}
    del grads, bucket
    qs = [torch.randint(0, 120, (n,), dtype=torch.uint8, device='cuda') for _ in range(64)]
    sis = [torch.ones((), device='cuda') for _ in qs]
    ms = _time_gpu(lambda: _backend.fp8_norms(qs, sis, _backend.DT_E4M3, 2.0), iters)
    out['fp8_l2_norms_64x4M_e4m3'] = {'ms': ms, 'GBps': n * len(qs) / ms / 1e6}
    return out


def bench_adam(iters=5, total_params=1_000_000_000):
    """Fused FP8 AdamW over 1.0e9 parameters held as [4096,1024] tensors (last one truncated):
    E4M3 weights, E5M2 grads, E4M3 exp_avg, scaled-fp16 exp_avg_sq; step t=2."""
    import numpy as np
    import torch
    from msamp import _backend
    per = 4096 * 1024
    sizes = [per] * (total_params // per)
    if total_params % per:
        sizes.append(total_params % per)
    tensors, rows = [], []
    for n in sizes:
        w = (torch.randn(n, device='cuda') * 0.02)
        g = (torch.randn(n, device='cuda') * 1e-3)
        d = {}
        for name, src, dt in (('w', w, _backend.DT_E4M3), ('g', g, _backend.DT_E5M2)):
            s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
            d[name] = (_backend.cast_to_fp8_intime(src, s, am, si, dt), s, si, am)
        m = (torch.randn(n, device='cuda') * 1e-4).abs_()
        s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
        d['m'] = (_backend.cast_to_fp8_intime(m, s, am, si, _backend.DT_E4M3), s, si, am)
        v = (torch.randn(n, device='cuda') * 1e-4).abs_()
        s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
        _backend.amax(v, am)
        s.copy_(_backend.compute_scaling_factor(am, s.reshape(1), 65504.0, 0)[0])
        si.copy_(1.0 / s)
        d['v'] = (_backend.scale_cast(v, s, torch.float16), s, si, am)
        del w, g, m, v
        tensors.append(d)
        rows.append((d['w'][0].data_ptr(), d['g'][0].data_ptr(), d['m'][0].data_ptr(), d['v'][0].data_ptr(),
                     d['w'][1].data_ptr(), d['w'][2].data_ptr(), d['w'][3].data_ptr(), d['g'][2].data_ptr(),
                     d['m'][1].data_ptr(), d['m'][2].data_ptr(), d['m'][3].data_ptr(),
                     d['v'][1].data_ptr(), d['v'][2].data_ptr(), d['v'][3].data_ptr(), n, 0, 0, 0, 0))
    desc = torch.from_numpy(np.asarray(rows, dtype=np.int64)).cuda()
    chunks = [(n + _backend.ADAMW_CHUNK - 1) // _backend.ADAMW_CHUNK for n in sizes]
    bm = np.stack([np.repeat(np.arange(len(sizes), dtype=np.int32), chunks),
                   np.concatenate([np.arange(c, dtype=np.int32) for c in chunks])], axis=1).copy()
    block_map = torch.from_numpy(bm).cuda()
    state = {'t': 1}

    def step():
        state['t'] += 1
        _backend.adamw_fused(desc, len(sizes), block_map, block_map.shape[0], _backend.DT_E4M3, _backend.DT_E5M2, 3e-4, 0.9,
                             0.95, 1e-8, 0.1, state['t'], True, False, False, True, blocks_per_tensor=chunks)

    ms = _time_gpu(step, iters, warm=2)
    return {'ms': ms, 'Gparams_per_s': total_params / ms / 1e6, 'GBps_algorithmic': total_params * 9 / ms / 1e6,
            'tensors': len(sizes), 'params': total_params}


def cpu_baseline():
    """The oracle (PyTorch CPU restatement of the reference math) on a bounded sample, all host cores."""
    import torch
    from oracle import adamw as oadam, cast as ocast, fp8
    from tests.gpu_util import c1_input
    from tests.test_gpu_adam import _inputs
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
    n = 4096 * 1024
    tens = [_inputs(n, i, fp8.E4M3, fp8.E5M2) for i in range(2)]

    def adam():
        for d in tens:
            oadam.step_tensor(d['w'], d['wm'], fp8.E4M3, d['g'], d['gm']['scale_inv'], fp8.E5M2, d['m'], d['mm'], d['v'], d['vm'],
                              lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=2)

    ta = med(adam, runs=3, warm=1)
    adam_gps = len(tens) * n / ta / 1e9
    # GEMM definition (fp32 matmul of dequantized operands) on 1024 of the 8192 token rows
    a = fp8.decode(fp8.encode(torch.randn(4096, 4096) * 0.02 * 64, fp8.E4M3), fp8.E4M3)
    b = fp8.decode(fp8.encode(torch.randn(1024, 4096), fp8.E4M3), fp8.E4M3)
    tg = med(lambda: b @ a.t(), runs=5, warm=1)
    gemm_tflops = 2.0 * 1024 * 4096 * 4096 / tg / 1e12
    return {
        'value': gemm_tflops, 'unit': 'TFLOP/s', 'cores': cores, 'threads': torch.get_num_threads(), 'kind': 'port',
        'sample': 'fp32 matmul of dequantized operands, 1024 of 8192 token rows of the forward GEMM; '
                  'cast: full config-1 tensor fp32[4096,4096] in-time E4M3; adam: 2 of 239 tensors [4096,1024]',
        'cast_amax': {'value': cast_gbps, 'unit': 'GB/s (5 B/elt)'},
        'fp8_adam': {'value': adam_gps, 'unit': 'Gparams/s'},
    }


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
    """HBM bytes per GEMM launch as last measured with rocprofv3 --pmc (profiles/fp8_gemm_hbm_traffic.json),
    or None when no measurement is on file."""
    path = os.path.join(ROOT, 'profiles', 'fp8_gemm_hbm_traffic.json')
    try:
        with open(path) as f:
            return json.load(f)['traffic_bytes_per_launch']
    except (OSError, KeyError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--skip-cpu', action='store_true', help='leave out the CPU-oracle baseline')
    ap.add_argument('--skip-extra', action='store_true', help='leave out the cast and Adam kernel sections')
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
    lin = bench_fp8linear(args.steps, args.warmup)
    result = {
        'metric': 'FP8 GEMM TFLOPS, cast+amax GB/s, FP8-Adam Gparams/s on 1 MI355X',
        'value': lin['step_tflops'],
        'unit': 'TFLOP/s (3 GEMMs of one FP8Linear fwd+bwd / whole step incl. casts and window update)',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': max(args.warmup, 17),
        'ms_per_step': lin['ms_per_step'],
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'fp8 (e4m3 x e4m3 / e4m3 x e5m2), fp32 accumulate',
        'data': 'synthetic',
        'config': {'workload': 'single FP8Linear fwd+bwd, x bf16[8192,4096], W bf16[4096,4096], dy bf16[8192,4096], '
                               'delayed scaling (history 16), outputs bf16, dW -> E4M3'},
        'roofline': {
            'kernel': 'fp8_gemm_dma_kernel', 'bound': 'mfma', 'achieved': lin['gemm_tflops'], 'peak': FP8_PEAK_TFLOPS,
            'unit': 'TFLOP/s', 'frac': lin['gemm_tflops'] / FP8_PEAK_TFLOPS, 'traffic': measured_gemm_traffic(),
            'avg_launch_ms': lin['gemm_ms'], 'launches': lin['gemm_launches'],
        },
    }
    if not args.skip_extra:
        cast = bench_cast()
        adam = bench_adam()
        torch.cuda.empty_cache()
        grad_side = bench_grad_side()
        torch.cuda.empty_cache()
        result['cast_amax_GBps'] = cast['c1_intime_fp32_e4m3']['GBps']
        result['fp8_adam_Gparams_per_s'] = adam['Gparams_per_s']
        result['kernels'] = {
            'cast': {k: {'ms': round(v['ms'], 4), 'GBps': round(v['GBps'], 1), 'frac_hbm': round(v['GBps'] / HBM_PEAK_GBS, 4)}
                     for k, v in cast.items()},
            'fused_adamw': {'ms': round(adam['ms'], 3), 'Gparams_per_s': round(adam['Gparams_per_s'], 1),
                            'GBps': round(adam['GBps_algorithmic'], 1),
                            'frac_hbm': round(adam['GBps_algorithmic'] / HBM_PEAK_GBS, 4), 'params': adam['params'],
                            'tensors': adam['tensors']},
            'grad_side': {k: {'ms': round(v['ms'], 4), 'GBps': round(v['GBps'], 1),
                              'frac_hbm': round(v['GBps'] / HBM_PEAK_GBS, 4)} for k, v in grad_side.items()},
        }
    if not args.skip_cpu:
        result['cpu_baseline'] = cpu_baseline()
    print(json.dumps(result))


if __name__ == '__main__':
    main()
