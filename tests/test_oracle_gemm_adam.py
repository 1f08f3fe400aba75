"""Pins the oracle's GEMM definition and AdamW step."""

import json
import os

import numpy as np
import torch

from oracle import adamw, fp8, gemm, cast as ocast, scaling

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'reference_kats.json')))


def _quant(x, fmt):
    meta = ocast.new_meta()
    q = ocast.cast_to_fp8(x, meta, fmt, in_time=True)
    return q, meta


def test_gemm_ones_exact():
    k = GOLDEN['gemm_ones']
    a, am = _quant(torch.ones(k['a_shape']), fp8.E4M3)
    b, bm = _quant(torch.ones(k['b_shape']), fp8.E4M3)
    out = gemm.fp8_gemm(a, am['scale_inv'], fp8.E4M3, b, bm['scale_inv'], fp8.E4M3)
    assert list(out.shape) == k['out_shape'] and torch.all(out == k['value'])


def test_gemm_is_b_times_a_transposed_and_linear():
    g = torch.Generator().manual_seed(0)
    a, am = _quant(torch.randn(5, 16, generator=g), fp8.E4M3)
    b, bm = _quant(torch.randn(7, 16, generator=g), fp8.E5M2)
    out = gemm.fp8_gemm(a, am['scale_inv'], fp8.E4M3, b, bm['scale_inv'], fp8.E5M2)
    af = fp8.decode(a, fp8.E4M3) * am['scale_inv']
    bf = fp8.decode(b, fp8.E5M2) * bm['scale_inv']
    # an asymmetric probe: element [n, m] pairs row n of b with row m of a
    for n, m in [(0, 0), (6, 4), (3, 1)]:
        assert abs(out[n, m].item() - float((bf[n].double() * af[m].double()).sum())) < 1e-5
    acc = gemm.fp8_gemm(a, am['scale_inv'], fp8.E4M3, b, bm['scale_inv'], fp8.E5M2, out=out.clone())
    assert torch.allclose(acc, 2 * out)
    bias = torch.arange(5, dtype=torch.float32)
    wb = gemm.fp8_gemm(a, am['scale_inv'], fp8.E4M3, b, bm['scale_inv'], fp8.E5M2, bias=bias)
    assert torch.allclose(wb - out, bias.expand(7, 5))


def _adam_inputs(n, seed):
    g = torch.Generator().manual_seed(seed)
    w, wm = _quant(0.02 * torch.randn(n, generator=g), fp8.E4M3)
    gq, gm = _quant(1e-3 * torch.randn(n, generator=g), fp8.E5M2)
    m, mm = _quant((1e-4 * torch.randn(n, generator=g)).abs(), fp8.E4M3)
    vm = ocast.new_meta()
    v = ocast.cast_to_fp16((1e-4 * torch.randn(n, generator=g)).abs(), vm, in_time=True)
    return w, wm, gq, gm, m, mm, v, vm


def test_adam_step_matches_textbook_adamw_in_fp32():
    """The fp32 intermediates of one oracle step equal torch.optim.AdamW started from the same
    dequantized state (to float rounding)."""
    n = 4096
    w, wm, gq, gm, m, mm, v, vm = _adam_inputs(n, 11)
    hyper = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    step = 5
    _, (p_new, m_new, v_new) = adamw.step_tensor(w, wm, fp8.E4M3, gq, gm['scale_inv'], fp8.E5M2, m, mm, v, vm, step=step, **hyper)
    p0 = (fp8.decode(w, fp8.E4M3) * wm['scale_inv']).double()
    g0 = (fp8.decode(gq, fp8.E5M2) * gm['scale_inv']).double()
    m0 = (fp8.decode(m, fp8.E4M3) * mm['scale_inv']).double()
    v0 = (v.double() * vm['scale_inv'].double())
    param = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([param], lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    opt.state[param] = {'step': torch.tensor(float(step - 1)), 'exp_avg': m0.clone(), 'exp_avg_sq': v0.clone()}
    param.grad = g0.clone()
    opt.step()
    assert torch.allclose(p_new.double(), param.detach(), rtol=0, atol=2e-8)
    assert torch.allclose(m_new.double(), opt.state[param]['exp_avg'], rtol=1e-6, atol=1e-10)
    assert torch.allclose(v_new.double(), opt.state[param]['exp_avg_sq'], rtol=1e-6, atol=1e-10)


def test_adam_requantization_half_ulp_and_metas():
    n = 8192
    w, wm, gq, gm, m, mm, v, vm = _adam_inputs(n, 5)
    (w2, wm2, m2, mm2, v2, vm2), (p, m_new, v_new) = adamw.step_tensor(
        w, wm, fp8.E4M3, gq, gm['scale_inv'], fp8.E5M2, m, mm, v, vm, lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8,
        weight_decay=0.1, step=1
    )
    for q, meta, real, fp_max in ((w2, wm2, p, 448.0), (m2, mm2, m_new, 448.0)):
        assert meta['amax'][0].item() == real.abs().max().item()
        assert meta['scale'].item() * meta['amax'][0].item() <= fp_max < 2 * meta['scale'].item() * meta['amax'][0].item()
        assert meta['scale_inv'].item() == 1.0 / meta['scale'].item()
        back = fp8.decode(q, fp8.E4M3) * meta['scale_inv']
        expo = torch.floor(torch.log2((real * meta['scale']).abs().clamp_min(2.0**-6)))
        half_ulp = 2.0**(expo - 4) * meta['scale_inv']
        assert torch.all((back - real).abs() <= half_ulp * (1 + 1e-6))
    assert vm2['scale'].item() * vm2['amax'][0].item() <= 65504.0
    backv = v2.float() * vm2['scale_inv']
    assert torch.allclose(backv, v_new, rtol=2.0**-10, atol=0)


def test_stage_functions_consistent_with_fused_step():
    n = 1024
    w, wm, gq, gm, m, mm, v, vm = _adam_inputs(n, 9)
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    (w2, wm2, m2, mm2, v2, vm2), (p, m_new, v_new) = adamw.step_tensor(
        w, wm, fp8.E4M3, gq, gm['scale_inv'], fp8.E5M2, m, mm, v, vm, weight_decay=0.0, step=3, **hyper
    )
    p0 = fp8.decode(w, fp8.E4M3) * wm['scale_inv']
    g0 = fp8.decode(gq, fp8.E5M2) * gm['scale_inv']
    inv_m, inv_v = (1.0 / mm['scale']).item(), (1.0 / vm['scale']).item()
    p1, am, av = adamw.stage1(p0, g0, m, inv_m, v, inv_v, step=3, **hyper)
    assert torch.equal(p1, p) and am.item() == mm2['amax'][0].item() and av.item() == vm2['amax'][0].item()
    ms, vs = adamw.stage2(g0, m, inv_m, mm2['scale'].item(), v, inv_v, vm2['scale'].item(), beta1=0.9, beta2=0.999)
    assert torch.equal(ms, m2) and torch.equal(vs, v2)


def test_host_constants():
    step_size, sbc2 = adamw.host_constants(1e-3, 0.9, 0.999, 1)
    assert abs(step_size - 1e-3 / (1 - 0.9)) < 1e-8 and abs(sbc2 - np.sqrt(1 - 0.999)) < 1e-6
    assert adamw.host_constants(1e-3, 0.9, 0.999, 7, bias_correction=False) == (float(np.float32(1e-3)), 1.0)


def test_scaling_helper_reexport():
    assert scaling.compute_scaling_factor(torch.tensor(10.0), torch.ones(()), 448.0).item() == 32.0


def test_float32_moment_step_matches_textbook_adamw_and_adam():
    """oracle.adamw.float32_step against torch.optim.AdamW / Adam in float64 from the same state (to float32 rounding),
    decoupled decay and L2 mode, with and without maximize; and two closed forms: a zero gradient with zero moments
    leaves the moments at zero and only decays the parameter, and at step 1 from zero moments the update is
    lr * sign(g) for |g| far above eps."""
    import numpy as np
    rng = np.random.default_rng(3)
    n = 5000
    p0 = rng.standard_normal(n).astype(np.float32) * 0.3
    g0 = rng.standard_normal(n).astype(np.float32) * 1e-2
    m0 = rng.standard_normal(n).astype(np.float32) * 1e-2
    v0 = (rng.standard_normal(n).astype(np.float32) * 1e-2) ** 2
    for cls, adam_mode in ((torch.optim.AdamW, False), (torch.optim.Adam, True)):
        for maximize in (False, True):
            step = 7
            got = adamw.float32_step(p0, g0, m0, v0, lr=3e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=step,
                                     adam_mode=adam_mode, maximize=maximize)
            param = torch.nn.Parameter(torch.from_numpy(p0).double())
            opt = cls([param], lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, maximize=maximize)
            opt.state[param] = {'step': torch.tensor(float(step - 1)), 'exp_avg': torch.from_numpy(m0).double(),
                                'exp_avg_sq': torch.from_numpy(v0).double()}
            param.grad = torch.from_numpy(g0).double()
            opt.step()
            want = (param.detach(), opt.state[param]['exp_avg'], opt.state[param]['exp_avg_sq'])
            for a, b, atol in zip(got, want, (3e-7, 1e-8, 1e-10)):
                assert a.dtype == np.float32
                assert torch.allclose(torch.from_numpy(a).double(), b, rtol=2e-6, atol=atol)
    zero = np.zeros(n, np.float32)
    p1, m1, v1 = adamw.float32_step(p0, zero, zero, zero, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.5, step=3)
    assert not m1.any() and not v1.any() and np.array_equal(p1, p0 * np.float32(1 - 1e-2 * 0.5))
    p1, m1, v1 = adamw.float32_step(p0, g0 + np.sign(g0), zero, zero, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
                                    step=1)
    assert np.allclose(p0 - p1, 1e-2 * np.sign(g0), rtol=1e-5, atol=0)
