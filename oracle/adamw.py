"""FP8 AdamW step (E4M3/E5M2 weights and grads, E4M3 first moment, scaled-fp16 second moment).

Test infrastructure only.  Follows msamp/optim/adamw.py:148-199 and the kernels at
msamp/optim/adamw.cu:39-50,66-72, evaluated left to right in float32 without fused
multiply-add.
"""

import math

import numpy as np
import torch

from . import fp8
from .scaling import compute_scaling_factor


def _sqrt(x):
    """IEEE correctly rounded float32 square root.  torch's CPU sqrt goes through a vector math
    library that is not correctly rounded on large tensors (about 0.6 % of results are one ulp
    off); numpy's is, and so are CUDA's sqrtf (the reference kernel) and the HIP kernel's."""
    return torch.from_numpy(np.sqrt(x.detach().numpy()))


def host_constants(lr, beta1, beta2, step, bias_correction=True):
    """float32 step_size and sqrt(bias_correction2) as msamp/optim/adamw.cu:104-107 forms them
    (float arguments, double pow, results narrowed to float)."""
    b1 = float(np.float32(beta1))
    b2 = float(np.float32(beta2))
    bc1 = np.float32(1.0 - b1**step) if bias_correction else np.float32(1.0)
    bc2 = np.float32(1.0 - b2**step) if bias_correction else np.float32(1.0)
    step_size = np.float32(np.float32(lr) / bc1)
    sbc2 = np.float32(math.sqrt(float(bc2)))
    return float(step_size), float(sbc2)


def moments(g, m_q, inv_m, v_q, inv_v, beta1, beta2, m_fmt=fp8.E4M3):
    """m' and v' (float32) from the stored quantized moments; adamw.cu:40-42."""
    b1 = torch.tensor(beta1, dtype=torch.float32)
    b2 = torch.tensor(beta2, dtype=torch.float32)
    one = torch.tensor(1.0, dtype=torch.float32)
    mf = fp8.decode(m_q, m_fmt) if m_q.dtype == torch.uint8 else m_q.to(torch.float32)
    vf = v_q.to(torch.float32)
    m_new = b1 * mf * inv_m + (one - b1) * g
    v_new = b2 * vf * inv_v + (one - b2) * (g * g)
    return m_new, v_new


def step_tensor(w_q, w_meta, w_fmt, g_q, g_scale_inv, g_fmt, m_q, m_meta, v_q, v_meta, *, lr, beta1, beta2, eps,
                weight_decay, step, bias_correction=True, adam_mode=False, maximize=False, tensor_scale=True,
                w_fp_max=None):
    """One fused step on one tensor.  Metas are dicts {'scale','scale_inv','amax'} of 0-d/1-d f32 tensors.

    Returns new (w_q, w_meta, m_q, m_meta, v_q, v_meta) and the fp32 intermediates (p, m', v').
    """
    f32 = torch.float32
    step_size, sbc2 = host_constants(lr, beta1, beta2, step, bias_correction)
    step_size = torch.tensor(step_size, dtype=f32)
    sbc2 = torch.tensor(sbc2, dtype=f32)
    epsf = torch.tensor(eps, dtype=f32)

    if w_fmt == 'f16':
        p = w_q.to(f32) * w_meta['scale_inv'].to(f32)
    else:
        p = fp8.decode(w_q, w_fmt) * w_meta['scale_inv'].to(f32)
    g = fp8.decode(g_q, g_fmt) * g_scale_inv.to(f32)
    if maximize:
        g = -g
    if weight_decay != 0:
        if adam_mode:
            g = g + torch.tensor(weight_decay, dtype=f32) * p
        else:
            p = p * torch.tensor(1 - lr * weight_decay, dtype=f32)
    inv_m = (1.0 / m_meta['scale']).to(f32)
    inv_v = (1.0 / v_meta['scale']).to(f32)
    m_new, v_new = moments(g, m_q, inv_m, v_q, inv_v, beta1, beta2)
    denom = _sqrt(v_new) / sbc2 + epsf
    p = p - step_size * (m_new / denom)

    # weight: in-time requantization with fresh amax (adamw.py:173-174)
    w_amax = p.abs().max()
    if w_fmt == 'f16':    # scaled fp16 weight (cast.py:68-95)
        w_scale = compute_scaling_factor(w_amax, w_meta['scale'], 65504.0, 0)
        w_new = (p * w_scale).to(torch.float16)
    else:
        w_scale = compute_scaling_factor(w_amax, w_meta['scale'], fp8.FP_MAX[w_fmt], 0)
        w_new = fp8.encode(p * w_scale, w_fmt)
    w_meta_new = {'scale': w_scale, 'scale_inv': torch.reciprocal(w_scale), 'amax': w_amax.reshape(1)}

    # moments: fresh amax, fallback scale 1.0 (adamw.py:176-184)
    one = torch.ones(())
    m_amax = m_new.abs().max()
    v_amax = v_new.abs().max()
    m_scale = compute_scaling_factor(m_amax, one, fp8.FP_MAX[fp8.E4M3], 0) if tensor_scale else one
    v_scale = compute_scaling_factor(v_amax, one, 65504.0, 0) if tensor_scale else one
    m_store, v_store = m_new, v_new
    if adam_mode and weight_decay != 0:
        # the second stage recomputes the moments from the gradient WITHOUT the L2 term (adamw.py:186-199)
        g_raw = fp8.decode(g_q, g_fmt) * g_scale_inv.to(f32)
        m_store, v_store = moments(-g_raw if maximize else g_raw, m_q, inv_m, v_q, inv_v, beta1, beta2)
    m_out = fp8.encode(m_store * m_scale, fp8.E4M3)
    v_out = (v_store * v_scale).to(torch.float16)
    m_meta_new = {'scale': m_scale, 'scale_inv': torch.reciprocal(m_scale), 'amax': m_amax.reshape(1)}
    v_meta_new = {'scale': v_scale, 'scale_inv': torch.reciprocal(v_scale), 'amax': v_amax.reshape(1)}
    return (w_new, w_meta_new, m_out, m_meta_new, v_out, v_meta_new), (p, m_new, v_new)


def stage1(p, g, m_q, inv_m, v_q, inv_v, *, lr, beta1, beta2, eps, step, bias_correction=True):
    """adamw_fp8_stage1_kernel (adamw.cu:30-59) on fp32 param/grad: returns p', amax_m, amax_v."""
    f32 = torch.float32
    step_size, sbc2 = host_constants(lr, beta1, beta2, step, bias_correction)
    m_new, v_new = moments(g, m_q, torch.tensor(inv_m, dtype=f32), v_q, torch.tensor(inv_v, dtype=f32), beta1, beta2)
    denom = _sqrt(v_new) / torch.tensor(sbc2, dtype=f32) + torch.tensor(eps, dtype=f32)
    p_new = p - torch.tensor(step_size, dtype=f32) * (m_new / denom)
    return p_new, m_new.abs().max(), v_new.abs().max()


def stage2(g, m_q, inv_m, new_m_scale, v_q, inv_v, new_v_scale, *, beta1, beta2):
    """adamw_fp8_stage2_kernel (adamw.cu:61-74): requantized moments."""
    f32 = torch.float32
    m_new, v_new = moments(g, m_q, torch.tensor(inv_m, dtype=f32), v_q, torch.tensor(inv_v, dtype=f32), beta1, beta2)
    m_out = fp8.encode(m_new * torch.tensor(new_m_scale, dtype=f32), fp8.E4M3)
    v_out = (v_new * torch.tensor(new_v_scale, dtype=f32)).to(v_q.dtype)
    return m_out, v_out


def _fma(a, b, c):
    """a * b + c with one rounding to float32: the product of two float32 is exact in float64, the sum is rounded to
    float64 and then to float32 (a second rounding that can differ from a true fused multiply-add only when the float64
    sum lands exactly on a float32 tie: about one element in 2**29)."""
    return (np.float64(a) * np.asarray(b, dtype=np.float64) + np.asarray(c, dtype=np.float64)).astype(np.float32)


def float32_step(p, g, m, v, *, lr, beta1, beta2, eps, weight_decay, step, bias_correction=True, adam_mode=False,
                 maximize=False):
    """The float32-moment branch of LBAdamW.adamw_fn (msamp/optim/adamw.py:200-232) on float32 numpy arrays: returns the
    new (p, m, v).  The reference runs it as a chain of torch calls; on a GPU each `x.add(y, alpha=a)` of the chain
    (lines 209, 223, 226, 232) evaluates x + a * y with one rounding, the division by the Python number
    sqrt(bias_correction2) (line 228) is a multiplication by its reciprocal -- taken in double, narrowed to float32 --
    and every other call rounds once; Python numbers are narrowed to float32 where they meet a tensor."""
    f = np.float32
    p, g, m, v = (np.asarray(t, dtype=np.float32) for t in (p, g, m, v))
    if maximize:
        g = -g
    if weight_decay != 0:
        if adam_mode:
            g = _fma(f(weight_decay), p, g)                                   # :209
        else:
            p = p * f(1 - lr * weight_decay)                                  # :211
    bc1 = 1 - beta1**step if bias_correction else 1.0                         # :213-217
    bc2 = 1 - beta2**step if bias_correction else 1.0
    m_new = _fma(f(1 - beta1), g, m * f(beta1))                               # :223
    v_new = _fma(f(1 - beta2), g * g, v * f(beta2))                           # :226
    denom = np.sqrt(v_new) * f(1.0 / math.sqrt(bc2)) + f(eps)                 # :228
    p_new = _fma(f(-(lr / bc1)), m_new / denom, p)                            # :232
    return p_new, m_new, v_new
