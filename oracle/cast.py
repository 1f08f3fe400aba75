"""Cast / dequantize / transpose semantics.  Test infrastructure only.

``meta`` here is a plain dict {'scale': 0-d f32, 'scale_inv': 0-d f32, 'amax': (window,) f32}.
"""

import torch

from . import fp8
from .scaling import compute_scaling_factor


def new_meta(window=1):
    return {'scale': torch.ones(()), 'scale_inv': torch.ones(()), 'amax': torch.zeros(window)}


def _atomic_max_float(old, val):
    """CUDA atomicMaxFloat for val >= 0: integer compare of the bit patterns; a (positive) NaN
    already in the cell compares above every finite value and stays."""
    if torch.isnan(old):
        return old.clone().reshape(())
    o = old.reshape(1).view(torch.int32)
    v = val.reshape(1).to(torch.float32).view(torch.int32)
    return torch.maximum(o, v).view(torch.float32).reshape(())


def amax_nan_skipping(x):
    """max|x| the way a fmaxf chain starting at 0 computes it: NaN elements are ignored."""
    a = x.to(torch.float32).abs().flatten()
    a = torch.where(torch.isnan(a), torch.zeros_like(a), a)
    return a.max() if a.numel() else torch.zeros(())


def cast_to_fp8(x, meta, fmt, in_time, sync=False):
    """msamp/common/tensor/cast.py:17-65 (non-transposing branch) on the CPU.

    in_time: amax[0] = max|x| (NaN propagates), scale recomputed from it.
    delayed: quantize with the stored scale; amax[0] = atomicMax(amax[0], NaN-skipping max|x|).
    Always: scale_inv = 1/scale.
    """
    xf = x.to(torch.float32)
    if in_time:
        meta['amax'][0] = xf.abs().max() if xf.numel() else torch.zeros(())
    if sync:
        meta['amax'][0:1].nan_to_num_(nan=float('inf'), posinf=float('inf'))
    if in_time or sync:
        meta['scale'] = compute_scaling_factor(meta['amax'][0], meta['scale'], fp8.FP_MAX[fmt], 0)
    q = fp8.encode(xf * meta['scale'], fmt)
    meta['amax'][0] = _atomic_max_float(meta['amax'][0], amax_nan_skipping(xf))
    meta['scale_inv'] = torch.reciprocal(meta['scale'])
    return q


def cast_from_fp8(q, scale_inv, fmt, out_dtype=torch.float32):
    """msamp/common/tensor/cast.py:98-119: otype(float(q) * scale_inv)."""
    return (fp8.decode(q, fmt) * scale_inv.to(torch.float32)).to(out_dtype)


def cast_to_fp16(x, meta, in_time, out_dtype=torch.float16, fp_max=65504.0):
    """msamp/common/tensor/cast.py:68-95: scaled fp16 tensor, (x*scale).to(fp16)."""
    if in_time:
        meta['amax'][0] = x.abs().max().to(torch.float32)
        meta['scale'] = compute_scaling_factor(meta['amax'][0], meta['scale'], fp_max, 0)
    meta['scale_inv'] = torch.reciprocal(meta['scale'])
    return (x * meta['scale'].view(1)).to(out_dtype)


def cast_transpose(x2d, meta, fmt, in_time, sync=False):
    """Fused cast + transpose (msamp/common/tensor/cast.py:47-52): same bytes, two layouts."""
    q = cast_to_fp8(x2d, meta, fmt, in_time, sync)
    return q, q.t().contiguous()


def scaled_fp16_to_fp8(value, old_meta, fmt):
    """ScalingTensor.cast from a scaled fp16/bf16/fp32 payload to FP8
    (msamp/common/tensor/tensor.py:241-265): reuse the stored amax, no new reduction."""
    new_scale = compute_scaling_factor(old_meta['amax'][0], torch.ones(()), fp8.FP_MAX[fmt], 0)
    scale_inv = torch.reciprocal(new_scale)
    qscale = new_scale * old_meta['scale_inv']
    q = fp8.encode(value.to(torch.float32) * qscale, fmt)
    meta = {'scale': qscale, 'scale_inv': scale_inv, 'amax': old_meta['amax'].clone()}
    return q, meta
