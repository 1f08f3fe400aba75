"""The compute steps of the FP8 gradient reducer, restated on the CPU.  Test infrastructure only.

Follows msamp/nn/distributed.py:143-184 (`_reduce_bucket`, steps 2 to 4) without its two collectives: per gradient
amax (NaN / +Inf -> +Inf), pow-2 scale times 1/sqrt(world size), FP8 codes into a flat buffer, scale_inv = 1/scale,
then the division of the ScalingTensor by the world size (a division of scale_inv, tensor.py:192-207).

Pinned by composition: every piece is a pinned oracle function (amax, scale rule, FP8 encode), and
tests/test_oracle_bucket.py checks what the composition must satisfy: the pre-scale is exact for world sizes
that are powers of four, the dequantized bucket times the world size is the gradient to half a code step, and the
sum of `world` identical buckets stays inside the format (the reason for the pre-scale).
"""

import math

import torch

from . import fp8
from .scaling import compute_scaling_factor


def quantize_bucket(grads, metas, world_size, fmt=fp8.E4M3, reduce_amax=None):
    """grads: list of fp32/fp16/bf16 tensors; metas: list of {'scale','scale_inv','amax'} dicts (updated in place).
    Returns the flat uint8 buffer and the (start, numel) ranges of the gradients in it.
    `reduce_amax` stands for the MAX all-reduce over the ranks (distributed.py:160)."""
    amaxs = torch.stack([g.to(torch.float32).abs().max() if g.numel() else torch.zeros(()) for g in grads]) \
        if grads else torch.zeros(0)
    amaxs.nan_to_num_(nan=float('inf'), posinf=float('inf'))                      # distributed.py:159
    if reduce_amax is not None:
        amaxs = reduce_amax(amaxs)
    scales = torch.stack([m['scale'].reshape(()) for m in metas]) if metas else torch.zeros(0)
    sf = compute_scaling_factor(amaxs, scales, fp8.FP_MAX[fmt], 0)                # distributed.py:166
    sf = sf * torch.tensor(1.0 / math.sqrt(world_size), dtype=torch.float32)      # distributed.py:165,167
    buffer = torch.zeros(sum(g.numel() for g in grads), dtype=torch.uint8)
    ranges, offset = [], 0
    for g, meta, amax, scale in zip(grads, metas, amaxs, sf):
        meta['amax'][0] = amax                                                    # distributed.py:169
        meta['scale'] = scale.clone()                                             # distributed.py:170
        q = fp8.encode(g.to(torch.float32).flatten() * meta['scale'], fmt)        # distributed.py:179-185
        meta['scale_inv'] = torch.reciprocal(meta['scale'])                       # distributed.py:186
        buffer[offset:offset + g.numel()] = q
        meta['scale_inv'] = meta['scale_inv'] / world_size                        # distributed.py:192 (div_)
        ranges.append((offset, g.numel()))
        offset += g.numel()
    return buffer, ranges
