"""What the gradient-bucket oracle must satisfy whatever its formula says (CPU)."""

import math

import torch

from oracle import bucket, cast as ocast, fp8
from oracle.scaling import compute_scaling_factor


def _grads(seed, sizes, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, generator=g) * 10.0 ** float(torch.randint(-4, 2, (1, ), generator=g))).to(dtype) for n in sizes]


def test_world_one_is_the_in_time_cast():
    """With one rank the bucket holds exactly what an in-time cast of each gradient gives (sync semantics)."""
    grads = _grads(0, [5, 1000, 16384 + 3])
    metas = [ocast.new_meta() for _ in grads]
    buf, ranges = bucket.quantize_bucket(grads, metas, 1)
    for g, meta, (start, n) in zip(grads, metas, ranges):
        ref = ocast.new_meta()
        q = ocast.cast_to_fp8(g, ref, fp8.E4M3, in_time=True, sync=True)
        assert torch.equal(buf[start:start + n], q)
        assert torch.equal(meta['scale'], ref['scale']) and torch.equal(meta['scale_inv'], ref['scale_inv'])
        assert meta['amax'][0] == ref['amax'][0]


def test_pre_scale_and_division_by_the_world_size():
    """world = 4: the pre-scale is exactly 1/2, so scale = rule/2 and scale_inv = 2/rule/4; dequantizing a code and
    multiplying by the world size gives the gradient back to within half a code step; the sum of `world` copies of
    any code stays within the format (|q| <= 448/2 * ... the reason for the pre-scale)."""
    grads = _grads(1, [4096, 77])
    metas = [ocast.new_meta() for _ in grads]
    world = 4
    buf, ranges = bucket.quantize_bucket(grads, metas, world)
    for g, meta, (start, n) in zip(grads, metas, ranges):
        rule = compute_scaling_factor(g.abs().max(), torch.ones(()), 448.0, 0)
        assert meta['scale'].item() == rule.item() / 2
        assert meta['scale_inv'].item() == (1.0 / meta['scale'].item()) / world
        vals = fp8.decode(buf[start:start + n], fp8.E4M3)
        assert vals.abs().max().item() <= 448.0 / 2
        back = vals * meta['scale_inv'] * world
        step = (2.0 ** torch.floor(torch.log2(vals.abs().clamp_min(2.0 ** -6)))) / 8 / meta['scale']
        assert ((back - g).abs() <= step / 2 * (1 + 1e-6)).all()


def test_non_finite_gradient_and_reduced_amax():
    """NaN or Inf in a gradient makes its amax +Inf, and then the rule's quirk applies (1 / fallback scale);
    a larger amax from another rank (the reduce hook) lowers the scale."""
    grads = [torch.tensor([1.0, float('nan'), 2.0]), torch.tensor([3.0, 4.0])]
    metas = [ocast.new_meta(), ocast.new_meta()]
    metas[0]['scale'] = torch.tensor(4.0)
    bucket.quantize_bucket(grads, metas, 1, reduce_amax=lambda a: torch.maximum(a, torch.tensor([0.0, 400.0])))
    assert math.isinf(metas[0]['amax'][0].item()) and metas[0]['scale'].item() == 0.25
    assert metas[1]['amax'][0].item() == 400.0 and metas[1]['scale'].item() == 1.0


def test_empty_bucket_and_empty_gradient():
    buf, ranges = bucket.quantize_bucket([], [], 2)
    assert buf.numel() == 0 and ranges == []
    meta = ocast.new_meta()
    buf, ranges = bucket.quantize_bucket([torch.zeros(0)], [meta], 2)
    assert buf.numel() == 0 and ranges == [(0, 0)] and meta['amax'][0].item() == 0.0
