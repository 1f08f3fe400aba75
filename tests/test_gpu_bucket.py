"""GPU parity of the gradient-bucket quantization (reducer steps 2 to 4) against the CPU oracle: FP8 codes, scale,
scale_inv and amax bit-exact."""

import math

import pytest
import torch

from oracle import bucket as obucket, cast as ocast, fp8
from tests.gpu_util import same_float

pytestmark = pytest.mark.gpu


def _grads(seed, sizes, dtype):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, generator=g) * 10.0 ** float(torch.randint(-4, 2, (1, ), generator=g))).to(dtype) for n in sizes]


def _check(bucket, out, grads, world, scales=None, reduce=None):
    metas = [ocast.new_meta() for _ in grads]
    for m, s in zip(metas, scales or []):
        m['scale'] = torch.tensor(s)
    buf, ranges = obucket.quantize_bucket(grads, metas, world, reduce_amax=reduce)
    assert torch.equal(bucket.flat.cpu(), buf)
    for t, g, meta, (start, n) in zip(out, grads, metas, ranges):
        assert t.numel() == n and t.value.data_ptr() == bucket.flat.data_ptr() + start
        assert same_float(t.meta.scale, meta['scale']) and same_float(t.meta.scale_inv, meta['scale_inv'])
        assert same_float(t.meta.amax[0], meta['amax'][0])


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('world', [1, 2, 3, 8])
def test_bucket_matches_oracle(dtype, world):
    """Ragged sizes: tensors of a few elements, sizes that leave the next tensor misaligned in the flat buffer,
    whole and partial chunks, and a 2-D gradient."""
    from msamp.nn import GradientBucket
    sizes = [5, 16384, 3, 16384 * 2 + 777, 1, 4096 * 33, 100]
    grads = _grads(world, sizes, dtype)
    grads[5] = grads[5].view(4096, 33)
    bucket = GradientBucket(sizes)
    out = bucket.quantize([g.cuda() for g in grads], world_size=world)
    _check(bucket, out, [g.flatten() for g in grads], world)
    for t, g in zip(out, grads):
        assert t.shape == g.shape


def test_bucket_non_finite_and_reduced_amax():
    """A NaN and an Inf gradient (amax -> +Inf, the rule's quirk gives 1 / fallback scale), a zero gradient (the
    fallback scale stays), and an amax raised by the reduce hook."""
    from msamp.nn import GradientBucket
    grads = [torch.tensor([1.0, float('nan'), 2.0]), torch.tensor([float('-inf'), 4.0]), torch.zeros(40000),
             torch.tensor([3.0, -4.0])]
    bucket = GradientBucket([g.numel() for g in grads])
    scales = [4.0, 2.0, 8.0, 1.0]
    for m, s in zip(bucket.metas, scales):
        m.scale.fill_(s)

    def reduce_gpu(cells):
        cells[3].fill_(400.0)

    def reduce_cpu(a):
        a = a.clone()
        a[3] = 400.0
        return a

    out = bucket.quantize([g.cuda() for g in grads], world_size=2, reduce_amax=reduce_gpu)
    _check(bucket, out, grads, 2, scales=scales, reduce=reduce_cpu)
    assert math.isinf(out[0].meta.amax[0].item()) and math.isinf(out[1].meta.amax[0].item())


def test_bucket_reuse_and_argument_checks():
    from msamp.nn import GradientBucket
    bucket = GradientBucket([1000, 20000])
    for seed in (1, 2):    # second call: new gradient tensors, same bucket (tables are rebuilt, scratch is clean)
        grads = _grads(seed, [1000, 20000], torch.float32)
        out = bucket.quantize([g.cuda() for g in grads], world_size=4)
        metas = [ocast.new_meta() for _ in grads]
        if seed == 2:
            for m, prev in zip(metas, scales_before):
                m['scale'] = prev
        buf, _ = obucket.quantize_bucket(grads, metas, 4)
        assert torch.equal(bucket.flat.cpu(), buf)
        scales_before = [t.meta.scale.cpu().clone() for t in out]
    with pytest.raises(ValueError):
        bucket.quantize([torch.zeros(3, device='cuda')])
    with pytest.raises(ValueError):
        bucket.quantize([torch.zeros(1000, device='cuda'), torch.zeros(20000, device='cuda', dtype=torch.bfloat16)])
    assert GradientBucket([]).quantize([]) == []


def test_bucket_sum_of_ranks_is_the_average():
    """What the pre-scale and the division are for: with `world` ranks holding the same gradient, adding the ranks'
    dequantized buckets (what the SUM all-reduce of the payloads amounts to) gives the gradient back to FP8
    accuracy, and the payload sum stays inside the format."""
    from msamp.nn import GradientBucket
    world = 4
    g = _grads(9, [50000], torch.float32)[0]
    bucket = GradientBucket([g.numel()])
    t = bucket.quantize([g.cuda()], world_size=world)[0]
    codes = fp8.decode(t.value.cpu(), fp8.E4M3)
    assert (codes * world).abs().max().item() <= 448.0 * math.sqrt(world)
    avg = t.float().cpu() * world
    assert ((avg - g).abs() <= g.abs() * 2.0 ** -4 + g.abs().max() * 2.0 ** -9).all()
