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


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_bucket_speculative_rounds_equal_plain_rounds(dtype):
    """Five reductions on one bucket, each taken with and without speculation from the same state: same buffer and
    metas every time.  The first finds scale 1 in the metas (every guess wrong); the second has gradients of the same
    size, so the amax pass alone already leaves the final bytes; in the third half of the gradients are 64 times larger
    (those are done again); the fourth has a NaN in one gradient; the fifth is back to normal."""
    from msamp import _backend
    from msamp.nn import GradientBucket
    sizes = [5, 16384, 3, 16384 * 2 + 777, 1, 4096 * 33, 100, 16384 * 4]
    world = 2
    plain, spec = GradientBucket(sizes, speculate=False), GradientBucket(sizes, speculate=True)
    base = _grads(77, sizes, dtype)
    for rnd in range(1, 6):
        noise = torch.Generator().manual_seed(100 + rnd)
        grads = [(g.float() * (1 + 0.01 * torch.randn(g.shape, generator=noise))).to(dtype) for g in base]
        if rnd == 3:
            grads = [g * 64 if i % 2 == 0 else g for i, g in enumerate(grads)]
        if rnd == 4:
            grads[3][12345] = float('nan')
        dev = [g.cuda() for g in grads]
        before = [m.scale.clone() for m in spec.metas]
        # what the speculative first pass alone leaves in the buffer
        items, block_map = spec._get_tables(dev)
        _backend.bucket_amax(items, block_map, _backend._dt(dev[0]), nan_to_inf=True, speculate_fp8_dt=int(spec.qtype))
        early = spec.flat.clone()
        _backend.bucket_cast(items, block_map, _backend._dt(dev[0]), int(spec.qtype), 1.0 / math.sqrt(world), float(world))
        out_p = plain.quantize(dev, world_size=world)
        assert torch.equal(spec.flat, plain.flat), rnd
        if rnd == 2:
            # a second cast of the same round (no new amax pass) may not rely on what the first one found in the buffer:
            # with the scales settled it must write the same bytes again
            spec.flat.zero_()
            _backend.bucket_cast(items, block_map, _backend._dt(dev[0]), int(spec.qtype), 1.0, 1.0)
            torch.cuda.synchronize()
            for view_offset, n, k in zip(_offsets(sizes), sizes, [same_float(m.scale, s) for m, s in zip(spec.metas, before)]):
                assert bool(spec.flat[view_offset:view_offset + n].any()), 'second cast skipped a tensor'
            # (its scale no longer carries the 1/sqrt(world) factor: bring buffer and metas back for the comparisons below)
            _backend.bucket_amax(items, block_map, _backend._dt(dev[0]), nan_to_inf=True)
            for m, sb in zip(spec.metas, before):
                m.scale.copy_(sb)
            _backend.bucket_cast(items, block_map, _backend._dt(dev[0]), int(spec.qtype), 1.0 / math.sqrt(world), float(world))
            assert torch.equal(spec.flat, plain.flat)
        for a, b in zip(spec.metas, plain.metas):
            assert same_float(a.scale, b.scale) and same_float(a.scale_inv, b.scale_inv) and same_float(a.amax[0], b.amax[0])
        kept = [same_float(m.scale, s) for m, s in zip(spec.metas, before)]
        for view_offset, n, k in zip(_offsets(sizes), sizes, kept):
            same_early = torch.equal(early[view_offset:view_offset + n], spec.flat[view_offset:view_offset + n])
            assert same_early or not k, rnd    # a kept scale means the first pass already wrote the final bytes
        if rnd == 1:
            assert not any(kept)
        if rnd in (2, 5):
            assert sum(kept) >= len(sizes) - 2 and torch.equal(early, spec.flat) == all(kept)
        if rnd == 3:
            assert not any(kept[0::2])
        _check(plain, out_p, [g.flatten() for g in grads], world, scales=[float(s) for s in before])
    # and through the class, speculation on by default
    a, b = GradientBucket(sizes), GradientBucket(sizes, speculate=False)
    for seed in (1, 1, 2):
        dev = [g.cuda() for g in _grads(seed, sizes, dtype)]
        a.quantize(dev, world_size=4)
        b.quantize(dev, world_size=4)
        assert torch.equal(a.flat, b.flat)


def _offsets(sizes):
    out, o = [], 0
    for n in sizes:
        out.append(o)
        o += n
    return out


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


@pytest.mark.parametrize('fp8_dt,fmt', [(5, fp8.E4M3), (6, fp8.E5M2)])
@pytest.mark.parametrize('norm_type', [1.0, 2.0, float('inf')])
def test_fp8_norms_against_float64(fp8_dt, fmt, norm_type):
    """Per-tensor norms straight from the codes against a float64 evaluation of the dequantized values (to one
    float32 rounding), and against what the reference computes (float32 torch.norm of the dequantized tensor)."""
    from msamp import _backend
    g = torch.Generator().manual_seed(int(norm_type if norm_type < 10 else 7) + fp8_dt)
    sizes = [1, 7, 16384, 16384 * 3 + 11, 100000, 4096 * 1024]
    values, sis = [], []
    for n in sizes:
        top = 0x7B if fmt == fp8.E4M3 else 0x7A
        q = torch.randint(0, top, (n + 1, ), generator=g, dtype=torch.uint8) | (torch.randint(0, 2, (n + 1, ), generator=g, dtype=torch.uint8) << 7)
        values.append(q[1:] if n % 2 else q[:n])    # odd sizes start one byte off a 16-byte boundary
        sis.append(torch.tensor(-2.0 ** float(torch.randint(-12, 3, (1, ), generator=g))))
    got = _backend.fp8_norms([v.cuda() for v in values], [s.cuda() for s in sis], fp8_dt, norm_type).cpu()
    for k, (v, s) in enumerate(zip(values, sis)):
        x = fp8.decode(v, fmt).double() * s.double()
        want = x.abs().max() if norm_type == float('inf') else x.abs().pow(norm_type).sum().pow(1.0 / norm_type)
        assert got[k].item() == pytest.approx(want.item(), rel=2e-7), (k, norm_type)
        ref32 = x.float().abs().max() if norm_type == float('inf') else torch.norm(x.float(), norm_type)
        if v.numel() <= 100000:    # beyond that the CPU's sequential float32 sum is itself off by more than 1e-4
            assert got[k].item() == pytest.approx(ref32.item(), rel=1e-4)


def test_fp8_norms_nan_empty_and_repeat():
    """A NaN code makes that tensor's norm NaN (as torch.norm would) and only that one; an empty tensor has norm 0;
    calling twice gives the same numbers (the scratch accumulators are left clean)."""
    from msamp import _backend
    a = torch.full((40000, ), 0x38, dtype=torch.uint8)    # 1.0 in E4M3
    b = a.clone()
    b[12345] = 0x7F
    vals = [a.cuda(), b.cuda(), torch.zeros(0, dtype=torch.uint8, device='cuda')]
    si = [torch.tensor(0.5, device='cuda')] * 3
    for norm_type, want in ((2.0, 100.0), (1.0, 20000.0), (float('inf'), 0.5)):
        for _ in range(2):
            got = _backend.fp8_norms(vals, si, 5, norm_type).cpu()
            assert got[0].item() == want and math.isnan(got[1].item()) and got[2].item() == 0.0


def test_clip_grad_norm_uses_the_codes():
    """clip_grad_norm_ over FP8 ScalingTensor gradients and a plain bias gradient: the total equals the norm of the
    dequantized gradients, and clipping multiplies every gradient by the same coefficient (scale_inv only for FP8)."""
    import msamp
    from msamp.common.dtype import Dtypes
    from msamp.nn import LinearReplacer
    torch.manual_seed(3)
    model = LinearReplacer.replace(torch.nn.Sequential(torch.nn.Linear(64, 48), torch.nn.Linear(48, 16)).cuda(), Dtypes.kfloat16)
    model(torch.randn(32, 64, device='cuda')).sum().backward()
    params = list(model.parameters())
    for norm_type in (2.0, 1.0, float('inf')):
        flat = torch.cat([p.grad.float().flatten() for p in params]).double()
        want = flat.abs().max() if norm_type == float('inf') else flat.abs().pow(norm_type).sum().pow(1 / norm_type)
        codes = [p.grad.value.clone() for p in params if hasattr(p.grad, 'value')]
        before = [p.grad.float().clone() for p in params]
        total = msamp.clip_grad_norm_(params, want.item() / 4, norm_type=norm_type)
        assert total.item() == pytest.approx(want.item(), rel=1e-5)
        coef = (want.item() / 4) / (total.item() + 1e-6)
        for p, old in zip(params, before):
            assert torch.allclose(p.grad.float(), old * coef, rtol=1e-5, atol=0)
        assert all(torch.equal(c, p.grad.value) for c, p in zip(codes, [p for p in params if hasattr(p.grad, 'value')]))


@pytest.mark.parametrize('speculate', [True, False])
def test_bucket_larger_than_the_caches_equals_its_tensors_one_by_one(speculate):
    """A bucket whose gradients add up to 128 MiB is read as a stream; the same gradients in buckets of one (32 MiB each)
    are not.  Same codes, scales and amax either way, on a first round (fresh metas) and a second one (the scales of
    the first are guessed and mostly hold)."""
    from msamp.nn import GradientBucket
    n = 16 * 1024 * 1024
    g = torch.Generator(device='cuda').manual_seed(9)
    grads = [(torch.randn(n, device='cuda', generator=g) * 10.0 ** (i - 3)).bfloat16() for i in range(4)]
    big = GradientBucket([n] * 4, speculate=speculate)
    small = [GradientBucket([n], speculate=speculate) for _ in range(4)]
    for rnd in range(2):
        if rnd == 1:
            grads = [x * 1.01 for x in grads]
        out_big = big.quantize(grads, world_size=4)
        for i, b in enumerate(small):
            out = b.quantize([grads[i]], world_size=4)[0]
            assert torch.equal(b.flat, big.flat[i * n:(i + 1) * n]), (rnd, i)
            for name in ('scale', 'scale_inv'):
                assert same_float(getattr(out.meta, name), getattr(out_big[i].meta, name)), (rnd, i, name)
            assert same_float(out.meta.amax[0], out_big[i].meta.amax[0])
