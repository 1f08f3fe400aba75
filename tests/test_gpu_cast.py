"""GPU parity of the cast group against the CPU oracle: bytes, amax, scale and scale_inv bit-exact.
All calls go through the C ABI (msamp._backend)."""

import json
import os

import pytest
import torch

from oracle import cast as ocast, fp8, scaling
from tests.gpu_util import FMT, c1_input, make_meta, oracle_meta, same_float

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'reference_kats.json')))


@pytest.fixture(scope='module')
def be():
    from msamp import _backend
    _backend.load()
    return _backend


@pytest.mark.parametrize('fp8_dt', [5, 6])
@pytest.mark.parametrize('src', [torch.float16, torch.bfloat16])
def test_quantize_every_16bit_pattern(be, fp8_dt, src):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(src)
    for scale in (1.0, 2.0**-7, 2.0**9, 3.0):
        s, si, am = make_meta(scale=scale)
        got = be.cast_to_fp8(x.cuda(), s, None, si, fp8_dt).cpu()
        want = fp8.encode(x.float() * torch.tensor(scale), FMT[fp8_dt])
        assert torch.equal(got, want), (fp8_dt, src, scale, (got != want).sum().item())
        assert si.item() == (torch.tensor(1.0) / torch.tensor(scale)).item()


@pytest.mark.parametrize('fp8_dt', [5, 6])
def test_quantize_fp32_fine_grid_and_specials(be, fp8_dt):
    # every float32 whose low 12 mantissa bits are a fixed pattern, across all exponents the format resolves
    hi = torch.arange(0, 1 << 20, dtype=torch.int64)
    bits = ((hi << 12) | 0x7ff).to(torch.int32)    # wraps into negative values too
    x = bits.view(torch.float32)
    s, si, am = make_meta(scale=1.0)
    got = be.cast_to_fp8(x.cuda(), s, None, None, fp8_dt).cpu()
    want = fp8.encode(x, FMT[fp8_dt])
    assert torch.equal(got, want)
    fmax = fp8.FP_MAX[FMT[fp8_dt]]
    sp = torch.tensor([float('nan'), -float('nan'), float('inf'), -float('inf'), fmax, fmax * 1.03, fmax * 1.07, -fmax * 4, 0.0, -0.0, 1e-30])
    got = be.cast_to_fp8(sp.cuda(), s, None, None, fp8_dt).cpu()
    assert torch.equal(got, fp8.encode(sp, FMT[fp8_dt]))


@pytest.mark.parametrize('fp8_dt', [5, 6])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_dequantize_all_codes(be, fp8_dt, out_dtype):
    codes = torch.arange(256, dtype=torch.uint8).repeat(67)    # vector body + scalar tail
    for si_val in (1.0, 1 / 32, 3.0):
        si = torch.full((), si_val, device='cuda')
        got = be.cast_from_fp8(codes.cuda(), si, fp8_dt, out_dtype).cpu()
        want = ocast.cast_from_fp8(codes, torch.tensor(si_val), FMT[fp8_dt], out_dtype)
        assert same_float(got, want)


def test_scale_rule_known_answers_and_adversarial(be):
    k = GOLDEN['scaling_factor']
    for c in k['cases']:
        out = be.compute_scaling_factor(torch.tensor([c['amax']], device='cuda'), torch.tensor([c['scale']], device='cuda'), k['fp_max'], k['margin'])
        assert out.item() == c['expected']
    vals = [0.0, -0.0, -1.0, float('inf'), float('nan'), 1e-45, 1e-42, 1e-38, 3.4e38, 448.0, 449.0, 224.0, 57344.0, 65504.0]
    for fp_max in (448.0, 57344.0, 65504.0):
        for kexp in range(-40, 41):
            base = torch.tensor(fp_max * 2.0**kexp, dtype=torch.float32)
            for _ in range(6):    # amax just around every power-of-two boundary of fp_max/amax
                vals.append(base.item())
                base = torch.nextafter(base, torch.tensor(float('inf')))
            base = torch.tensor(fp_max * 2.0**kexp, dtype=torch.float32)
            for _ in range(6):
                base = torch.nextafter(base, torch.tensor(0.0))
                vals.append(base.item())
    g = torch.Generator().manual_seed(1)
    amax = torch.cat([torch.tensor(vals, dtype=torch.float32), torch.exp(torch.rand(50000, generator=g) * 80 - 40)])
    scale = torch.full_like(amax, 3.0)
    for fp_max in (448.0, 57344.0, 65504.0):
        for margin in (0, 2):
            got = be.compute_scaling_factor(amax.cuda(), scale.cuda(), fp_max, margin).cpu()
            want = scaling.compute_scaling_factor(amax, scale, fp_max, margin)
            assert same_float(got, want), (fp_max, margin, amax[(got != want) & ~(got.isnan() & want.isnan())][:8])
    # one-element fallback scale broadcasts
    got = be.compute_scaling_factor(amax.cuda(), torch.tensor([3.0], device='cuda'), 448.0, 0).cpu()
    assert same_float(got, scaling.compute_scaling_factor(amax, torch.tensor(3.0), 448.0, 0))


@pytest.mark.parametrize('fp8_dt', [5, 6])
def test_config1_in_time_cast_full_size(be, fp8_dt):
    x = c1_input(seed=0)
    s, si, am = make_meta()
    q = be.cast_to_fp8_intime(x.cuda(), s, am[0:1], si, fp8_dt)
    om = oracle_meta()
    want = ocast.cast_to_fp8(x, om, FMT[fp8_dt], in_time=True)
    assert torch.equal(q.cpu(), want)
    assert same_float(am[0], om['amax'][0]) and same_float(s, om['scale']) and same_float(si, om['scale_inv'])
    back = be.cast_from_fp8(q, si, fp8_dt, torch.float32).cpu()
    assert torch.equal(back, ocast.cast_from_fp8(want, om['scale_inv'], FMT[fp8_dt]))
    # run to run determinism
    s2, si2, am2 = make_meta()
    q2 = be.cast_to_fp8_intime(x.cuda(), s2, am2[0:1], si2, fp8_dt)
    assert torch.equal(q, q2) and am2[0].item() == am[0].item()


def test_config5_weight_cast_full_size(be):
    """In-time cast of one Llama-70B MLP weight, bf16 [28672, 8192] = 234 881 024 elements drawn N(0, 0.01) with
    0.01 % of them multiplied by 50.  The oracle checks a slice; the whole tensor is checked through properties that do
    not depend on its size: the amax is the maximum, the scale follows the rule, dequantizing and casting again with
    the same scale gives the same bytes, and no code exceeds the code of the largest element."""
    rows, cols = 28672, 8192
    g = torch.Generator(device='cuda').manual_seed(5)
    x = torch.randn(rows, cols, generator=g, device='cuda') * 0.01
    n = x.numel()
    idx = torch.randint(0, n, (n // 10000, ), generator=g, device='cuda')
    x.view(-1)[idx] *= 50
    x = x.bfloat16()
    for fp8_dt in (5, 6):
        s, si, am = make_meta()
        q = be.cast_to_fp8_intime(x, s, am[0:1], si, fp8_dt)
        assert am[0].item() == x.abs().max().item()
        fp_max = 448.0 if fp8_dt == 5 else 57344.0
        assert same_float(s.cpu(), scaling.compute_scaling_factor(am[0].cpu(), torch.tensor(1.0), fp_max, 0))
        assert same_float(si.cpu(), 1.0 / s.cpu())
        # a slice against the oracle, quantized with the tensor's scale
        part = slice(1234567, 1234567 + (1 << 20))
        om = oracle_meta()
        om['scale'].copy_(s.cpu())
        want = ocast.cast_to_fp8(x.view(-1)[part].cpu(), om, FMT[fp8_dt], in_time=False)
        assert torch.equal(q.view(-1)[part].cpu(), want)
        # idempotence: dequantize, cast with the same (stored) scale -> same bytes
        back = be.cast_from_fp8(q, si, fp8_dt, torch.float32)
        s2, si2, am2 = make_meta()
        s2.copy_(s)
        q2 = be.cast_to_fp8(back, s2, am2[0:1], si2, fp8_dt)
        assert torch.equal(q, q2)
        assert (q & 0x7F).max().item() == (q.view(-1)[x.view(-1).abs().argmax()] & 0x7F).item()
        del back, q2


def test_config5_whole_layer_weight_casts(be):
    """The seven weight matrices of one Llama-70B layer (q, k, v, o, gate, up, down: 855 638 016 bf16 elements), each
    cast in-time twice in a row the way a training loop meets them: the first call finds a fresh meta, the second the
    scale of the step before (the case the speculative kernels are written for), after the weights moved a little.
    Every call: amax is the maximum, the scale follows the rule, the bytes equal those of the plain two-pass kernels
    without speculation, and a slice equals the oracle's cast."""
    shapes = dict(q=(8192, 8192), k=(1024, 8192), v=(1024, 8192), o=(8192, 8192), gate=(28672, 8192), up=(28672, 8192),
                  down=(8192, 28672))
    assert sum(r * c for r, c in shapes.values()) == 855_638_016
    g = torch.Generator(device='cuda').manual_seed(70)
    for i, (name, (rows, cols)) in enumerate(shapes.items()):
        w = (torch.randn(rows, cols, generator=g, device='cuda') * 0.02).bfloat16()
        s, si, am = make_meta()
        for step in range(2):
            if step == 1:
                w = (w.float() * (1.0 + 0.001 * i) + 1e-4).bfloat16()
            q = be.cast_to_fp8_intime(w, s, am[0:1], si, 5)
            assert am[0].item() == w.abs().max().item(), name
            assert same_float(s.cpu(), scaling.compute_scaling_factor(am[0].cpu(), torch.tensor(1.0), 448.0, 0)), name
            assert same_float(si.cpu(), 1.0 / s.cpu()), name
            s2, si2, am2 = make_meta()
            plain = be.cast_to_fp8_intime(w, s2, am2[0:1], si2, 5, two_pass=True, speculate=False)
            assert torch.equal(q, plain) and same_float(s, s2) and same_float(am[0], am2[0]), name
            del plain
            start = (rows * cols // 3) & ~15
            part = slice(start, start + (1 << 18))
            om = oracle_meta()
            om['scale'].copy_(s.cpu())
            want = ocast.cast_to_fp8(w.view(-1)[part].cpu(), om, FMT[5], in_time=False)
            assert torch.equal(q.view(-1)[part].cpu(), want), name
            del q
        del w


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('n', [1, 3, 1000, 4097, 16384 * 3 + 5, 1 << 20])
def test_in_time_cast_ragged_sizes(be, dtype, n):
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(n + 1, generator=g) * 3).to(dtype)
    xg = x.cuda()
    for off, fp8_dt in ((0, 5), (1, 6)):    # offset 1 makes the device view misaligned for vector loads
        view = x[off:off + n]
        s, si, am = make_meta()
        q = be.cast_to_fp8_intime(xg[off:off + n], s, am[0:1], si, fp8_dt)
        om = oracle_meta()
        want = ocast.cast_to_fp8(view, om, FMT[fp8_dt], in_time=True)
        assert torch.equal(q.cpu(), want)
        assert same_float(am[0], om['amax'][0]) and same_float(s, om['scale']) and same_float(si, om['scale_inv'])


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('n', [512 * 4 + 3, 5_000_003, 512 * 512 * 16 * 4 + 8, 20_000_000])
def test_in_time_cast_one_pass_matches_two_pass(be, dtype, n):
    """The register-resident kernel (partly filled rounds, the largest tensor it takes, one past it)
    against the two-pass kernels: same bytes, same meta; repeated calls reuse the workspace slots."""
    g = torch.Generator().manual_seed(n % 1000)
    x = (torch.randn(n, generator=g) * 5).to(dtype).cuda()
    x[n // 3] = 300.0
    for fp8_dt in (5, 6):
        s1, si1, am1 = make_meta(scale=2.0)
        q1 = be.cast_to_fp8_intime(x, s1, am1[0:1], si1, fp8_dt)
        s2, si2, am2 = make_meta(scale=2.0)
        q2 = be.cast_to_fp8_intime(x, s2, am2[0:1], si2, fp8_dt, two_pass=True)
        assert torch.equal(q1, q2)
        assert same_float(am1, am2) and same_float(s1, s2) and same_float(si1, si2)
        assert am1[0].item() == 300.0


def test_in_time_cast_on_a_second_stream(be):
    """Only one stream per device runs the one-pass kernel; another stream gets the same answer."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1 << 20, generator=g).cuda()
    s1, si1, am1 = make_meta()
    q1 = be.cast_to_fp8_intime(x, s1, am1[0:1], si1, 5)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        s2, si2, am2 = make_meta()
        q2 = be.cast_to_fp8_intime(x, s2, am2[0:1], si2, 5)
    side.synchronize()
    assert torch.equal(q1, q2) and same_float(am1, am2) and same_float(s1, s2) and same_float(si1, si2)


def test_casts_beyond_2_31_elements(be):
    """64-bit indexing: 2^31 + 8 bf16 elements through the in-time cast (two passes at this size), the delayed cast
    and the dequantization; the maximum sits in the last element, slices at both ends and across the 2^31 mark are
    compared with the oracle."""
    n = (1 << 31) + 8
    x = torch.empty(n, dtype=torch.bfloat16, device='cuda')
    g = torch.Generator(device='cuda').manual_seed(31)
    step = 1 << 28
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        x[lo:hi] = torch.randn(hi - lo, generator=g, device='cuda').bfloat16()
    x[n - 1] = 77.0
    s, si, am = make_meta()
    q = be.cast_to_fp8_intime(x, s, am[0:1], si, 5)
    assert am[0].item() == 77.0 and s.item() == 4.0 and si.item() == 0.25
    s2, si2, am2 = make_meta(scale=4.0)
    q2 = be.cast_to_fp8(x, s2, am2[0:1], si2, 5)
    assert am2[0].item() == 77.0
    back = be.cast_from_fp8(q, si, 5, torch.bfloat16)
    for lo, hi in ((0, 4096), ((1 << 31) - 2048, (1 << 31) + 8), (n - 4099, n)):
        om = oracle_meta(scale=4.0)
        want = ocast.cast_to_fp8(x[lo:hi].cpu(), om, FMT[5], in_time=False)
        assert torch.equal(q[lo:hi].cpu(), want) and torch.equal(q2[lo:hi].cpu(), want)
        assert torch.equal(back[lo:hi].cpu(), ocast.cast_from_fp8(want, torch.tensor(0.25), FMT[5], torch.bfloat16))
    assert torch.equal(q[1 << 30:(1 << 30) + (1 << 20)], q2[1 << 30:(1 << 30) + (1 << 20)])


def test_two_pass_casts_on_two_streams_at_once(be):
    """Two streams each run two-pass in-time casts of different tensors with nothing ordering them: each stream has
    its own scratch words, so neither sees the other's partial maxima."""
    g = torch.Generator().manual_seed(4)
    xa = (torch.randn(6_000_000, generator=g) * 3).cuda()
    xb = (torch.randn(6_000_000, generator=g) * 0.01).cuda()
    want = []
    for x in (xa, xb):
        s, si, am = make_meta()
        want.append((be.cast_to_fp8_intime(x, s, am[0:1], si, 5, two_pass=True), s, am))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    got_a, got_b = [], []
    for _ in range(8):
        s, si, am = make_meta()
        got_a.append((be.cast_to_fp8_intime(xa, s, am[0:1], si, 5, two_pass=True), s, am))
        with torch.cuda.stream(side):
            s, si, am = make_meta()
            got_b.append((be.cast_to_fp8_intime(xb, s, am[0:1], si, 5, two_pass=True), s, am))
    torch.cuda.synchronize()
    for got, ref in ((got_a, want[0]), (got_b, want[1])):
        for q, s, am in got:
            assert torch.equal(q, ref[0]) and same_float(s, ref[1]) and same_float(am, ref[2])


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('counter', [0, 3, 4, 100])
def test_gated_casts_follow_the_device_counter(be, dtype, counter):
    """Warm-up test on the GPU: counter < window -> the in-time cast, else the delayed cast; both byte
    for byte, plain and with the fused transpose, NaN input included."""
    window = 4
    g = torch.Generator().manual_seed(counter)
    x = (torch.randn(192, 320, generator=g) * 3).to(dtype)
    x[5, 7] = float('nan')
    xg = x.cuda()
    cnt = torch.full((), counter, dtype=torch.int32, device='cuda')
    in_time = counter < window
    for fp8_dt in (5, 6):
        s, si, am = make_meta(window=window, scale=2.0)
        am[0] = 0.5
        q = be.cast_to_fp8_gated(xg, s, am[0:1], si, fp8_dt, cnt, window)
        s2, si2, am2 = make_meta(window=window, scale=2.0)
        am2[0] = 0.5
        if in_time:
            want = be.cast_to_fp8_intime(xg, s2, am2[0:1], si2, fp8_dt)
        else:
            want = be.cast_to_fp8(xg, s2, am2[0:1], si2, fp8_dt)
        assert torch.equal(q, want) and same_float(am, am2) and same_float(s, s2) and same_float(si, si2)
        s, si, am = make_meta(window=window, scale=2.0)
        q, qt = be.cast_transpose_gated(xg, s, am[0:1], si, fp8_dt, cnt, window)
        s2, si2, am2 = make_meta(window=window, scale=2.0)
        want, want_t = be.cast_transpose(xg, s2, am2[0:1], si2, fp8_dt, in_time=in_time)
        assert torch.equal(q, want) and torch.equal(qt, want_t)
        assert same_float(am, am2) and same_float(s, s2) and same_float(si, si2)
    assert cnt.item() == counter


def test_window_update_keeps_device_counters(be):
    scales = torch.tensor([1.0, 2.0, 4.0], device='cuda')
    amaxs = torch.tensor([[3.0, 1.0], [float('inf'), 2.0], [float('nan'), 0.0]], device='cuda')
    counters = torch.tensor([5, 6, 7], dtype=torch.int32, device='cuda')
    assert be.scale_update(scales, amaxs, 448.0, 0, counters=counters, want_mask=False) is None
    assert counters.tolist() == [6, 0, 0]
    assert amaxs.tolist() == [[0.0, 3.0], [0.0, 0.0], [0.0, 0.0]]
    assert scales.tolist() == [128.0, 128.0, 4.0]


def test_grouped_window_update_matches_group_by_group(be):
    """Two groups of different format, size and window in one launch against one launch per group; a window wider
    than a wavefront takes the group-by-group route inside the library."""
    g = torch.Generator().manual_seed(3)
    for windows in ((16, 16), (16, 1), (3, 70)):
        groups = []
        for n, window, fp_max in ((5, windows[0], 448.0), (9, windows[1], 57344.0)):
            scales = torch.rand(n, generator=g) + 0.5
            amaxs = torch.rand(n, window, generator=g) * 100
            amaxs[1, 0] = float('inf')
            amaxs[n - 1, 0] = float('nan')
            counters = torch.randint(0, 20, (n, ), generator=g, dtype=torch.int32)
            groups.append((scales, amaxs, fp_max, counters))
        one = [(s.clone().cuda(), a.clone().cuda(), f, c.clone().cuda()) for s, a, f, c in groups]
        be.scale_update_groups(one, 0)
        for (s, a, f, c), (s1, a1, _, c1) in zip(groups, one):
            s2, a2, c2 = s.clone().cuda(), a.clone().cuda(), c.clone().cuda()
            be.scale_update(s2, a2, f, 0, counters=c2, want_mask=False)
            assert same_float(s1, s2) and same_float(a1, a2) and torch.equal(c1, c2)
    be.scale_update_groups([], 0)
    # more groups than one launch takes: the wrapper splits them, the library itself refuses
    be.scale_update_groups([(s.clone().cuda(), a.clone().cuda(), f, None) for s, a, f, _ in groups] * 3, 0)
    assert be.load().msamp_scale_update_groups(None, be.MAX_SCALE_GROUPS + 1, 0, None) == -2


def test_delayed_cast_accumulates_amax_and_skips_nan(be):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(100000, generator=g).to(torch.bfloat16)
    x[17] = float('nan')
    s, si, am = make_meta(window=4, scale=16.0)
    om = oracle_meta(window=4, scale=16.0)
    for mult in (1.0, 4.0, 0.5):
        xm = x * mult    # formed once on the host so both sides see identical bits (NaN included)
        q = be.cast_to_fp8(xm.cuda(), s, am[0:1], si, 5)
        want = ocast.cast_to_fp8(xm, om, fp8.E4M3, in_time=False)
        assert torch.equal(q.cpu(), want)
        assert same_float(am, om['amax']) and s.item() == 16.0 and si.item() == 1 / 16
    assert q.cpu()[17].item() & 0x7F == 0x7F


def test_in_time_nan_inf_and_sync_semantics(be):
    x = torch.tensor([1.0, float('nan'), -2.0, 0.5] * 300)
    s, si, am = make_meta(scale=8.0)
    q = be.cast_to_fp8_intime(x.cuda(), s, am[0:1], si, 5)
    om = oracle_meta(scale=8.0)
    want = ocast.cast_to_fp8(x, om, fp8.E4M3, in_time=True)
    assert torch.isnan(am[0]).item() and s.item() == 8.0 and si.item() == 0.125 and torch.equal(q.cpu(), want)
    s, si, am = make_meta(scale=8.0)
    q = be.cast_to_fp8_intime(x.cuda(), s, am[0:1], si, 5, nan_to_inf=True)
    om = oracle_meta(scale=8.0)
    want = ocast.cast_to_fp8(x, om, fp8.E4M3, in_time=True, sync=True)
    assert am[0].item() == float('inf') and s.item() == 0.125 and si.item() == 8.0 and torch.equal(q.cpu(), want)
    xi = torch.tensor([1.0, float('inf'), -float('inf')] * 100)
    s, si, am = make_meta(scale=8.0)
    q = be.cast_to_fp8_intime(xi.cuda(), s, am[0:1], si, 6)
    om = oracle_meta(scale=8.0)
    want = ocast.cast_to_fp8(xi, om, fp8.E5M2, in_time=True)
    assert am[0].item() == float('inf') and same_float(s, om['scale']) and torch.equal(q.cpu(), want)
    z = torch.zeros(5000)
    s, si, am = make_meta(scale=4.0)
    q = be.cast_to_fp8_intime(z.cuda(), s, am[0:1], si, 5)
    assert am[0].item() == 0.0 and s.item() == 4.0 and si.item() == 0.25 and q.sum().item() == 0


@pytest.mark.parametrize('shape', [(64, 64), (100, 36), (17, 5), (1, 130), (257, 1), (512, 1024), (96, 4100), (144, 272), (4112, 48), (16, 1040)])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_cast_transpose(be, shape, dtype):
    g = torch.Generator().manual_seed(shape[0] * 7 + shape[1])
    x = (torch.randn(*shape, generator=g) * 2).to(dtype)
    # in time, E5M2 (the output-gradient case)
    s, si, am = make_meta()
    q, qt = be.cast_transpose(x.cuda(), s, am[0:1], si, 6, in_time=True)
    om = oracle_meta()
    want, want_t = ocast.cast_transpose(x, om, fp8.E5M2, in_time=True)
    assert torch.equal(q.cpu(), want) and torch.equal(qt.cpu(), want_t)
    assert same_float(am[0], om['amax'][0]) and same_float(s, om['scale']) and same_float(si, om['scale_inv'])
    # delayed, E4M3
    s, si, am = make_meta(window=2, scale=4.0)
    q, qt = be.cast_transpose(x.cuda(), s, am[0:1], si, 5)
    om = oracle_meta(window=2, scale=4.0)
    want, want_t = ocast.cast_transpose(x, om, fp8.E4M3, in_time=False)
    assert torch.equal(q.cpu(), want) and torch.equal(qt.cpu(), want_t)
    assert same_float(am, om['amax']) and si.item() == 0.25
    # separate transpose of the payload equals the fused one
    assert torch.equal(be.fp8_transpose(q), qt)


def test_fp8_transpose_is_involution_at_full_size(be):
    g = torch.Generator().manual_seed(2)
    q = torch.randint(0, 256, (8192, 4096), dtype=torch.uint8, generator=g).cuda()
    t = be.fp8_transpose(q)
    assert t.shape == (4096, 8192) and torch.equal(t, q.t().contiguous())
    assert torch.equal(be.fp8_transpose(t), q)


@pytest.mark.parametrize('shape', [(16, 16), (144, 272), (4112, 48), (128, 128), (48, 1040), (130, 64), (64, 130)])
def test_fp8_transpose_shapes(be, shape):
    """Multiples of 16 take the 128x128-tile kernel (partial tiles at the edges), the rest the 64x64 one;
    a misaligned view must not take the 16-byte path."""
    g = torch.Generator().manual_seed(shape[0] + shape[1])
    q = torch.randint(0, 256, shape, dtype=torch.uint8, generator=g).cuda()
    assert torch.equal(be.fp8_transpose(q), q.t().contiguous())
    flat = torch.randint(0, 256, (shape[0] * shape[1] + 1,), dtype=torch.uint8, generator=g).cuda()
    view = flat[1:].view(shape)
    assert torch.equal(be.fp8_transpose(view), view.t().contiguous())


def test_scaled_16bit_payloads(be):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(70001, generator=g) * 1e-3
    for out_dtype in (torch.float16, torch.bfloat16, torch.float32):
        sc = torch.tensor(2.0**14)
        got = be.scale_cast(x.cuda(), sc.cuda(), out_dtype).cpu()
        assert same_float(got.float(), (x * sc.view(1)).to(out_dtype).float())
    big = torch.tensor([70000.0, -70000.0, 1.0]).cuda()
    assert be.scale_cast(big, torch.ones((), device='cuda'), torch.float16).cpu().tolist() == [float('inf'), -float('inf'), 1.0]
    am = torch.zeros(1, device='cuda')
    be.amax(x.cuda().half(), am)
    assert am.item() == x.half().abs().max().item()
    be.amax(x.cuda(), am)
    assert am.item() == x.abs().max().item()


def test_window_update_sequence(be):
    k = GOLDEN['window']
    w = k['window_size']
    scales = torch.ones(3, device='cuda')
    amaxs = torch.zeros(3, w, device='cuda')
    o_scales, o_amaxs, o_cnt = torch.ones(3), torch.zeros(3, w), torch.zeros(3, dtype=torch.int32)
    recent = []
    for step, i in enumerate(list(range(k['inputs_cycle'])) * k['repeats']):
        cur = torch.tensor([float(i), float(i) * 0.37, float('inf') if step % 11 == 5 else 2.0 * i])
        amaxs[:, 0] = cur.cuda()
        o_amaxs[:, 0] = cur
        recent = (recent + [i])[-w:]
        assert amaxs[0].max().item() == max(recent)
        bad = be.scale_update(scales, amaxs, 448.0, 0).cpu().bool()
        o_bad = scaling.update_scaling_factors(o_scales, o_amaxs, o_cnt, 448.0)
        assert torch.equal(bad, o_bad) and same_float(scales, o_scales) and same_float(amaxs, o_amaxs)


def _spec_sequence(be, xs, fp8_dt, two_pass, nan_to_inf=False):
    """The same calls on two metas: with speculation (the default) and with the plain kernels; everything must agree
    after every call.  Returns the speculative side's outputs and meta snapshots."""
    ms, mr = make_meta(), make_meta()
    outs = []
    for x in xs:
        q = be.cast_to_fp8_intime(x, ms[0], ms[2][0:1], ms[1], fp8_dt, two_pass=two_pass, nan_to_inf=nan_to_inf)
        r = be.cast_to_fp8_intime(x, mr[0], mr[2][0:1], mr[1], fp8_dt, two_pass=True, speculate=False, nan_to_inf=nan_to_inf)
        torch.cuda.synchronize()
        assert torch.equal(q, r)
        assert same_float(ms[0], mr[0]) and same_float(ms[1], mr[1]) and same_float(ms[2], mr[2])
        outs.append((q, ms[0].clone(), ms[1].clone(), ms[2].clone()))
    return outs


@pytest.mark.parametrize('two_pass', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fmt,dt', [(fp8.E4M3, 5), (fp8.E5M2, 6)])
def test_speculative_in_time_cast_hit_miss_and_special_values(be, dtype, two_pass, fmt, dt):
    """Speculation on the old scale (one-pass kernel: stores before the meeting; two-pass: stores in the first pass):
    never-used meta, confirmed scale, changed scale (both directions), NaN / Inf / all-zero inputs, a ragged length --
    bit-equal to the plain kernels after every call, and to the oracle."""
    g = torch.Generator().manual_seed(21)
    n = 1024 * 1024 + 13
    x = (torch.randn(n, generator=g) * 3).to(dtype)
    bad = x.clone()
    bad[17], bad[n - 1] = float('nan'), float('inf')
    inf = x.clone()
    inf[5] = -float('inf')
    cpu = [x, x, x * 8, x * 8, (x.float() * 2.0**-6).to(dtype), bad, x, torch.zeros(n, dtype=dtype), inf, x[:1000], x[:3]]
    outs = _spec_sequence(be, [c.cuda() for c in cpu], dt, two_pass)
    om = oracle_meta()
    for c, (q, s, si, am) in zip(cpu, outs):
        want = ocast.cast_to_fp8(c, om, fmt, in_time=True)
        assert torch.equal(q.cpu(), want)
        assert same_float(s, om['scale']) and same_float(si, om['scale_inv']) and same_float(am[0], om['amax'][0])
    _spec_sequence(be, [c.cuda() for c in cpu[:6]], dt, two_pass, nan_to_inf=True)


@pytest.mark.parametrize('dtype,n', [(torch.float32, 17 * 1024 * 1024 + 9), (torch.bfloat16, 34 * 1024 * 1024 + 24)])
def test_speculative_in_time_cast_beyond_the_one_pass_limit(be, dtype, n):
    """More than 64 MiB of input: two launches, the first one writing the output on speculation."""
    g = torch.Generator(device='cuda').manual_seed(22)
    x = (torch.randn(n, device='cuda', generator=g) * 0.01).to(dtype)
    y = x.clone()
    y[n // 3] = 50.0
    outs = _spec_sequence(be, [x, x, y, y, x], be.DT_E4M3, False)
    # the oracle on the first 2 Mi elements of the confirmed-scale call and of the changed-scale call
    head = 2 * 1024 * 1024
    for idx, src in ((1, x), (2, y)):
        q, s, si, am = outs[idx]
        assert am[0].item() == src.float().abs().max().item()
        want = fp8.encode(src[:head].float().cpu() * s.cpu(), fp8.E4M3)
        assert torch.equal(q[:head].cpu(), want)
