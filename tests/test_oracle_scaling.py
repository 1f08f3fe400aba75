"""Pins the oracle's pow-2 scale rule and amax-window update."""

import json
import math
import os

import numpy as np
import torch

from oracle import scaling, cast as ocast, fp8

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'reference_kats.json')))


def _sf(amax, scale=1.0, fp_max=448.0, margin=0):
    return scaling.compute_scaling_factor(torch.tensor(amax, dtype=torch.float32), torch.tensor(scale), fp_max, margin).item()


def test_reference_known_answers():
    k = GOLDEN['scaling_factor']
    for c in k['cases']:
        assert _sf(c['amax'], c['scale'], k['fp_max'], k['margin']) == c['expected']


def test_closed_form_and_invariants():
    g = torch.Generator().manual_seed(3)
    amax = torch.exp(torch.rand(20000, generator=g) * 60 - 30)    # 1e-13 .. 1e13
    for fp_max in (448.0, 57344.0, 65504.0):
        sf = scaling.compute_scaling_factor(amax, torch.ones(()), fp_max, 0)
        # power of two
        m, _ = np.frexp(sf.numpy().astype(np.float64))
        assert np.all(m == 0.5)
        # sf * amax <= fp_max < 2 * sf * amax, except for the few amax within float-log2 rounding of a
        # power-of-two boundary (fp_max/amax a hair below 2^k rounds up to k): there sf may be one binade up
        prod = sf.double() * amax.double()
        ok = (prod <= fp_max) & (2 * prod > fp_max)
        near = (prod / fp_max - 1).abs() < 1e-6
        assert torch.all(ok | near)
        # exact closed form in double away from boundaries
        exact = torch.pow(2.0, torch.floor(torch.log2(torch.tensor(fp_max, dtype=torch.float64) / amax.double())))
        frac = torch.log2(torch.tensor(fp_max, dtype=torch.float64) / amax.double())
        away = (frac - torch.round(frac)).abs() > 1e-5
        assert torch.equal(sf.double()[away], exact[away])


def test_margin_shifts_by_binades():
    for margin in (1, 3):
        assert _sf(10.0, margin=margin) == 32.0 / 2**margin
        assert _sf(10000.0, margin=margin) == 1.0 / 32 / 2**margin


def test_special_values():
    inf, nan = float('inf'), float('nan')
    assert _sf(0.0, scale=3.0) == 3.0
    assert _sf(-1.0, scale=3.0) == 3.0
    assert _sf(nan, scale=3.0) == 3.0
    assert _sf(inf, scale=4.0) == 0.25    # exp = -inf < 0 inverts the kept scale
    assert _sf(1e-42, scale=3.0) == inf    # fp_max / denormal overflows
    assert _sf(448.0) == 1.0 and _sf(449.0) == 0.5 and _sf(224.0) == 2.0 and _sf(224.00002) == 1.0


def test_power_of_two_boundary_follows_float_log2():
    # fp_max/amax one float below 2^5: the float log2 rounds to 5.0, so the rule yields 32, not 16
    q = np.nextafter(np.float32(32.0), np.float32(0))
    amax = np.float32(448.0) / q
    assert np.float32(448.0) / np.float32(amax) == q
    assert _sf(float(amax)) == 32.0
    assert math.floor(math.log2(float(q))) == 4


def test_window_update_sequence():
    k = GOLDEN['window']
    w = k['window_size']
    scales, amaxs, counters = torch.ones(1), torch.zeros(1, w), torch.zeros(1, dtype=torch.int32)
    recent = []
    step = 0
    for i in list(range(k['inputs_cycle'])) * k['repeats']:
        amaxs[0, 0] = max(amaxs[0, 0].item(), float(i))    # what a cast of full((1,4), i) leaves in amax[0]
        recent = (recent + [i])[-w:]
        assert amaxs.max().item() == max(recent)
        scaling.update_scaling_factors(scales, amaxs, counters, 448.0)
        step += 1
        assert counters.item() == step
        assert amaxs[0, 0].item() == 0
        assert scales.item() == _sf(float(max(recent)))


def test_window_update_drops_nonfinite_and_resets_counter():
    scales, amaxs, counters = torch.tensor([2.0, 2.0]), torch.tensor([[float('inf'), 3.0], [5.0, 1.0]]), torch.tensor([7, 7], dtype=torch.int32)
    bad = scaling.update_scaling_factors(scales, amaxs, counters, 448.0)
    assert bad.tolist() == [True, False]
    assert counters.tolist() == [0, 8]
    assert amaxs.tolist() == [[0.0, 0.0], [0.0, 5.0]]
    assert scales.tolist() == [_sf(3.0), _sf(5.0)]


def test_cast_state_machine_in_time_and_delayed():
    x = torch.tensor([0.5, -3.0, 10.0, 0.0])
    meta = ocast.new_meta(window=2)
    q = ocast.cast_to_fp8(x, meta, fp8.E4M3, in_time=True)
    assert meta['amax'][0].item() == 10.0 and meta['scale'].item() == 32.0 and meta['scale_inv'].item() == 1 / 32
    assert torch.equal(fp8.decode(q, fp8.E4M3) / 32, x)
    # delayed: keeps the scale, folds the larger amax in
    q2 = ocast.cast_to_fp8(x * 4, meta, fp8.E4M3, in_time=False)
    assert meta['scale'].item() == 32.0 and meta['amax'][0].item() == 40.0
    assert fp8.decode(q2, fp8.E4M3).tolist() == [64.0, -384.0, 448.0, 0.0]    # 1280 saturates
    # delayed amax ignores NaN, in-time amax propagates it and then keeps the old scale
    xn = torch.tensor([1.0, float('nan')])
    m2 = ocast.new_meta()
    ocast.cast_to_fp8(xn, m2, fp8.E4M3, in_time=False)
    assert m2['amax'][0].item() == 1.0
    m3 = ocast.new_meta()
    m3['scale'] = torch.tensor(8.0)
    q3 = ocast.cast_to_fp8(xn, m3, fp8.E4M3, in_time=True)
    assert math.isnan(m3['amax'][0].item()) and m3['scale'].item() == 8.0
    assert q3.tolist() == [fp8.encode(torch.tensor([8.0]), fp8.E4M3).item(), 0x7F]
    # sync: NaN amax becomes +Inf and the rule then returns 1/scale
    m4 = ocast.new_meta()
    m4['scale'] = torch.tensor(8.0)
    ocast.cast_to_fp8(xn, m4, fp8.E4M3, in_time=True, sync=True)
    assert m4['amax'][0].item() == float('inf') and m4['scale'].item() == 0.125


def test_scaled_fp16_to_fp8_reference_case_and_invariants():
    """The reference's own case (tests/common/tensor/test_tensor.py:186-196): 2**-17 as a scaled float16 tensor, then
    to E4M3, comes back exactly.  Worked by hand: amax 2**-17 gives the float16 scale 2**32 (payload 2**15) and the
    E4M3 scale 2**25, so the payload is quantized with 2**25 / 2**32 = 2**-7 to 256 = code 0x78, and the new
    scale_inv is 2**-25."""
    for src in (torch.float16, torch.float32):
        value = torch.tensor([2.0**-17], dtype=torch.float16).to(src)
        m16 = ocast.new_meta()
        v16 = ocast.cast_to_fp16(value, m16, in_time=True)
        assert v16.dtype == torch.float16 and v16.item() == 2.0**15
        assert m16['scale'].item() == 2.0**32 and m16['scale_inv'].item() == 2.0**-32
        q, m8 = ocast.scaled_fp16_to_fp8(v16, m16, fp8.E4M3)
        assert q.tolist() == [0x78] and m8['scale_inv'].item() == 2.0**-25 and m8['scale'].item() == 2.0**-7
        assert m8['amax'][0].item() == 2.0**-17
        assert (fp8.decode(q, fp8.E4M3) * m8['scale_inv']).item() == 2.0**-17
    # Values with few significant bits survive the float16 stop unchanged, so the two-step route must give the codes
    # and the scale_inv of the direct in-time cast (a missing or inverted factor fails here for every element).
    g = torch.Generator().manual_seed(3)
    x = torch.randint(-15, 16, (4096, ), generator=g).float() * torch.exp2(torch.randint(-6, 3, (4096, ), generator=g).float())
    x[0] = 15 * 4.0    # the amax
    for fmt in (fp8.E4M3, fp8.E5M2):
        direct_meta = ocast.new_meta()
        direct = ocast.cast_to_fp8(x, direct_meta, fmt, in_time=True)
        m16 = ocast.new_meta()
        v16 = ocast.cast_to_fp16(x, m16, in_time=True)
        assert torch.equal(v16.float() * m16['scale_inv'], x)
        q, m8 = ocast.scaled_fp16_to_fp8(v16, m16, fmt)
        assert torch.equal(q, direct) and m8['scale_inv'].item() == direct_meta['scale_inv'].item()
        assert m8['amax'][0].item() == 60.0


def test_cast_again_after_the_scale_was_touched():
    """tests/common/tensor/test_tensor.py:277-285: an in-time cast recomputes the scale, so doubling the stored scale
    between two casts of one tensor changes nothing."""
    x = torch.randn(64, generator=torch.Generator().manual_seed(0))
    for fmt in (fp8.E4M3, fp8.E5M2):
        meta = ocast.new_meta()
        q1 = ocast.cast_to_fp8(x, meta, fmt, in_time=True)
        first = fp8.decode(q1, fmt) * meta['scale_inv']
        meta['scale'] = meta['scale'] * 2
        q2 = ocast.cast_to_fp8(x, meta, fmt, in_time=True)
        assert torch.equal(q1, q2) and torch.equal(fp8.decode(q2, fmt) * meta['scale_inv'], first)
