"""Pins the CPU oracle's FP8 codec: closed form, brute force, library cross-check, reference bytes."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import fp8

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'reference_kats.json')))


def test_reference_byte_vectors():
    table = fp8.decode_table(fp8.E4M3)
    for code, value in GOLDEN['e4m3_bytes']['pairs']:
        assert table[code] == value
    # the reference's FP8 all-reduce sums: decode, add, encode gives the expected byte
    for a, b, s in GOLDEN['e4m3_bytes']['sums']:
        total = torch.tensor([float(table[a] + table[b])])
        assert fp8.encode(total, fp8.E4M3).item() == s
    for a, b, m in GOLDEN['e4m3_bytes']['max']:
        assert max(table[a], table[b]) == table[m]
    for a, b, m in GOLDEN['e4m3_bytes']['min']:
        assert min(table[a], table[b]) == table[m]


@pytest.mark.parametrize('fmt,fmax,min_sub,n_nan', [(fp8.E4M3, 448.0, 2.0**-9, 2), (fp8.E5M2, 57344.0, 2.0**-16, 6)])
def test_decode_table_structure(fmt, fmax, min_sub, n_nan):
    t = fp8.decode_table(fmt)
    finite = t[np.isfinite(t)]
    assert finite.max() == fmax and finite.min() == -fmax
    assert np.isnan(t).sum() == n_nan
    assert np.isinf(t).sum() == (0 if fmt == fp8.E4M3 else 2)
    pos = t[:128][np.isfinite(t[:128])]
    assert np.all(np.diff(pos) > 0), 'positive codes must be strictly increasing'
    assert pos[0] == 0.0 and pos[1] == min_sub
    assert np.array_equal(t[128:][np.isfinite(t[128:])], -pos)
    # torch's own decode of the same bytes
    dt = torch.float8_e4m3fn if fmt == fp8.E4M3 else torch.float8_e5m2
    ref = torch.arange(256, dtype=torch.uint8).view(dt).to(torch.float32).numpy()
    assert np.array_equal(np.nan_to_num(ref, nan=1e30), np.nan_to_num(t, nan=1e30))


@pytest.mark.parametrize('fmt', [fp8.E4M3, fp8.E5M2])
def test_encode_round_trip_all_codes(fmt):
    t = fp8.decode_table(fmt)
    codes = np.array([c for c in range(256) if np.isfinite(t[c])], dtype=np.uint8)
    back = fp8.encode(torch.from_numpy(t[codes]), fmt).numpy()
    # -0 and +0 are distinct codes and both must survive
    assert np.array_equal(back, codes)


@pytest.mark.parametrize('fmt', [fp8.E4M3, fp8.E5M2])
@pytest.mark.parametrize('src', ['fp16', 'bf16'])
@pytest.mark.parametrize('scale', [1.0, 2.0**-7, 2.0**9])
def test_encode_matches_bruteforce_on_every_16bit_pattern(fmt, src, scale):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.float16 if src == 'fp16' else torch.bfloat16).to(torch.float32)
    y = x * scale
    got = fp8.encode(y, fmt).numpy()
    want = fp8.encode_bruteforce(y.numpy(), fmt)
    assert np.array_equal(got, want)


@pytest.mark.parametrize('fmt', [fp8.E4M3, fp8.E5M2])
def test_saturation_ties_and_specials(fmt):
    fmax = fp8.FP_MAX[fmt]
    x = torch.tensor([fmax, fmax * 1.01, fmax * 1.07, fmax * 2, 1e30, float('inf'), -float('inf'), -1e30])
    top = 0x7E if fmt == fp8.E4M3 else 0x7B
    assert fp8.encode(x, fmt).tolist() == [top] * 6 + [top | 0x80] * 2
    nan = torch.tensor([float('nan'), -float('nan')])
    assert fp8.encode(nan, fmt).tolist() == [0x7F, 0xFF]
    # ties to even at the smallest subnormal step: 0.5 ulp -> 0, 1.5 ulp -> 2 ulp
    ulp = 2.0**-9 if fmt == fp8.E4M3 else 2.0**-16
    assert fp8.encode(torch.tensor([0.5 * ulp, 1.5 * ulp, 2.5 * ulp, -0.5 * ulp]), fmt).tolist() == [0, 2, 2, 0x80]


def test_half_ulp_error_bound():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(100000, generator=g) * 20
    for fmt in (fp8.E4M3, fp8.E5M2):
        q = fp8.encode(x, fmt)
        back = fp8.decode(q, fmt)
        mbits = 3 if fmt == fp8.E4M3 else 2
        emin = -6 if fmt == fp8.E4M3 else -14
        expo = torch.floor(torch.log2(x.abs().clamp_min(2.0**emin)))
        half_ulp = 2.0**(expo - mbits - 1)
        assert torch.all((back - x).abs() <= half_ulp * (1 + 1e-6))
