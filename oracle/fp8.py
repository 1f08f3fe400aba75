"""OCP FP8 codec (E4M3FN, E5M2) on the CPU.  Test infrastructure only.

Follows the formats named at msamp/common/dtype/floating.py:39-46 (E4M3 without
infinities, max 448; E5M2 IEEE-like, max 57344) and the saturating
round-to-nearest-even conversion the reference obtains from TransformerEngine
(msamp/common/utils/transformer_engine_wrapper.py:106-137).
"""

import numpy as np
import torch

E4M3 = 'e4m3'
E5M2 = 'e5m2'

FP_MAX = {E4M3: 448.0, E5M2: 57344.0}
_TORCH_DT = {E4M3: torch.float8_e4m3fn, E5M2: torch.float8_e5m2}


def decode_table(fmt):
    """All 256 code values as float32, from the bit-field definition of the format."""
    ebits, mbits, bias = (4, 3, 7) if fmt == E4M3 else (5, 2, 15)
    out = np.zeros(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> mbits) & ((1 << ebits) - 1)
        m = code & ((1 << mbits) - 1)
        if fmt == E4M3 and e == 15 and m == 7:
            val = float('nan')
        elif fmt == E5M2 and e == 31:
            val = float('inf') if m == 0 else float('nan')
        elif e == 0:
            val = m * 2.0**(1 - bias - mbits)
        else:
            val = (1.0 + m * 2.0**(-mbits)) * 2.0**(e - bias)
        out[code] = sign * val
    return out


def decode(codes, fmt):
    """uint8 tensor -> float32 tensor (exact)."""
    table = torch.from_numpy(decode_table(fmt))
    return table[codes.to(torch.int64)]


def encode(x, fmt):
    """float32 tensor -> uint8 codes: clamp to +-fp_max (saturate, Inf included), round to
    nearest even; NaN gives sign|0x7F."""
    x = x.to(torch.float32)
    fmax = FP_MAX[fmt]
    y = torch.clamp(x, -fmax, fmax)    # NaN passes through clamp
    return y.to(_TORCH_DT[fmt]).view(torch.uint8)


def encode_bruteforce(x, fmt):
    """Independent encoder: nearest finite code by exhaustive search, ties to the even code.

    Used only to pin ``encode``; O(n*128) so keep n small (<= a few 100k).
    """
    x = np.asarray(x, dtype=np.float64)
    table = decode_table(fmt).astype(np.float64)
    fmax = FP_MAX[fmt]
    pos_codes = np.array([c for c in range(128) if np.isfinite(table[c])], dtype=np.int64)
    pos_vals = table[pos_codes]
    ax = np.minimum(np.abs(x), fmax)
    idx = np.searchsorted(pos_vals, ax, side='left')    # pos_vals[idx-1] < ax <= pos_vals[idx]
    idx = np.clip(idx, 0, len(pos_vals) - 1)
    lo = np.clip(idx - 1, 0, len(pos_vals) - 1)
    d_hi = np.abs(pos_vals[idx] - ax)
    d_lo = np.abs(ax - pos_vals[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (pos_codes[lo] % 2 == 0))
    code = np.where(pick_lo, pos_codes[lo], pos_codes[idx])
    code = np.where(np.isnan(x), 0x7F, code)
    code = code | np.where(np.signbit(x), 0x80, 0)
    return code.astype(np.uint8)
