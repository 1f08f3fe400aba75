"""Largest finite value of each floating-point format (msamp/common/dtype/floating.py:17-53)."""

import torch

from msamp.common.dtype.dtypes import Dtypes


class Floating:
    """fp_max tables keyed by torch dtype and by QType."""
    fp_maxs: dict = {}
    qfp_max: dict = {}

    @staticmethod
    def _get_fp_max(exp, man, inf_existed=True):
        """Maximum finite value of a binary float with `exp` exponent and `man` mantissa bits.

        With infinities the top exponent is reserved; without them (E4M3FN) only the all-ones
        mantissa of the top exponent is (NaN).
        """
        bias = 2**(exp - 1) - 1
        if inf_existed:
            top_exp = (2**exp - 2) - bias
            mant = 2.0 - 2.0**(-man)
        else:
            top_exp = (2**exp - 1) - bias
            mant = 2.0 - 2.0**(1 - man)
        return float(mant * 2.0**top_exp)


_E4M3 = Floating._get_fp_max(4, 3, inf_existed=False)
_E5M2 = Floating._get_fp_max(5, 2)
_F16 = Floating._get_fp_max(5, 10)
_BF16 = Floating._get_fp_max(8, 7)
_F32 = Floating._get_fp_max(8, 23)

Floating.fp_maxs = {
    torch.fp8e4m3: _E4M3,
    torch.fp8e5m2: _E5M2,
    torch.float16: _F16,
    torch.bfloat16: _BF16,
    torch.float32: _F32,
}
Floating.qfp_max = {
    Dtypes.kfloat8_e4m3: _E4M3,
    Dtypes.kfloat8_e5m2: _E5M2,
    Dtypes.kfloat16: _F16,
    Dtypes.kbfloat16: _BF16,
    Dtypes.kfloat32: _F32,
}
