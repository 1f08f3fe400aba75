"""Arithmetic.add_to_fp8 (msamp/operators/arithmetic/arithmetic.py:12-35) on the HIP library."""

import torch

from msamp import _backend
from msamp.common.dtype import Dtypes


class Arithmetic:
    """Arithmetic operator for FP8 tensors."""
    @staticmethod
    def add_to_fp8(fp8_tensor, meta, other):
        """Add the high-precision tensor `other` to `fp8_tensor` in place.

        The FP8 payload is dequantized to other's dtype, the sum is formed in that dtype, and the result is
        requantized with in-time scaling: meta.amax[0], meta.scale and meta.scale_inv are replaced.  Bit for bit
        what `(scaling_tensor.to(dtype) + other).cast(qtype, meta=meta)` gives.

        Args:
            fp8_tensor (torch.Tensor): uint8 / int8 FP8 payload to add to.
            meta (ScalingMeta): its meta.
            other (torch.Tensor): fp32 / fp16 / bf16 tensor with the same number of elements.
        """
        if not (fp8_tensor.is_cuda and fp8_tensor.is_contiguous()):
            raise ValueError('The fp8 tensor is not in cuda memory or contiguous.')
        if not (other.is_cuda and other.is_contiguous()):
            raise ValueError('The other tensor is not in cuda memory or contiguous.')
        if fp8_tensor.dtype not in (torch.uint8, torch.int8):
            raise ValueError('The fp8 tensor is not in uint8 or int8.')
        if meta.qtype not in (Dtypes.kfloat8_e4m3, Dtypes.kfloat8_e5m2):
            raise ValueError('The fp8 tensor is not in e4m3 or e5m2 format.')
        if fp8_tensor.numel() != other.numel():
            raise ValueError('The fp8 tensor and the other tensor differ in size.')
        _backend.add_to_fp8(fp8_tensor, int(meta.qtype), meta.scale, meta.scale_inv, meta.amax[0:1], other)
