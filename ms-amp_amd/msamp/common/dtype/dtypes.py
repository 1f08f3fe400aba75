"""Data-type vocabulary of the FP8 path.

Mirrors msamp/common/dtype/dtypes.py:9-80 of the reference: FP8 payloads are stored in uint8
tensors whatever the format, ``torch.fp8e4m3`` / ``torch.fp8e5m2`` are aliases used as dictionary
keys, and QType values are the codes the native library understands.
"""

from dataclasses import dataclass

import torch

if not hasattr(torch, 'fp8e4m3'):
    torch.fp8e4m3 = torch.uint8
if not hasattr(torch, 'fp8e5m2'):
    torch.fp8e5m2 = torch.int8


@dataclass
class QType:
    """A named quantization type with the integer code used across the C ABI."""
    name: str
    value: int

    def __int__(self):
        return self.value

    def __hash__(self):
        return self.value


class Dtypes:
    """Static maps between torch dtypes and QTypes."""
    kbyte = QType('kByte', 0)
    kint32 = QType('kInt32', 1)
    kfloat32 = QType('kFloat32', 2)
    kfloat16 = QType('kFloat16', 3)
    kbfloat16 = QType('kBFloat16', 4)
    kfloat8_e4m3 = QType('kFloat8E4M3', 5)
    kfloat8_e5m2 = QType('kFloat8E5M2', 6)

    dtype_to_qtype = {
        torch.float16: kfloat16,
        torch.bfloat16: kbfloat16,
        torch.float32: kfloat32,
        torch.fp8e4m3: kfloat8_e4m3,
        torch.fp8e5m2: kfloat8_e5m2,
    }
    qtype_to_dtype = {q: d for d, q in dtype_to_qtype.items()}

    dtype_to_size = {
        torch.float32: 4,
        torch.float16: 2,
        torch.bfloat16: 2,
        torch.uint8: 1,
        torch.int8: 1,
        torch.int64: 8,
        torch.int32: 4,
    }

    @classmethod
    def is_fp8_qtype(cls, qtype):
        return qtype in (cls.kfloat8_e4m3, cls.kfloat8_e5m2)

    @classmethod
    def get_dtype_from_qtype(cls, qtype):
        """Storage dtype of a qtype: uint8 for both FP8 formats."""
        return torch.uint8 if cls.is_fp8_qtype(qtype) else cls.qtype_to_dtype[qtype]
