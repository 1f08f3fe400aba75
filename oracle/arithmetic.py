"""CPU restatement of Arithmetic.add_to_fp8 -- test infrastructure only.

The reference defines the operation by an identity its own test demands bit for bit
(tests/operators/test_arithmetic.py:25-42): after `Arithmetic.add_to_fp8(t.value, t.meta, other)` the tensor
equals `(t.to(dtype) + other).cast(qtype, meta=t.meta)`.  The kernel (msamp/operators/arithmetic/
vectorized_pointwise.h:184-301) is that identity fused: dequantize into other's dtype, add in that dtype, take
max|sum| as the new amax[0], derive the scale with the pow-2 rule (fallback: the old scale), requantize.
Pinned by: that identity (composition of the already pinned dequantize and in-time cast) and a hand-worked case in
tests/test_oracle_arithmetic.py.
"""

import torch

from oracle import cast as ocast


def add_to_fp8(q, meta, fmt, other):
    """Returns the new payload; `meta` (dict scale / scale_inv / amax) is updated in place."""
    t = ocast.cast_from_fp8(q, meta['scale_inv'], fmt, out_dtype=other.dtype) + other
    return ocast.cast_to_fp8(t, meta, fmt, in_time=True)
