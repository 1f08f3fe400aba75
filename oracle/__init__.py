"""CPU oracle for the FP8 hot path: TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A plain PyTorch-CPU / numpy restatement of the reference's scaling, cast, GEMM and
AdamW arithmetic.  Only tests, the smoke check and the benchmark's CPU-baseline leg
may import it; the product package never does.

Pinning status of each function (what fixes its output besides its own formula):

* ``fp8.decode_table`` / ``fp8.encode``: OCP 8-bit float closed form over all 256
  codes, brute-force nearest-code search with ties-to-even over every fp16/bf16 bit
  pattern, torch's float8 dtypes as a library cross-check, and the reference's byte
  vectors (tests/operators/test_dist.py:112-116).
* ``scaling.compute_scaling_factor``: reference known answers
  (tests/common/tensor/test_meta.py:19-38), the closed form
  ``2**floor(log2(fp_max/amax))``, the invariant ``sf*amax <= fp_max < 2*sf*amax`` and
  the special-value table read from msamp/common/tensor/meta.py:51-56.
* ``scaling.update_scaling_factors``: the window sequence of
  tests/optim/test_adamw.py:203-220.
* ``arithmetic.add_to_fp8``: the identity the reference's test demands
  (tests/operators/test_arithmetic.py:25-42: equal to dequantize, add, in-time cast) and a
  hand-worked case.
* ``bucket.quantize_bucket``: a composition of the pinned pieces above (amax, scale rule,
  encode) in the order of msamp/nn/distributed.py:143-184, plus what the composition must
  satisfy: an exact pre-scale for world sizes that are powers of four, the gradient back
  to half a code step after dequantizing and multiplying by the world size, and a sum of
  ``world`` identical buckets that stays inside the format.
* ``gemm.fp8_gemm``: definition (fp32 matmul of dequantized operands) and the exact
  case of tests/operators/test_gemm.py:45-56.
* ``adamw.*``: textbook AdamW against ``torch.optim.AdamW`` to the reference's own
  tolerance (tests/optim/test_adamw.py:49-85) and the half-ulp requantization
  invariant.
* parity unpinned: the byte produced for NaN inputs by the E5M2 cast and the
  NaN-skipping amax of the delayed-scaling cast kernel live in TransformerEngine v1.1
  (not in the reference tree); the oracle follows torch's float8 conversion
  (sign | 0x7F) and CUDA fmaxf semantics there.
"""
