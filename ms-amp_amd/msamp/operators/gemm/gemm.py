"""Gemm.fp8_gemm (msamp/operators/gemm/gemm.py:58-179) on the gfx950 FP8 MFMA kernel."""

import torch
import torch.nn.functional as F

from msamp import _backend
from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingTensor


class Gemm:
    """FP8 GEMM entry point."""
    _te_base = 16

    @staticmethod
    def _round2times(value, base):
        """Smallest multiple of base that is >= value."""
        return (value + base - 1) // base * base

    @staticmethod
    def _aligned(payload):
        """The kernels fetch operands 16 bytes at a time.  A payload that starts elsewhere (a view into a flat buffer
        at an odd offset) is copied to a fresh allocation first, as the reference pads and copies what its library
        cannot take (msamp/operators/gemm/gemm.py:107-121)."""
        return payload if payload.data_ptr() % 16 == 0 else payload.clone()

    @classmethod
    def kmajor_supported(cls, m, n, k, a_kmajor=True, b_kmajor=False):
        """True if fp8_gemm reads K-major operands of this problem in place (else it transposes them first)."""
        return _backend.gemm_kmajor_supported(m, n, k, a_kmajor, b_kmajor)

    @classmethod
    @torch.no_grad()
    def fp8_gemm_cast(cls, mat_a, mat_b, out_qtype, meta, sync=False, a_kmajor=False, b_kmajor=False, accumulate=False,
                      out=None):
        """fp8_gemm(mat_a, mat_b, out_qtype, accumulate=accumulate, out=out).cast(meta.qtype, meta=meta, sync=sync) for a
        meta with in-time scaling, without reading the product back (not in the reference, which takes the two steps:
        nn/functional.py:100-123).  Small products take one launch and are never stored; larger ones are stored in
        `out` (a scratch tensor if not given) next to the codes for the scale the meta holds, and are read again only
        when the scale rule moves the scale.  Returns the FP8 ScalingTensor, or None if the kernel does not take this
        problem -- the caller then takes the two steps itself; the result is the same bit for bit."""
        assert isinstance(mat_a, ScalingTensor) and isinstance(mat_b, ScalingTensor)
        assert mat_a.is_cuda and mat_a.is_contiguous() and mat_b.is_cuda and mat_b.is_contiguous()
        assert Dtypes.is_fp8_qtype(mat_a.qtype) and Dtypes.is_fp8_qtype(mat_b.qtype) and Dtypes.is_fp8_qtype(meta.qtype)
        if meta.scaling_mode() != 'in_time' or (a_kmajor != b_kmajor):
            return None
        out_dtype = Dtypes.get_dtype_from_qtype(out_qtype)
        if out is not None:
            assert out.is_cuda and out.is_contiguous() and out.dtype == out_dtype
        else:
            assert not accumulate, 'accumulate needs an output tensor'
        payload = _backend.fp8_gemm_cast(
            cls._aligned(mat_a.value), int(mat_a.qtype), mat_a.meta.scale_inv, cls._aligned(mat_b.value), int(mat_b.qtype),
            mat_b.meta.scale_inv, out_dtype, int(meta.qtype), meta.scale, meta.amax[0:1], meta.scale_inv,
            nan_to_inf=sync, a_kmajor=a_kmajor, b_kmajor=b_kmajor, hp_out=out, accumulate=accumulate
        )
        return None if payload is None else ScalingTensor(payload, meta)

    @classmethod
    @torch.no_grad()
    def fp8_gemm(
        cls, mat_a, mat_b, out_qtype, bias=None, accumulate=False, out=None, use_split_accumulator=False, a_kmajor=False,
        b_kmajor=False
    ):
        """out[N, M] = (mat_b[N, K] @ mat_a[M, K].T) * a.scale_inv * b.scale_inv.

        mat_a, mat_b: contiguous FP8 ScalingTensors on the GPU.  The kernel accumulates in fp32
        over the full K (use_split_accumulator has nothing to switch) and writes out_qtype; with
        `accumulate` it adds into `out`.  Only K needs padding (to a multiple of 16 bytes, with
        FP8 zeros); ragged M and N are handled inside the kernel.

        a_kmajor / b_kmajor (not in the reference): the tensor passed is the transpose of the operand,
        [K, M] / [K, N], as the backward pass of a linear layer has them; the kernel reads it in place
        when the shape allows, otherwise it is transposed first.  Same result either way.
        """
        assert isinstance(mat_a, ScalingTensor)
        assert isinstance(mat_b, ScalingTensor)
        assert mat_a.is_cuda and mat_a.is_contiguous()
        assert mat_b.is_cuda and mat_b.is_contiguous()
        assert Dtypes.is_fp8_qtype(mat_a.qtype) and Dtypes.is_fp8_qtype(mat_b.qtype)

        if a_kmajor or b_kmajor:
            K, M = mat_a.shape if a_kmajor else mat_a.shape[::-1]
            N = mat_b.shape[1] if b_kmajor else mat_b.shape[0]
            if cls.kmajor_supported(M, N, K, a_kmajor, b_kmajor):
                out_dtype = Dtypes.get_dtype_from_qtype(out_qtype)
                if out is None:
                    assert not accumulate, 'accumulate needs an output tensor'
                    out = torch.empty(N, M, dtype=out_dtype, device=mat_a.device)
                else:
                    assert out.is_cuda and out.is_contiguous() and out.dtype == out_dtype
                _backend.fp8_gemm(
                    cls._aligned(mat_a.value), int(mat_a.qtype), mat_a.meta.scale_inv, cls._aligned(mat_b.value),
                    int(mat_b.qtype), mat_b.meta.scale_inv, out, accumulate, bias, a_kmajor=a_kmajor, b_kmajor=b_kmajor
                )
                return out
            if a_kmajor:
                mat_a = mat_a.fp8_transpose()
            if b_kmajor:
                mat_b = mat_b.fp8_transpose()

        M, K = mat_a.shape
        N = len(mat_b)
        a, b = cls._aligned(mat_a.value), cls._aligned(mat_b.value)
        pK = cls._round2times(K, cls._te_base) - K
        if pK > 0:
            a = F.pad(a, (0, pK))
            b = F.pad(b, (0, pK))
        out_dtype = Dtypes.get_dtype_from_qtype(out_qtype)
        if out is None:
            assert not accumulate, 'accumulate needs an output tensor'
            out = torch.empty(N, M, dtype=out_dtype, device=a.device)
        else:
            assert out.is_cuda and out.is_contiguous() and out.dtype == out_dtype
        _backend.fp8_gemm(
            a, int(mat_a.qtype), mat_a.meta.scale_inv, b, int(mat_b.qtype), mat_b.meta.scale_inv, out, accumulate, bias
        )
        return out
