"""The five native FP8 calls of the hot path under the names the reference gives them
(msamp/common/utils/transformer_engine_wrapper.py:63-176), served by the HIP library instead of
TransformerEngine.  The kernels handle ragged shapes themselves, so nothing is padded here;
PaddingTensor remains for callers that want the 16-element padding explicitly."""

import torch
import torch.nn.functional as F

from msamp import _backend


class PaddingTensor:
    """Context manager that pads a 2-D tensor to multiples of `pad_base` and slices it back on exit."""
    def __init__(self, val, transpose=False, pad_base=16):
        assert val.dim() == 2, 'Input must have 2 dimensions.'
        self.val = val
        self.dim = val.shape
        self.transpose = transpose
        self.pad = [-d % pad_base for d in self.dim]
        self.require_pad = any(p > 0 for p in self.pad)

    def __enter__(self):
        if self.require_pad:
            self.val = F.pad(self.val, (0, self.pad[1], 0, self.pad[0]))
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        if self.require_pad:
            rows, cols = (self.dim[1], self.dim[0]) if self.transpose else (self.dim[0], self.dim[1])
            self.val = self.val[:rows, :cols]
        return None


class TransformerEngineWrapper:
    """Static wrappers; qtype arguments are msamp QTypes."""
    @staticmethod
    def cast_to_fp8(input, scale, amax, scale_inv, otype):
        """Quantize with `scale`; amax (1-element) is atomically maxed with max|input|, scale_inv = 1/scale."""
        return _backend.cast_to_fp8(input, scale, amax, scale_inv, int(otype))

    @staticmethod
    def cast_from_fp8(input, scale_inv, itype, otype):
        from msamp.common.dtype import Dtypes
        return _backend.cast_from_fp8(input, scale_inv, int(itype), Dtypes.get_dtype_from_qtype(otype))

    @staticmethod
    def fp8_fused_cast_transpose(input, qtype, meta):
        """(cast, cast^T) of a 2-D tensor with the meta's stored scale."""
        return _backend.cast_transpose(input, meta.scale, meta.amax[0:1], meta.scale_inv, int(qtype))

    @staticmethod
    def fp8_transpose(input):
        return input.fp8_transpose()

    @staticmethod
    def te_gemm(mat_a, a_scale_inv, a_qtype, transa, mat_b, b_scale_inv, b_qtype, transb, out, out_scale, out_qtype,
                out_amax, bias, bias_qtype, pre_gelu_out, grad, workspace, workspace_size, accumulate,
                use_split_accumulator, math_sm_count=0):
        """out[N,M] (+)= (mat_b[N,K] . mat_a[M,K]^T) * a_scale_inv * b_scale_inv (+ bias); only the
        TN form the FP8 path uses (transa=True, transb=False) exists."""
        if not transa or transb:
            raise ValueError('only the TN form (transa=True, transb=False) is implemented')
        b = bias if (bias is not None and bias.numel() > 0) else None
        return _backend.fp8_gemm(mat_a, int(a_qtype), a_scale_inv, mat_b, int(b_qtype), b_scale_inv, out, accumulate, b)


__all__ = ['TransformerEngineWrapper', 'PaddingTensor', 'torch']
