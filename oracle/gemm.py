"""FP8 GEMM definition.  Test infrastructure only."""

import torch

from . import fp8


def fp8_gemm(a_q, a_scale_inv, a_fmt, b_q, b_scale_inv, b_fmt, out_dtype=torch.float32, bias=None, out=None):
    """out[N,M] = (B[N,K] . A[M,K]^T) * a_scale_inv * b_scale_inv (+ bias[M]) (+ out);
    follows msamp/operators/gemm/gemm.py:88-144 with an fp32 matmul on the dequantized operands."""
    a = fp8.decode(a_q, a_fmt) * a_scale_inv.to(torch.float32)
    b = fp8.decode(b_q, b_fmt) * b_scale_inv.to(torch.float32)
    d = b.double() @ a.double().t()
    if bias is not None:
        d = d + bias.double().view(1, -1)
    if out is not None:
        d = d + out.double()
    return d.to(torch.float32).to(out_dtype)
