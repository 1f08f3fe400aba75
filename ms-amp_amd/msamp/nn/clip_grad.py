"""Gradient-norm clipping over mixed torch.Tensor / ScalingTensor gradients (msamp/nn/clip_grad.py:11-88)."""

import torch

from msamp import _backend
from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingTensor


def _fused_fp8_norms(grads, norm_type):
    """Norms of the FP8 ScalingTensor gradients among `grads`, straight from their codes (one pass at a byte per
    element instead of dequantizing each to float32 first); None for the others."""
    norms = [None] * len(grads)
    if norm_type not in (1.0, 2.0, float('inf')):
        return norms
    by_qtype = {}
    for i, g in enumerate(grads):
        if isinstance(g, ScalingTensor) and Dtypes.is_fp8_qtype(g.qtype) and g.is_cuda and g.value.is_contiguous():
            by_qtype.setdefault(g.qtype, []).append(i)
    for qtype, idx in by_qtype.items():
        out = _backend.fp8_norms([grads[i].value for i in idx], [grads[i].meta.scale_inv for i in idx], int(qtype), norm_type)
        for k, i in enumerate(idx):
            norms[i] = out[k]
    return norms


def _compute_total_norm(parameters, norm_type=2.0):
    grads = [p.grad for p in parameters if p.grad is not None]
    if not grads:
        return torch.tensor(0.)
    device = grads[0].device
    norm_type = float(norm_type)
    norms = _fused_fp8_norms(grads, norm_type)
    for i, g in enumerate(grads):
        if norms[i] is None:
            g32 = g.to(torch.float32).detach()
            norms[i] = (g32.abs().max() if norm_type == float('inf') else torch.norm(g32, norm_type)).to(device)
    if norm_type == float('inf'):
        return norms[0] if len(norms) == 1 else torch.max(torch.stack(norms))
    return torch.norm(torch.stack(norms), norm_type)


def clip_grad_norm_(parameters, max_norm, norm_type=2.0, error_if_nonfinite=False):
    """Clip the global gradient norm in place and return it.  ScalingTensor gradients are dequantized
    for the norm and clipped by scaling their scale_inv (no pass over the payload)."""
    if isinstance(parameters, (torch.Tensor, ScalingTensor)):
        parameters = [parameters]
    else:
        parameters = list(parameters)
    total_norm = _compute_total_norm(parameters, norm_type=norm_type)
    if error_if_nonfinite and torch.logical_or(total_norm.isnan(), total_norm.isinf()):
        raise RuntimeError(
            f'The total norm of order {norm_type} for gradients from `parameters` is non-finite, so it cannot be '
            'clipped. To disable this error and scale the gradients by the non-finite norm anyway, set '
            '`error_if_nonfinite=False`'
        )
    max_norm = float(max_norm)
    if max_norm > 0:
        coef = torch.clamp(max_norm / (total_norm + 1e-6), max=1.0)
        if coef.item() < 1.0:
            for p in parameters:
                if p.grad is not None:
                    p.grad.detach().mul_(coef)
    return total_norm
