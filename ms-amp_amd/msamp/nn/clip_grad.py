"""Gradient-norm clipping over mixed torch.Tensor / ScalingTensor gradients (msamp/nn/clip_grad.py:11-88)."""

import torch

from msamp.common.tensor import ScalingTensor


def _compute_total_norm(parameters, norm_type=2.0):
    grads = [p.grad for p in parameters if p.grad is not None]
    if not grads:
        return torch.tensor(0.)
    device = grads[0].device
    norm_type = float(norm_type)
    as_f32 = [g.to(torch.float32).detach() for g in grads]
    if norm_type == float('inf'):
        norms = [g.abs().max().to(device) for g in as_f32]
        return norms[0] if len(norms) == 1 else torch.max(torch.stack(norms))
    return torch.norm(torch.stack([torch.norm(g, norm_type).to(device) for g in as_f32]), norm_type)


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
