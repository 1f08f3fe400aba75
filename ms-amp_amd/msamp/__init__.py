"""MS-AMP API on the MI355X FP8 kernels: msamp.initialize and msamp.clip_grad_norm_
(msamp/__init__.py:17-100 of the reference)."""

import torch

from msamp.nn import clip_grad_norm_
from msamp.nn import LinearReplacer
from msamp.optim import LBAdam, LBAdamW, DSAdam

try:    # optional: DeepSpeed's FusedAdam is accepted as an input optimizer when DeepSpeed is installed
    from deepspeed.ops.adam import FusedAdam as _FusedAdam
except Exception:    # pragma: no cover
    _FusedAdam = None

opt_levels = ['O1', 'O2']


def initialize(model, optimizer=None, opt_level='O1', use_te=False):
    """Cast a model and its Adam/AdamW optimizer to the FP8 path.

    Every nn.Linear becomes an FP8Linear (FP8 GEMMs, scaled-fp16 weight, FP8 weight gradient) and
    the optimizer is rebuilt as LBAdam/LBAdamW/DSAdam over the new parameters, keeping the order
    and grouping of the original one.  O1 keeps float32 moments; O2 stores exp_avg in E4M3 and
    exp_avg_sq in scaled fp16.  Returns (model, optimizer).
    """
    if not isinstance(model, torch.nn.Module):
        raise ValueError('Model must be an instance of torch.nn.Module')
    if opt_level not in opt_levels:
        raise ValueError('Invalid optimization level. Please choose from {}'.format(opt_levels))
    if use_te:
        raise ValueError('use_te=True needs NVIDIA TransformerEngine, which this build does not use')
    if not optimizer:
        optimizer = torch.optim.AdamW(model.parameters())
    accepted = (torch.optim.AdamW, torch.optim.Adam) + ((_FusedAdam, ) if _FusedAdam is not None else ())
    if not isinstance(optimizer, accepted):
        raise ValueError('Optimizer {} is not supported in optimization level {}'.format(optimizer, opt_level))

    # position of every optimizer parameter in model.parameters() order; the replaced model keeps that order
    position = {id(p): i for i, p in enumerate(model.parameters())}
    order = []
    for group in optimizer.param_groups:
        for p in group['params']:
            assert id(p) in position
            order.append(position[id(p)])

    cast_model = LinearReplacer.replace(model)

    new_params = list(cast_model.parameters())
    cursor = 0
    for group in optimizer.param_groups:
        for i in range(len(group['params'])):
            group['params'][i] = new_params[order[cursor]]
            cursor += 1

    args = optimizer.defaults
    args['exp_avg_dtype'] = torch.uint8 if opt_level == 'O2' else torch.float32
    args['exp_avg_sq_dtype'] = torch.float16 if opt_level == 'O2' else torch.float32
    for k in ('foreach', 'capturable', 'differentiable', 'fused', 'decoupled_weight_decay'):
        args.pop(k, None)

    # torch.optim.AdamW subclasses Adam in recent torch, so test the subclass first
    if isinstance(optimizer, torch.optim.AdamW):
        cast_optimizer = LBAdamW(optimizer.param_groups, **args)
    elif isinstance(optimizer, torch.optim.Adam):
        cast_optimizer = LBAdam(optimizer.param_groups, **args)
    else:
        cast_optimizer = DSAdam(optimizer.param_groups, **args, adam_w_mode=optimizer.adam_w_mode)
    return cast_model, cast_optimizer


__version__ = '0.4.0'
__author__ = 'Microsoft'
__all__ = ['clip_grad_norm_', 'initialize']
