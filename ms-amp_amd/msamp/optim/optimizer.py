"""LBOptimizer: optimizer base class for low-bit (ScalingTensor) parameters and the per-step update
of the delayed-scaling windows (msamp/optim/optimizer.py:20-285)."""

from collections import defaultdict, abc as container_abcs
from copy import deepcopy
from itertools import chain
import warnings

import torch
from torch.optim.optimizer import Optimizer, required

from msamp import _backend
from msamp.common.dtype import Floating
from msamp.common.tensor import ScalingTensor, ScalingMeta
from msamp.nn import model_state, ScalingParameter


class LBOptimizer(Optimizer):
    """torch.optim.Optimizer whose parameter groups may hold ScalingTensors."""
    def __init__(self, params, defaults):
        super().__init__(params, defaults)
        self.set_grad_none = False

    def step(self, closure=None):
        """One optimization step followed by the scaling-factor update of all FP8 layers."""
        # A bounded wait that ran out inside a cast, GEMM or optimizer kernel of an earlier step surfaces here, before this
        # step changes anything, and without a device-to-host synchronisation (the copy of the error word requested by
        # the previous step is looked at).  What such a kernel wrote is invalid, and so is what was computed from it
        # since: the caller goes back to its last good state.
        _backend.check_async_error(block=False)
        rtn = self.lb_step(closure)
        self._update_scaling_factors()
        return rtn

    def all_reduce_grads(self, model):
        """Average the ScalingTensor gradients of `model`'s parameters over the data-parallel ranks
        (optimizer.py:45-51); skipped when the FP8 DDP wrapper reduces them itself."""
        if model_state.use_fp8_ddp:
            return
        grads = [p.grad for p in model.parameters() if isinstance(p, ScalingParameter) and p.grad is not None]
        self._all_reduce_avg(grads)

    @staticmethod
    def _all_reduce_avg(grads):
        """Nothing to do with one rank (tensor_dist.py:118-120); more ranks are outside this single-GPU build."""
        if torch.distributed.is_available() and torch.distributed.is_initialized() \
                and torch.distributed.get_world_size() > 1:
            raise NotImplementedError('FP8 gradient all-reduce is outside this single-GPU build')

    def lb_step(self, closure=None):
        raise NotImplementedError('lb_step is not implemented')

    def _update_scaling_factors(self, training=True):
        """Once per step, if any FP8 linear ran: for the `input` and `ograd` metas (and `wgrad` when
        in-time scaling is globally off) recompute the scale from the amax window, shift the window and
        count the step; a non-finite current amax is dropped and restarts that meta's warm-up."""
        if not model_state.ready_to_scale_tensor:
            return
        model_state.ready_to_scale_tensor = False
        metas = model_state.flattened_scaling_metas
        if metas is None:
            return
        names = ['input']
        if training:
            names.append('ograd')
            if not ScalingMeta.in_time_scaling:
                names.append('wgrad')
        margin = 0
        if all(metas[name]['amax_counters'].is_cuda for name in names):
            # counters live on the GPU and are updated by the same kernel (no device-to-host copy), and all
            # groups go in one launch
            _backend.scale_update_groups(
                [(metas[n]['scales'], metas[n]['amaxs'], Floating.qfp_max[metas[n]['qtype']], metas[n]['amax_counters'])
                 for n in names], margin
            )
            return
        for name in names:
            meta = metas[name]
            fp_max = Floating.qfp_max[meta['qtype']]
            counters = meta['amax_counters']
            if counters.is_cuda:
                _backend.scale_update(meta['scales'], meta['amaxs'], fp_max, margin, counters=counters, want_mask=False)
            else:
                bad = _backend.scale_update(meta['scales'], meta['amaxs'], fp_max, margin).cpu().bool()
                counters += 1
                counters[bad] = 0

    # ---- state (de)serialisation with order indices instead of tensors ---------------------------
    def state_dict(self):
        """{'state': {index: {...}}, 'param_groups': [...]} with parameters replaced by their order index."""
        mapping = {}
        start = 0

        def pack(group):
            nonlocal start
            packed = {k: v for k, v in group.items() if k != 'params'}
            mapping.update({id(p): i for i, p in enumerate(group['params'], start) if id(p) not in mapping})
            packed['params'] = [mapping[id(p)] for p in group['params']]
            start += len(packed['params'])
            return packed

        groups = [pack(g) for g in self.param_groups]
        state = {(mapping[id(k)] if isinstance(k, (torch.Tensor, ScalingTensor)) else k): v for k, v in self.state.items()}
        return {'state': state, 'param_groups': groups}

    def load_state_dict(self, state_dict):
        """Inverse of state_dict(); state tensors are moved to the parameter's device but keep their dtype."""
        state_dict = deepcopy(state_dict)
        groups, saved_groups = self.param_groups, state_dict['param_groups']
        if len(groups) != len(saved_groups):
            raise ValueError('loaded state dict has a different number of parameter groups')
        if any(len(g['params']) != len(s['params']) for g, s in zip(groups, saved_groups)):
            raise ValueError("loaded state dict contains a parameter group that doesn't match the size of optimizer's group")
        id_map = dict(
            zip(chain.from_iterable(g['params'] for g in saved_groups), chain.from_iterable(g['params'] for g in groups))
        )

        def move(param, value, key=None):
            if isinstance(value, torch.Tensor):
                return value.to(param.device) if key != 'step' else value
            if isinstance(value, ScalingTensor):
                return value
            if isinstance(value, dict):
                return {k: move(param, v, key=k) for k, v in value.items()}
            if isinstance(value, container_abcs.Iterable) and not isinstance(value, str):
                return type(value)(move(param, v) for v in value)
            return value

        state = defaultdict(dict)
        for k, v in state_dict['state'].items():
            if k in id_map:
                state[id_map[k]] = move(id_map[k], v)
            else:
                state[k] = v
        new_groups = []
        for g, ng in zip(groups, saved_groups):
            ng['params'] = g['params']
            new_groups.append(ng)
        self.__setstate__({'state': state, 'param_groups': new_groups})

    def zero_grad(self, set_to_none=None):
        if set_to_none is None:
            set_to_none = self.set_grad_none
        for group in self.param_groups:
            for p in group['params']:
                if p.grad is None:
                    continue
                if set_to_none:
                    p.grad = None
                elif isinstance(p.grad, ScalingTensor):
                    p.grad.zero_()
                else:
                    p.grad.detach_()
                    p.grad.requires_grad_(False)
                    p.grad.zero_()

    def add_param_group(self, param_group):
        """torch's add_param_group, accepting ScalingTensor entries."""
        assert isinstance(param_group, dict), 'param group must be a dict'
        params = param_group['params']
        if isinstance(params, (torch.Tensor, ScalingTensor)):
            param_group['params'] = [params]
        elif isinstance(params, set):
            raise TypeError(
                'optimizer parameters need to be organized in ordered collections, but the ordering of tensors in '
                'sets will change between runs. Please use a list instead.'
            )
        else:
            param_group['params'] = list(params)
        for p in param_group['params']:
            if not isinstance(p, (torch.Tensor, ScalingTensor)):
                raise TypeError('optimizer can only optimize Tensors, but one of the params is ' + torch.typename(p))
            if not self.defaults.get('differentiable', None) and not (p.is_leaf or p.retains_grad):
                raise ValueError("can't optimize a non-leaf Tensor")
        for name, default in self.defaults.items():
            if default is required and name not in param_group:
                raise ValueError("parameter group didn't specify a value of required optimization parameter " + name)
            param_group.setdefault(name, default)
        ids = [id(p) for p in param_group['params']]
        if len(ids) != len(set(ids)):
            warnings.warn('optimizer contains a parameter group with duplicate parameters', stacklevel=3)
        seen = {id(p) for g in self.param_groups for p in g['params']}
        if not seen.isdisjoint(ids):
            raise ValueError('some parameters appear in more than one parameter group')
        self.param_groups.append(param_group)
