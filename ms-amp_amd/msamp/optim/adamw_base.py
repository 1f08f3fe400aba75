"""LBAdamWBase: AdamW on low-bit tensors written with whole-tensor operations -- the semantic
reference for the fused kernels (msamp/optim/adamw_base.py:17-309)."""

import math

import torch

from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingTensor
from msamp.optim.optimizer import LBOptimizer


class LBAdamWBase(LBOptimizer):
    """AdamW (decoupled weight decay; L2 when `use_adam`) with selectable moment dtypes.

    exp_avg_dtype / exp_avg_sq_dtype: torch.float32 keeps plain tensors; torch.uint8 (E4M3),
    torch.int8 (E5M2) or torch.float16 make the moment a ScalingTensor with a per-tensor scale.
    """
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2,
                 amsgrad=False, *, maximize=False, exp_avg_dtype=torch.uint8, exp_avg_sq_dtype=torch.float16):
        if not 0.0 <= lr:
            raise ValueError('Invalid learning rate: {}'.format(lr))
        if not 0.0 <= eps:
            raise ValueError('Invalid epsilon value: {}'.format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError('Invalid beta parameter at index 0: {}'.format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError('Invalid beta parameter at index 1: {}'.format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError('Invalid weight_decay value: {}'.format(weight_decay))
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad, maximize=maximize)
        self.bias_correction = bias_correction
        self.exp_avg_dtype = exp_avg_dtype
        self.exp_avg_sq_dtype = exp_avg_sq_dtype
        self.use_adam = False
        super().__init__(params, defaults)

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('amsgrad', False)
            group.setdefault('maximize', False)

    def _get_state_tensor(self, state, dtype):
        """A fresh float32 zero state, quantized to `dtype` unless that is float32."""
        if dtype == torch.float32:
            return state
        if dtype not in (torch.uint8, torch.int8, torch.float16):
            raise TypeError('Unsupported dtype: {}'.format(dtype))
        return state.cast(Dtypes.dtype_to_qtype[dtype])

    def _update_lp_tensor(self, lp, hp):
        if lp is hp:
            return
        if isinstance(lp, ScalingTensor):
            lp.copy_(hp.cast(lp.qtype))
        else:
            lp.copy_(hp)

    @torch.no_grad()
    def lb_step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, steps = [], [], [], [], [], []
            amsgrad = group['amsgrad']
            beta1, beta2 = group['betas']
            for p in group['params']:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError('AdamW does not support sparse gradients')
                params.append(p)
                grads.append(p.grad)
                state = self.state[p]
                if len(state) == 0:
                    state['step'] = 0
                    zeros = lambda: torch.zeros_like(p, memory_format=torch.preserve_format, dtype=torch.float32)    # noqa: E731
                    state['exp_avg'] = self._get_state_tensor(zeros(), self.exp_avg_dtype)
                    state['exp_avg_sq'] = self._get_state_tensor(zeros(), self.exp_avg_sq_dtype)
                    if amsgrad:
                        state['max_exp_avg_sq'] = self._get_state_tensor(zeros(), self.exp_avg_sq_dtype)
                exp_avgs.append(state['exp_avg'])
                exp_avg_sqs.append(state['exp_avg_sq'])
                if amsgrad:
                    max_exp_avg_sqs.append(state['max_exp_avg_sq'])
                state['step'] += 1
                steps.append(state['step'])
            self.adamw_fn(
                params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, steps, amsgrad=amsgrad, beta1=beta1, beta2=beta2,
                lr=group['lr'], weight_decay=group['weight_decay'], eps=group['eps'], maximize=group['maximize']
            )
        return loss

    def adamw_fn(self, params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, *, amsgrad, beta1, beta2, lr,
                 weight_decay, eps, maximize):
        """Dequantize everything to float32, take the AdamW step, requantize param and both moments."""
        if amsgrad:
            raise ValueError('Only amsgrad=False is supported for now.')
        for i, param_lp in enumerate(params):
            grad = grads[i].float()
            if maximize:
                grad = -grad
            param = param_lp.float()
            if weight_decay != 0:
                if self.use_adam:
                    grad = grad.add(param, alpha=weight_decay)
                else:
                    param.mul_(1 - lr * weight_decay)
            exp_avg = exp_avgs[i].float()
            exp_avg_sq = exp_avg_sqs[i].float()
            step = state_steps[i]
            bc1 = 1 - beta1**step if self.bias_correction else 1.0
            bc2 = 1 - beta2**step if self.bias_correction else 1.0
            exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
            exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
            denom = (exp_avg_sq.sqrt() / math.sqrt(bc2)).add_(eps)
            param.addcdiv_(exp_avg, denom, value=-(lr / bc1))
            self._update_lp_tensor(param_lp, param)
            self._update_lp_tensor(exp_avgs[i], exp_avg)
            self._update_lp_tensor(exp_avg_sqs[i], exp_avg_sq)
