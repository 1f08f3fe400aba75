"""Adam-flavoured variants of LBAdamW (msamp/optim/adam.py:9-65)."""

from msamp.optim.adamw import LBAdamW


class LBAdam(LBAdamW):
    """Adam: weight decay enters the gradient as an L2 term instead of decaying the weight."""
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False, maximize=False,
                 *args, **kwargs):
        super().__init__(
            params, *args, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad, maximize=maximize,
            **kwargs
        )
        self.use_adam = True


class DSAdam(LBAdamW):
    """LBAdamW with DeepSpeed FusedAdam's constructor flags (adam_w_mode, set_grad_none)."""
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, adam_w_mode=True,
                 weight_decay=0., amsgrad=False, set_grad_none=True, **kwargs):
        super().__init__(
            params, lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay,
            amsgrad=amsgrad, **kwargs
        )
        self.use_adam = not adam_w_mode
        self.set_grad_none = set_grad_none
