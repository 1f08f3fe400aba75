"""ScalingModule: nn.Module whose parameter dict may hold ScalingParameters (msamp/nn/module.py:13-93)."""

import torch
from torch import nn
from torch.nn.parameter import Parameter

from msamp.nn.parameter import ScalingParameter


class ScalingModule(nn.Module):
    """Base class of FP8 layers."""
    def __init__(self):
        super().__init__()
        self.scaling_metas = None

    def __setattr__(self, name, value):
        if isinstance(value, ScalingParameter):
            self._parameters[name] = value
        else:
            super().__setattr__(name, value)

    def _apply(self, fn, recurse=True):
        """nn.Module._apply that also carries ScalingParameters through .cuda()/.to(): for those the
        function is applied and the result re-seated through the `.data` setter; dtype conversions
        skip them because they report is_floating_point() == False."""
        if recurse:
            for module in self.children():
                module._apply(fn)

        for key, param in self._parameters.items():
            if param is None:
                continue
            with torch.no_grad():
                applied = fn(param)
            if isinstance(param, ScalingParameter):
                param.data = applied
                if param.grad is not None:
                    with torch.no_grad():
                        param.grad.data = fn(param.grad)
                continue
            use_set_data = (
                torch._has_compatible_shallow_copy_type(param, applied)
                and not torch.__future__.get_overwrite_module_params_on_conversion()
            )
            if use_set_data:
                param.data = applied
                out_param = param
            else:
                out_param = Parameter(applied, param.requires_grad)
                self._parameters[key] = out_param
            if param.grad is not None:
                with torch.no_grad():
                    grad_applied = fn(param.grad)
                if use_set_data:
                    out_param.grad.data = grad_applied
                else:
                    out_param.grad = grad_applied.requires_grad_(param.grad.requires_grad)

        for key, buf in self._buffers.items():
            if buf is not None:
                self._buffers[key] = fn(buf)
        return self
