"""FP8Linear and the nn.Linear -> FP8Linear replacer (msamp/nn/linear.py:14-197)."""

import torch
import torch.nn.functional as F

from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingTensor, ScalingMeta
from msamp.nn.module import ScalingModule
from msamp.nn.parameter import ScalingParameter
from msamp.nn.state import model_state


class FP8Linear(ScalingModule):
    """Linear layer whose weight is a ScalingParameter and whose GEMMs run in FP8.

    Three metas drive the casts: `input` (E4M3) and `ograd` (E5M2) use delayed scaling over a
    16-step amax window; `wgrad` (E4M3) has window 1, i.e. always in-time scaling.
    """
    DEFAULT_WINDOW_SIZE = 16
    DEFAULT_WGRAD_WINDOW_SIZE = 1

    def __init__(self, in_features, out_features, use_bias=True, weight_qtype=Dtypes.kfloat16, bias_type=torch.float32):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight_qtye = weight_qtype
        self.weight_qtype = weight_qtype
        dev = 'cuda' if torch.cuda.is_available() else 'cpu'
        payload = torch.empty((out_features, in_features), dtype=Dtypes.get_dtype_from_qtype(weight_qtype))
        meta = ScalingMeta(weight_qtype, window_size=1, device=dev)
        self.weight = ScalingParameter(ScalingTensor(payload, meta=meta))
        if use_bias:
            self.bias = torch.nn.Parameter(torch.empty(out_features, dtype=bias_type))
        else:
            self.register_parameter('bias', None)
        self.scaling_metas = dict(
            input=ScalingMeta(Dtypes.kfloat8_e4m3, window_size=FP8Linear.DEFAULT_WINDOW_SIZE, device=dev),
            wgrad=ScalingMeta(Dtypes.kfloat8_e4m3, window_size=FP8Linear.DEFAULT_WGRAD_WINDOW_SIZE, device=dev),
            ograd=ScalingMeta(Dtypes.kfloat8_e5m2, window_size=FP8Linear.DEFAULT_WINDOW_SIZE, device=dev),
        )
        self.weight._scaling_metas = self.scaling_metas

    def forward(self, input):
        return F.linear(input, self.weight, bias=self.bias)

    def extra_repr(self):
        return f'in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}'


class LinearReplacer:
    """Swaps every nn.Linear of a model for an FP8Linear holding the same (quantized) weight."""
    @staticmethod
    @torch.no_grad()
    def _build_fp8linear(linear, weight_qtype):
        if not isinstance(linear, torch.nn.Linear):
            raise TypeError('type of m must be torch.nn.Linear')
        has_bias = linear.bias is not None
        fp8_linear = FP8Linear(
            linear.in_features, linear.out_features, use_bias=has_bias, weight_qtype=weight_qtype,
            bias_type=linear.bias.dtype if has_bias else torch.float32
        ).cuda()
        linear = linear.cuda()
        if has_bias:
            fp8_linear.bias.data.copy_(linear.bias)
        weight = linear.weight.cast(weight_qtype)
        if fp8_linear.weight.dtype != weight.dtype:
            raise ValueError(
                f'weight dtype is not same, dtype ins fp8 linear is {fp8_linear.weight.dtype}, dtype in weight is {weight.dtype}'
            )
        fp8_linear.weight.copy_(weight)

        # carry user-defined attributes over (module, weight, bias)
        pairs = [(fp8_linear, linear), (fp8_linear.weight, linear.weight)]
        if has_bias:
            pairs.append((fp8_linear.bias, linear.bias))
        for new, old in pairs:
            _, custom = LinearReplacer._compare_attrs(type(old), old)
            for attr in custom:
                if not hasattr(new, attr):
                    setattr(new, attr, getattr(old, attr))
        return fp8_linear

    @staticmethod
    def _compare_attrs(x, y):
        """(names only x has, names only y has)."""
        xs, ys = set(dir(x)), set(dir(y))
        return xs - ys, ys - xs

    @classmethod
    def _replace(cls, model, weight_qtype):
        if isinstance(model, torch.nn.Linear):
            if getattr(model, 'use_fp32_linear', False):
                return model
            return cls._build_fp8linear(model, weight_qtype)
        for name, child in list(model.named_children()):
            setattr(model, name, cls._replace(child, weight_qtype))
        return model

    @classmethod
    def replace(cls, model, weight_qtype=Dtypes.kfloat16, src_rank=0, group=None):
        """Replace the Linear layers, name the FP8 weights, hide them from DistributedDataParallel and
        register the layers' metas with the model state.  (Weight broadcast over a process group is a
        multi-GPU step and is not part of this build.)"""
        model = cls._replace(model, weight_qtype)
        fp8_names = []
        for name, p in model.named_parameters():
            if isinstance(p, ScalingParameter):
                p._param_name = name
                fp8_names.append(name)
        torch.nn.parallel.DistributedDataParallel._set_params_and_buffers_to_ignore_for_model(model, fp8_names)
        model_state.register_scaling_metas(model, group)
        return model
