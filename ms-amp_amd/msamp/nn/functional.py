"""F.linear with ScalingTensor weights: FP8 forward, dgrad and wgrad (msamp/nn/functional.py:16-194)."""

import torch
import torch.nn.functional as F

from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingTensor
from msamp.operators.gemm import Gemm
from msamp.nn.state import model_state


class _FP8GemmFunction(torch.autograd.Function):
    """y = x W^T (+ bias) with x, W in E4M3; dx = dy W and dW = dy^T x with dy in E5M2; fp32 accumulation.

    The reference adds the bias in a separate elementwise pass after the function (nn/functional.py:184-185); here it
    rides in the epilogue of the forward GEMM (fma(acc, scale, bias), one rounding to the output type instead of
    two) and its gradient, the column sums of dy in the output type, is returned from backward as autograd would
    have formed it."""
    @staticmethod
    def forward(ctx, input, weight, metas, dtype_holder, bias=None):
        ctx.metas = metas
        model_state.check_metas_in_flat(metas)
        input_fp8 = input.cast(Dtypes.kfloat8_e4m3, meta=metas['input'])
        weight_fp8 = weight.cast(Dtypes.kfloat8_e4m3)

        ctx.input_fp8 = input_fp8
        ctx.input_fp8.requires_grad = input.requires_grad
        ctx.weight_fp8 = weight_fp8
        ctx.weight = weight
        ctx.output_dtype = dtype_holder.dtype
        ctx.output_qtype = Dtypes.dtype_to_qtype[dtype_holder.dtype]
        ctx.bias_dtype = None if bias is None else bias.dtype
        ctx.need_bias_grad = bias is not None and bias.requires_grad
        if bias is not None:
            bias = bias.detach().to(ctx.output_dtype).contiguous()
        return Gemm.fp8_gemm(weight_fp8, input_fp8, ctx.output_qtype, bias=bias, use_split_accumulator=False)

    @staticmethod
    def backward(ctx, output_grad):
        output_grad = output_grad.contiguous()
        metas = ctx.metas
        tokens, d_out = output_grad.shape
        d_in = ctx.input_fp8.shape[1]
        need_dgrad, need_wgrad = ctx.input_fp8.requires_grad, ctx.weight.requires_grad
        # The reference materializes dy^T, W^T and x^T (fused cast-transpose + two FP8 transposes) because its
        # GEMM reads K-contiguous operands only.  This kernel also reads [K, rows] operands in place, so when
        # the shapes allow, dy is only cast and W, x, dy go to the GEMMs as they are (same results).
        in_place = (not need_dgrad or Gemm.kmajor_supported(d_in, tokens, d_out, True, False)) and \
            (not need_wgrad or Gemm.kmajor_supported(d_in, d_out, tokens, True, True))
        if in_place:
            ograd_fp8 = output_grad.cast(Dtypes.kfloat8_e5m2, meta=metas['ograd'])
            ograd_fp8_t = None
        else:
            ograd_fp8, ograd_fp8_t = output_grad.fused_cast_transpose(Dtypes.kfloat8_e5m2, meta=metas['ograd'])

        input_grad = None
        if need_dgrad:
            if in_place:
                input_grad = Gemm.fp8_gemm(ctx.weight_fp8, ograd_fp8, ctx.output_qtype, use_split_accumulator=True, a_kmajor=True)
            else:
                weight_fp8_t = ctx.weight_fp8.fp8_transpose()
                input_grad = Gemm.fp8_gemm(weight_fp8_t, ograd_fp8, ctx.output_qtype, use_split_accumulator=True)

        if need_wgrad:
            if in_place:
                mat_a, mat_b, layout = ctx.input_fp8, ograd_fp8, dict(a_kmajor=True, b_kmajor=True)
            else:
                mat_a, mat_b, layout = ctx.input_fp8.fp8_transpose(), ograd_fp8_t, {}
            wgrad = None
            old_wgrad = None
            if ctx.weight.grad is not None:
                # gradient accumulation: add into the dequantized previous gradient
                old_wgrad = ctx.weight.grad.to(ctx.output_dtype)
            if not model_state.use_fp8_ddp:
                # GEMM and cast without reading the product back, where the kernel takes the problem (same bits as the
                # two steps below)
                wgrad = Gemm.fp8_gemm_cast(
                    mat_a, mat_b, ctx.output_qtype, metas['wgrad'], sync=True, accumulate=old_wgrad is not None, out=old_wgrad,
                    **layout
                )
            if wgrad is None:
                if old_wgrad is None:
                    wgrad = Gemm.fp8_gemm(mat_a, mat_b, ctx.output_qtype, use_split_accumulator=True, **layout)
                else:
                    wgrad = Gemm.fp8_gemm(
                        mat_a, mat_b, ctx.output_qtype, accumulate=True, out=old_wgrad, use_split_accumulator=True, **layout
                    )
                if model_state.use_fp8_ddp:
                    wgrad.meta = metas['wgrad']
                else:
                    wgrad = wgrad.cast(Dtypes.kfloat8_e4m3, meta=metas['wgrad'], sync=True)
            del old_wgrad
            ctx.weight.backward_grad_update(wgrad)

        bias_grad = output_grad.sum(0).to(ctx.bias_dtype) if ctx.need_bias_grad else None
        return input_grad, None, None, None, bias_grad


class FunctionalOverider:
    """Replaces torch.nn.functional.linear with a version that routes ScalingTensor weights to FP8."""
    EMPTY_GRAD_TENSOR = torch.nn.Parameter(torch.tensor([]))
    _installed = False

    @classmethod
    def override(cls):
        if cls._installed:
            return
        cls._installed = True
        F.linear = cls._get_wrapper_for_linear(F.linear)

    @classmethod
    def _get_wrapper_for_linear(cls, old_fn):
        def new_fn(input, weight, bias=None):
            """linear(input, weight, bias=None): y = x A^T + b; `weight` may be a ScalingTensor carrying
            `_scaling_metas`, in which case the three GEMMs run in FP8 and the bias, rounded to the output dtype
            (the autocast dtype if autocast is on, else the input's), is added in the forward GEMM's epilogue."""
            if not isinstance(input, torch.Tensor):
                raise TypeError(f'input should be a torch.Tensor. current type: {type(input)}')
            if not isinstance(weight, (torch.Tensor, ScalingTensor)):
                raise TypeError(f'weight should be a torch.Tensor or ScalingTensor. current type: {type(weight)}')
            if bias is not None and not isinstance(bias, torch.Tensor):
                raise TypeError(f'bias should be a torch.Tensor. current type: {type(bias)}')
            if isinstance(weight, torch.Tensor):
                return old_fn(input, weight, bias=bias)
            if not hasattr(weight, '_scaling_metas'):
                raise ValueError('weight (ScalingTensor) should have _scaling_metas attribute.')

            model_state.ready_to_scale_tensor = True
            shape = input.shape
            if len(shape) != 2:
                input = input.reshape(-1, shape[-1])
            if torch.is_autocast_enabled():
                output_dtype = torch.get_autocast_dtype('cuda')
            else:
                output_dtype = input.dtype
            out = _FP8GemmFunction.apply(input, weight, weight._scaling_metas, cls.EMPTY_GRAD_TENSOR.type(output_dtype), bias)
            if len(shape) != 2:
                out = out.view(shape[:-1] + (-1, ))
            return out

        return new_fn


FunctionalOverider.override()
