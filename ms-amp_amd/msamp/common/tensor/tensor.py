"""ScalingTensor: a quantized payload plus its ScalingMeta, and the torch patches that make plain
tensors castable to it (msamp/common/tensor/tensor.py:15-849)."""

import functools

import torch
import torch.nn.functional as F

from msamp import _backend
from msamp.common.dtype import Dtypes, Floating
from msamp.common.tensor.cast import TypeCast
from msamp.common.tensor.hook import HookManager
from msamp.common.tensor.meta import ScalingMeta


class ScalingTensor:
    """`value` (uint8 FP8 codes, or a scaled fp16/bf16/fp32 payload) with `meta`; the real values
    are value * meta.scale_inv.  Duck-types the parts of torch.Tensor that modules, optimizers and
    AMP touch."""

    def __init__(self, value, meta):
        self.value = value
        self.meta = meta
        self._grad = None
        self._backward_post_hooks = HookManager()
        self._requires_grad = False
        expected = Dtypes.get_dtype_from_qtype(meta.qtype)
        if expected != value.dtype:
            raise TypeError(
                f'Type mismatch, value.dtype is {value.dtype}, meta.dtype is {expected} (meta.qtype is {meta.qtype}).'
            )

    # ---- gradient plumbing ----------------------------------------------------------------
    @property
    def grad(self):
        return self._grad

    @grad.setter
    def grad(self, grad):
        self._grad = grad

    @grad.deleter
    def grad(self):
        del self._grad

    def register_backward_post_hook(self, fn):
        """fn(owner, (grad,), grad) runs each time backward_grad_update stores a gradient."""
        return self._backward_post_hooks.register_hook(fn)

    def backward_grad_update(self, grad):
        self.grad = grad
        self._backward_post_hooks(grad)

    @property
    def grad_fn(self):
        return None

    def requires_grad_(self, requires_grad=True):
        self._requires_grad = requires_grad
        return self

    @property
    def is_leaf(self):
        return True

    # ---- construction of relatives --------------------------------------------------------
    def detach(self):
        return ScalingTensor(self.value, self.meta)

    @property
    def data(self):
        return self.detach()

    @data.setter
    def data(self, data):
        with torch.no_grad():
            if isinstance(data, ScalingTensor):
                if self.meta.locked and self.meta is not data.meta:
                    raise ValueError('This ScalingTensor is locked.')
                self.value.data = data.value
                self.meta = data.meta
            elif isinstance(data, torch.Tensor):
                self.value.data = data
            else:
                raise TypeError('The type of data is not supported')

    def clone(self):
        return ScalingTensor(self.value.clone(), self.meta.clone())

    def t(self):
        return ScalingTensor(self.value.t(), self.meta)

    def flatten(self):
        return ScalingTensor(self.value.flatten(), self.meta)

    def pad(self, pad):
        return ScalingTensor(F.pad(self.value, pad), self.meta)

    def contiguous(self):
        meta = self.meta if self.value.is_contiguous() else self.meta.clone()
        return ScalingTensor(self.value.contiguous(), meta)

    def cpu(self, *args, **kwargs):
        return ScalingTensor(self.value.cpu(), self.meta.clone())

    def cuda(self, *args, **kwargs):
        self.value = self.value.cuda()
        if not self.meta.is_cuda:
            if self.meta.locked:
                raise ValueError('This ScalingTensor is locked.')
            self.meta = self.meta.cuda()
        return self

    def to(self, *args, **kwargs):
        """to(dtype | device | non_blocking ...): a float dtype dequantizes; a device moves the payload.

        Positional arguments are told apart by type and each kind may appear once.
        """
        slots = {torch.dtype: 'dtype', torch.device: 'device', bool: 'non_blocking'}
        for a in args:
            if a is None:
                continue
            name = slots.get(type(a))
            if name is None:
                raise TypeError(f'Unsupported dtype in arguments: {type(a)}')
            if name in kwargs:
                raise TypeError(f'Duplicated argument: {name}')
            kwargs[name] = a
        dtype = kwargs.pop('dtype', None)
        out = self
        if dtype is not None:
            if dtype == torch.float32:
                out = self.float()
            elif dtype == torch.float16:
                out = self.half()
            elif dtype == torch.bfloat16:
                out = self.bfloat16()
            else:
                raise TypeError(f'unsupported dtype: {dtype}')
        if isinstance(out, ScalingTensor):
            out.value = out.value.to(**kwargs)
            return out
        return out.to(**kwargs)

    # ---- arithmetic that only touches the scale -------------------------------------------
    @torch.no_grad()
    def mul_(self, other):
        if torch.is_tensor(other):
            if other.numel() != 1:
                raise ValueError('The tensor must by single-element tensor.')
            other = other.view_as(self.meta.scale_inv)
        self.meta.scale_inv *= other
        return self

    @torch.no_grad()
    def div_(self, other):
        if torch.is_tensor(other):
            if other.numel() != 1:
                raise ValueError('The tensor must by single-element tensor.')
            other = other.view_as(self.meta.scale_inv)
        self.meta.scale_inv /= other
        return self

    # ---- casts ----------------------------------------------------------------------------
    def _dequantize(self, otype):
        qtype = self.meta.qtype
        if Dtypes.is_fp8_qtype(qtype):
            return TypeCast.cast_from_fp8(self.value, self.meta, otype)
        if qtype in (Dtypes.kfloat16, Dtypes.kbfloat16):
            return TypeCast.cast_from_fp16(self.value, self.meta, otype)
        if qtype == Dtypes.kfloat32:
            return TypeCast.cast_from_fp32(self.value, self.meta, otype)
        raise TypeError(f'Unsupported Type: {qtype}')

    def float(self):
        return self._dequantize(Dtypes.kfloat32)

    def half(self):
        return self._dequantize(Dtypes.kfloat16)

    def bfloat16(self):
        return self._dequantize(Dtypes.kbfloat16)

    def cast(self, qtype):
        """Re-quantize to `qtype`.  An FP8 source goes through float32; a scaled 16/32-bit source
        is rescaled in one multiply using its stored amax, with no new reduction: the new scale is
        the pow-2 rule of amax for `qtype`, the payload is multiplied by new_scale * old_scale_inv,
        and the new meta keeps amax with scale_inv = 1/new_scale (tensor.py:223-265)."""
        if qtype == self.meta.qtype:
            return self
        if Dtypes.is_fp8_qtype(self.meta.qtype):
            return self.float().cast(qtype)
        old = self.meta
        if Dtypes.is_fp8_qtype(qtype):
            # the whole recipe, new meta included, in one kernel
            meta = ScalingMeta._uninitialized(qtype, old.window_size, old.amax.device)
            value = _backend.cast_scaled_to_fp8(
                self.value.contiguous(), old.amax, old.scale_inv, meta.scale, meta.scale_inv, int(qtype),
                amax_out=meta.amax, counter_out=meta.amax_counter
            )
            return ScalingTensor(value, meta)
        meta = ScalingMeta(qtype, amax=old.amax.clone(), window_size=old.window_size, device=old.amax.device)
        meta.reset_scaling_factor()
        scale_inv = torch.reciprocal(meta.scale)
        meta.scale.mul_(old.scale_inv)
        value = _backend.scale_cast(self.value.contiguous(), meta.scale, Dtypes.get_dtype_from_qtype(qtype))
        meta.scale_inv.copy_(scale_inv)
        return ScalingTensor(value, meta)

    def cast_(self, qtype):
        if self.qtype == qtype:
            return self
        other = self.cast(qtype)
        self.value.data = other.value
        self.meta.copy_(other.meta)
        return self

    def fp8_transpose(self):
        """Materialize the transposed FP8 payload of a 2-D tensor (same meta)."""
        if not Dtypes.is_fp8_qtype(self.meta.qtype):
            raise TypeError(f'Unsupported FP8 transpose type: {self.meta.qtype}')
        return ScalingTensor(_backend.fp8_transpose(self.value.contiguous()), self.meta)

    # ---- element-wise queries -------------------------------------------------------------
    def has_inf_or_nan(self):
        return not bool(torch.isfinite(self.meta.amax[0]))

    def isnan(self):
        if Dtypes.is_fp8_qtype(self.qtype):
            return self.value == 127
        return torch.isnan(self.value)

    def abs(self):
        if self.value.dtype == torch.uint8:
            return ScalingTensor(self.value & 0x7F, self.meta.clone())
        if self.value.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            raise TypeError(f'not support {self.value.dtype}')
        return ScalingTensor(self.value.abs(), self.meta.clone())

    def min(self):
        return self.float().min()

    def max(self):
        return self.float().max()

    def zero_(self):
        self.value.zero_()
        return self

    def copy_(self, src):
        if not isinstance(src, ScalingTensor):
            raise TypeError(f'The input should be a ScalingTensor rather than {type(src)}')
        with torch.no_grad():
            if self.value.dtype != src.value.dtype:
                raise TypeError('The dtype of value must be same.')
            self.value.copy_(src.value)
            self.meta.copy_(src.meta)
        return self

    # ---- tensor-like attributes -----------------------------------------------------------
    @property
    def qtype(self):
        return self.meta.qtype

    @property
    def dtype(self):
        return self.value.dtype

    @property
    def shape(self):
        return self.value.shape

    @property
    def size(self):
        return self.value.size

    @property
    def device(self):
        return self.value.device

    @property
    def is_cuda(self):
        return self.value.is_cuda

    @property
    def is_meta(self):
        return self.value.is_meta

    @property
    def is_sparse(self):
        return self.value.is_sparse

    def numel(self):
        return self.value.numel()

    nelement = numel

    def dim(self):
        return self.value.dim()

    def data_ptr(self):
        return self.value.data_ptr()

    def type(self):
        return f'{self.__class__.__module__}.{self.__class__.__qualname__}'

    def is_contiguous(self):
        return self.value.is_contiguous()

    def is_floating_point(self):
        """False on purpose: module.float()/half() must leave the quantized payload alone."""
        return False

    def is_complex(self):
        return False

    def __len__(self):
        return len(self.value)

    def __repr__(self):
        return f'ScalingTensor({self.float()}, meta={self.meta})'


class TorchOverider:
    """Installs Tensor.cast / Tensor.fused_cast_transpose / Tensor.qtype and makes a handful of
    torch functions accept ScalingTensor (tensor.py:663-849)."""
    one_scales = {}
    torch_unary_funcs = ['torch.zeros_like', 'torch.ones_like', 'torch.overrides.is_tensor_like']
    _installed = False

    @classmethod
    def override(cls):
        if cls._installed:
            return
        cls._installed = True
        torch.Tensor.cast = cls._cast_to_scalingtensor
        torch.Tensor.fused_cast_transpose = cls._fused_cast_transpose_to_scalingtensors
        torch.Tensor.qtype = property(lambda self: Dtypes.dtype_to_qtype[self.dtype])
        for path in cls.torch_unary_funcs:
            owner, name = cls._get_func_base_and_name(path)
            setattr(owner, name, cls._get_wrapper_for_torch_unary(getattr(owner, name)))
        torch.is_floating_point = cls._get_wrapper_for_scalingtensor(torch.is_floating_point, lambda x: x.is_floating_point())
        torch._amp_foreach_non_finite_check_and_unscale_ = cls._get_wrapper_for_grad_check_and_unscale(
            torch._amp_foreach_non_finite_check_and_unscale_
        )

    @staticmethod
    def _cast_to_scalingtensor(self, qtype, meta=None, sync=False):
        """tensor.cast(qtype, meta=None, sync=False) -> ScalingTensor (new window-1 meta by default)."""
        src = self.contiguous()
        if meta is None:
            meta = ScalingMeta(qtype, device=src.device)
        if Dtypes.is_fp8_qtype(qtype):
            return ScalingTensor(TypeCast.cast_to_fp8(src, meta, sync=sync), meta=meta)
        return ScalingTensor(TypeCast.cast_to_fp16(src, meta, sync=sync), meta=meta)

    @staticmethod
    def _fused_cast_transpose_to_scalingtensors(self, qtype, meta=None, sync=False):
        """tensor.fused_cast_transpose(qtype, ...) -> (ScalingTensor, transposed ScalingTensor)."""
        src = self.contiguous()
        if meta is None:
            meta = ScalingMeta(qtype, device=src.device)
        if not Dtypes.is_fp8_qtype(qtype):
            raise TypeError(f'Unsupported Cast: {self.dtype} -> {qtype}')
        q, q_t = TypeCast.cast_to_fp8(src, meta, sync=sync, fuse_transpose=True)
        return ScalingTensor(q, meta=meta), ScalingTensor(q_t, meta=meta)

    @staticmethod
    def _get_func_base_and_name(func_name):
        parts = func_name.split('.')
        if len(parts) < 2:
            raise ValueError(f'Invalid function name: {func_name}')
        owner = globals()[parts[0]]
        for p in parts[1:-1]:
            owner = getattr(owner, p)
        return owner, parts[-1]

    @staticmethod
    def _get_wrapper_for_scalingtensor(old_fn, scaling_fn):
        @functools.wraps(old_fn)
        def fn(input, *args, **kwargs):
            if isinstance(input, ScalingTensor):
                return scaling_fn(input, *args, **kwargs)
            return old_fn(input, *args, **kwargs)

        return fn

    @classmethod
    def _get_wrapper_for_torch_unary(cls, old_fn):
        return cls._get_wrapper_for_scalingtensor(old_fn, lambda x, *a, **k: old_fn(x.value, *a, **k))

    @classmethod
    def _get_wrapper_for_grad_check_and_unscale(cls, old_fn):
        @torch.no_grad()
        def new_fn(grads, found_inf, inv_scale):
            """AMP unscale that also takes ScalingTensor grads: those are unscaled by multiplying
            their scale_inv and checked through amax[0], O(1) per tensor."""
            plain_gpu, plain_cpu, st_scale_inv, st_amax0 = [], [], [], []
            for g in grads:
                if isinstance(g, ScalingTensor):
                    st_scale_inv.append(g.meta.scale_inv)
                    st_amax0.append(g.meta.amax[0])
                elif g.is_cuda:
                    plain_gpu.append(g)
                else:
                    plain_cpu.append(g)
            if plain_gpu:
                old_fn(plain_gpu, found_inf, inv_scale)
            for g in plain_cpu:
                g.mul_(inv_scale)
                if not torch.isfinite(g).all():
                    found_inf.fill_(True)
            if st_scale_inv:
                old_fn(st_scale_inv, found_inf, inv_scale)
                dev = found_inf.device
                if dev not in cls.one_scales:
                    cls.one_scales[dev] = torch.ones(1, device=dev)
                old_fn(st_amax0, found_inf, cls.one_scales[dev])

        return new_fn


TorchOverider.override()

__all__ = ['ScalingTensor', 'TorchOverider', 'Floating']
