"""ScalingMeta: per-tensor scale, reciprocal scale and amax window (msamp/common/tensor/meta.py:12-159)."""

import copy

import torch

from msamp import _backend
from msamp.common.dtype import Floating, Dtypes


class ScalingMeta:
    """Scaling state of one quantized tensor.

    scale, scale_inv: 0-d float32; amax: (window_size,) float32 with amax[0] the current value;
    amax_counter: 0-d int32 counting window updates.  All four live on the meta's device.  With the
    counter on the GPU the casts take the warm-up test on the device (scaling_mode() == 'gated'), so
    nothing in a training step waits for the GPU; is_warmup() / is_in_time_scaling() still answer on
    the host, at the price of a synchronisation.
    """
    in_time_scaling: bool = True

    def __init__(self, qtype, scale=None, scale_inv=None, amax=None, window_size=1, group=None, device='cuda'):
        self.qtype = qtype
        self.scale = scale if scale is not None else torch.ones((), device=device)
        self.scale_inv = scale_inv if scale_inv is not None else torch.ones((), device=device)
        self.amax = amax if amax is not None else torch.zeros((window_size, ), device=device)
        self.amax_counter = torch.zeros((), dtype=torch.int32, device=self.amax.device)
        self.window_size = window_size
        self.group = group
        self.locked = False

    @classmethod
    def _uninitialized(cls, qtype, window_size, device, group=None):
        """A meta whose four tensors are views of one uninitialised buffer, for callers whose kernel
        writes every field (scale, scale_inv, counter, amax window) itself."""
        self = cls.__new__(cls)
        slab = torch.empty(3 + window_size, dtype=torch.float32, device=device)
        self.qtype = qtype
        self.scale, self.scale_inv = slab[0], slab[1]
        self.amax_counter = slab[2:3].view(torch.int32).reshape(())
        self.amax = slab[3:]
        self.window_size = window_size
        self.group = group
        self.locked = False
        return self

    @staticmethod
    def compute_scaling_factor(amax, scale, fp_max: float, margin: int):
        """Largest power of two sf with sf * amax <= fp_max (shifted down by `margin` binades).

        Evaluated on the GPU by the library with the float32 semantics of
        meta.py:51-56 of the reference: `scale` is kept where amax is zero, negative or NaN; for
        amax = +Inf the result is 1/scale; a denormal amax gives +Inf.
        """
        shape = amax.shape
        out = _backend.compute_scaling_factor(amax.reshape(-1), scale.reshape(-1), float(fp_max), int(margin))
        return out.reshape(shape)

    def is_warmup(self):
        return self.amax_counter < self.window_size

    def is_in_time_scaling(self):
        return ScalingMeta.in_time_scaling and (self.window_size == 1 or bool(self.is_warmup()))

    def scaling_mode(self):
        """'in_time', 'delayed', or 'gated' when only the GPU-resident counter can tell (no sync)."""
        if not ScalingMeta.in_time_scaling:
            return 'delayed'
        if self.window_size == 1:
            return 'in_time'
        if self.amax_counter.is_cuda:
            return 'gated'
        return 'in_time' if bool(self.is_warmup()) else 'delayed'

    @staticmethod
    def in_time_scaling_context(enabled):
        """Context manager that sets the class-wide in_time_scaling flag and restores it on exit."""
        class _Ctx:
            def __enter__(self):
                self.saved = ScalingMeta.in_time_scaling
                ScalingMeta.in_time_scaling = enabled

            def __exit__(self, exc_type, exc_val, exc_tb):
                ScalingMeta.in_time_scaling = self.saved

        return _Ctx()

    def reset_scaling_factor(self, qtype=None):
        """scale <- rule(amax[0]) for quantized types, 1 for float32 / bfloat16 payloads."""
        if qtype is None:
            qtype = self.qtype
        if qtype in (Dtypes.kfloat32, Dtypes.kbfloat16):
            self.scale.fill_(1)
        else:
            fp_max = Floating.qfp_max[qtype]
            self.scale.copy_(ScalingMeta.compute_scaling_factor(self.amax[0], self.scale, fp_max, 0))

    def copy_(self, src):
        self.qtype = src.qtype
        self.scale.copy_(src.scale)
        self.scale_inv.copy_(src.scale_inv)
        self.amax.copy_(src.amax)
        self.amax_counter.copy_(src.amax_counter)
        self.window_size = src.window_size

    def clone(self):
        group, self.group = self.group, None
        obj = copy.deepcopy(self)
        self.group = obj.group = group
        return obj

    def cuda(self):
        self.scale = self.scale.cuda()
        self.scale_inv = self.scale_inv.cuda()
        self.amax = self.amax.cuda()
        self.amax_counter = self.amax_counter.cuda()
        return self

    def cpu(self):
        self.scale = self.scale.cpu()
        self.scale_inv = self.scale_inv.cpu()
        self.amax = self.amax.cpu()
        self.amax_counter = self.amax_counter.cpu()
        return self

    @property
    def is_cuda(self):
        return self.scale.is_cuda

    def __repr__(self):
        return (f'ScalingMeta(qtype={self.qtype}, scale={self.scale.item():g}, scale_inv={self.scale_inv.item():g}, '
                f'amax={self.amax.max().item():g}, window_size={self.window_size})')
