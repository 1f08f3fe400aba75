"""Scaling-tensor package."""

from msamp.common.tensor.cast import TypeCast
from msamp.common.tensor.hook import HookManager
from msamp.common.tensor.meta import ScalingMeta
from msamp.common.tensor.tensor import ScalingTensor, TorchOverider

__all__ = ['TypeCast', 'HookManager', 'ScalingMeta', 'ScalingTensor', 'TorchOverider']
