"""Optimizers for low-bit parameters."""

from msamp.optim.optimizer import LBOptimizer
from msamp.optim.adamw_base import LBAdamWBase
from msamp.optim.adamw import LBAdamW
from msamp.optim.adam import LBAdam, DSAdam

__all__ = ['LBOptimizer', 'LBAdamWBase', 'LBAdamW', 'LBAdam', 'DSAdam']
