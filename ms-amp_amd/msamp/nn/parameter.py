"""ScalingParameter: a ScalingTensor registered as a module parameter (msamp/nn/parameter.py:9-28)."""

from msamp.common.tensor import ScalingTensor


class ScalingParameter(ScalingTensor):
    """Trainable ScalingTensor."""
    def __init__(self, tensor, requires_grad=True):
        super().__init__(tensor.value, tensor.meta)
        self._is_param = True
        self.requires_grad = requires_grad

    def __repr__(self):
        return f'ScalingParameter({super().__repr__()}, requires_grad={self.requires_grad})'

    def clone(self):
        return ScalingParameter(super().clone(), requires_grad=self.requires_grad)
