"""nn.Parameter: a named constant tensor of a Module (counterpart of frontend/nn/parameter.py)."""
from ...compiler.base import Tensor


class Parameter:
    def __init__(self, shape, dtype: str, name: str = None, value=None):
        self._tensor = Tensor(shape=shape, dtype=dtype, name=name)
        self._value = value

    def tensor(self) -> Tensor:
        return self._tensor

    def value(self):
        return self._value
