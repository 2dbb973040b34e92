"""A Python number with a shape and dtype (minit/core/scalar.py:8-43); tensor
shapes are tuples of these."""
from numbers import Number
from typing import Tuple

from .dtype import dtype_info
from .tensor import Tensor


class ScalarTensor(Tensor):
    __slots__ = ["_value", "_shape", "_dtype"]

    def __init__(self, value: Number, shape: Tuple[Tensor, ...], dtype: str) -> None:
        assert not isinstance(value, Tensor)
        assert shape is not None and dtype is not None
        self._value = value
        self._shape = shape
        self._dtype = dtype

    @property
    def shape(self):
        return self._shape

    @property
    def dtype(self):
        return self._dtype

    @property
    def device(self):
        return "host"

    def value(self):
        return self._value

    def item(self) -> Number:
        assert len(self.shape) == 0
        return dtype_info(self._dtype).python_type(self._value)

    def __repr__(self) -> str:
        return f"Scalar({self._value}: {self._dtype})"

    def type(self):
        return ScalarTensor


def to_immediate_shape(shape) -> Tuple[int, ...]:
    """minit/core/shape.py:13-14."""
    return tuple(dim.item() if isinstance(dim, Tensor) else int(dim) for dim in shape)
