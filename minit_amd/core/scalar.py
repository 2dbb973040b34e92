"""Host-side scalars: a Python number that carries a tensor's surface (shape, dtype,
device), so that tensor shapes can be tuples of tensors as in the reference
(minit/core/scalar.py:8-43, minit/core/shape.py:13-14)."""
from numbers import Number
from typing import Iterable, Tuple

from .dtype import dtype_info
from .tensor import Tensor


class ScalarTensor(Tensor):
    """Immutable (value, shape, dtype) triple.  ``value()`` hands back what was stored,
    ``item()`` converts it to the Python type of the dtype and is defined for rank 0 only."""

    __slots__ = ("_triple",)

    def __init__(self, value: Number, shape: Tuple[Tensor, ...], dtype: str) -> None:
        if isinstance(value, Tensor):
            raise AssertionError("a scalar wraps a plain number, not a tensor")
        if shape is None or dtype is None:
            raise AssertionError("a scalar needs a shape and a dtype")
        self._triple = (value, shape, dtype)

    shape = property(lambda self: self._triple[1])
    dtype = property(lambda self: self._triple[2])
    device = property(lambda self: "host")

    def value(self):
        return self._triple[0]

    def item(self) -> Number:
        stored, shape, dtype = self._triple
        assert len(shape) == 0, "item() is defined for rank-0 scalars"
        return dtype_info(dtype).python_type(stored)

    def type(self):
        return ScalarTensor

    def __repr__(self) -> str:
        return "Scalar({}: {})".format(self._triple[0], self._triple[2])


def to_immediate_shape(shape: Iterable) -> Tuple[int, ...]:
    """Plain ints out of a shape whose entries may be scalars or ints."""
    return tuple(int(dim.item()) if isinstance(dim, Tensor) else int(dim) for dim in shape)
