"""Abstract tensor (minit/core/tensor.py:6-20) with the method sugar the hot
path's callers use (minit/core/array.py:45-55 and the special functions)."""
from typing import Tuple

from .object import Object


class Tensor(Object):
    @property
    def shape(self) -> Tuple["Tensor", ...]:
        raise NotImplementedError()

    @property
    def dtype(self) -> str:
        raise NotImplementedError()

    @property
    def device(self) -> str:
        raise NotImplementedError()

    def type(self):
        return type(self)

    # method sugar, as on the reference's Array mixin
    def sum(self, axis: int):
        from ..functional.reduce import sum
        return sum(self, axis)

    def max(self, axis: int):
        from ..functional.reduce import max
        return max(self, axis)

    def rms_norm(self, weight: "Tensor", axis: int, eps: float):
        from ..functional.special import rms_norm
        return rms_norm(self, weight, axis, eps)

    def rope(self, freqs_cos: "Tensor", freqs_sin: "Tensor"):
        from ..functional.special import rope
        return rope(self, freqs_cos, freqs_sin)

    def softmax(self, axis: int):
        from ..functional.special import softmax
        return softmax(self, axis)

    def __add__(self, other: "Tensor"):
        from ..functional.arith import add
        return add(self, other)

    def __mul__(self, other: "Tensor"):
        from ..functional.arith import multiply
        return multiply(self, other)

    def __matmul__(self, other: "Tensor"):
        from ..functional.linalg import matrix_multiply
        return matrix_multiply(self, other)
