"""``dequantize`` (minit/quantize/functional.py:6-8)."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from .operator import Dequantize


def dequantize(x: Tensor, group: Tensor, zero: Tensor, scale: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Dequantize(axis), x, group, zero, scale)
    return z
