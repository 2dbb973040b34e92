"""``dequantize`` (minit/quantize/functional.py:6-8): the functional face of the
``Dequantize`` operator; whichever rule is registered for the argument types runs."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from .operator import Dequantize


def dequantize(x: Tensor, group: Tensor, zero: Tensor, scale: Tensor, axis: int) -> Tensor:
    """``x`` packed sub-words, ``group`` the row -> group map (or the no-group marker),
    ``zero`` / ``scale`` per group; ``axis`` is the axis the sub-words are packed along."""
    outputs = dispatch(Dequantize(axis=axis), x, group, zero, scale)
    assert len(outputs) == 1
    return outputs[0]
