"""``sum`` / ``max`` with keepdim semantics (minit/functional/reduce.py:9-23)."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import Max, Sum


def sum(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Sum(axis=axis), x)
    return z


def max(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Max(axis=axis), x)
    return z
