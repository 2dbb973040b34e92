"""``sum`` / ``mean`` / ``max`` with keepdim semantics (minit/functional/reduce.py:9-23)."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import Max, Mean, Sum


def sum(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Sum(axis=axis), x)
    return z


def mean(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Mean(axis=axis), x)
    return z


def max(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Max(axis=axis), x)
    return z
