"""Operator descriptors of the hot path; same names and fields as the reference
(minit/operator/linalg.py:9-16, special.py:6-23, reduce.py:6-13, arith.py:20-22)."""
from dataclasses import dataclass

from ..core.operator import Operator


@dataclass
class MatrixMultiply(Operator):
    ...


@dataclass
class BatchMatrixMultiply(Operator):
    ...


class Sigmoid(Operator):
    ...


@dataclass
class Multiply(Operator):
    """minit/operator/arith.py:20-22."""
    ...


@dataclass
class Add(Operator):
    """minit/operator/arith.py (the residual add of the models)."""
    ...


@dataclass
class RMSNorm(Operator):
    axis: int
    eps: float


@dataclass
class RoPE(Operator):
    ...


@dataclass
class Softmax(Operator):
    axis: int


@dataclass
class Sum(Operator):
    axis: int


@dataclass
class Max(Operator):
    axis: int


@dataclass
class Mean(Operator):
    """Not an operator of the reference, whose ``mean`` dispatches Sum, Fill and
    Divide (minit/functional/reduce.py:14-18); one operator here so that the three
    steps are one launch with the same two roundings."""
    axis: int
