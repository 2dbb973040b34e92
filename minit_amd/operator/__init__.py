"""Operator descriptors of the hot path; same names and fields as the reference
(minit/operator/linalg.py:9-16, special.py:6-23, reduce.py:6-13)."""
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
