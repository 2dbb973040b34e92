"""Element-wise arithmetic descriptors (minit/operator/arith.py:20-22)."""
from dataclasses import dataclass

from ..core.operator import Operator


@dataclass
class Multiply(Operator):
    ...


@dataclass
class Add(Operator):
    """The residual add of the models."""
    ...
