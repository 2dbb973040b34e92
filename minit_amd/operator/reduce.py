"""Reductions along one axis (minit/operator/reduce.py:6-13)."""
from dataclasses import dataclass

from ..core.operator import Operator


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
