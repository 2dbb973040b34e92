"""``Dequantize(axis)`` (minit/quantize/operator.py:5-7)."""
from dataclasses import dataclass

from ..core.operator import Operator


@dataclass
class Dequantize(Operator):
    axis: int
