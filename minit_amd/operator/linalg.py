"""Matrix products (minit/operator/linalg.py:9-16).  ``MatrixMultiply`` is ``x [.., K] @ w [N, K]^T``
(:29-35 gives the orientation); the dispatch rule registered for it with a quantized second operand is
the hot path of this package."""
from dataclasses import dataclass

from ..core.operator import Operator


@dataclass
class MatrixMultiply(Operator):
    ...


@dataclass
class BatchMatrixMultiply(Operator):
    ...
