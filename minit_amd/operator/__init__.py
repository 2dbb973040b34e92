"""Operator descriptors of the hot path; same names, fields and module layout as the reference
(minit/operator/linalg.py, special.py, reduce.py, arith.py)."""
from .arith import Add, Multiply  # noqa: F401
from .linalg import BatchMatrixMultiply, MatrixMultiply  # noqa: F401
from .reduce import Max, Mean, Sum  # noqa: F401
from .special import RMSNorm, RoPE, Sigmoid, Softmax  # noqa: F401
