from . import BatchMatrixMultiply, MatrixMultiply  # noqa: F401
