"""``matrix_multiply`` (minit/functional/linalg.py:9-20): the right operand is
2-D, leading dimensions of the left operand are folded into M and restored;
``batch_matrix_multiply`` (minit/functional/linalg.py:23-33): leading dimensions
of both operands are folded into one batch axis."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import BatchMatrixMultiply, MatrixMultiply


def matrix_multiply(x: Tensor, y: Tensor) -> Tensor:
    assert len(y.shape) == 2
    lead = None
    if len(x.shape) > 2:
        lead = tuple(d.item() for d in x.shape[:-1])
        m = 1
        for d in lead:
            m *= d
        x = x.reshape((m, x.shape[-1].item()))
    (z,) = dispatch(MatrixMultiply(), x, y)
    if lead is not None:
        z = z.reshape((*lead, z.shape[-1].item()))
    return z


def batch_matrix_multiply(x: Tensor, y: Tensor) -> Tensor:
    assert len(x.shape) > 2 and len(y.shape) > 2
    lead = tuple(d.item() for d in x.shape[:-2])
    batch = 1
    for d in lead:
        batch *= d
    x = x.reshape((batch, x.shape[-2].item(), x.shape[-1].item()))
    y = y.reshape((batch, y.shape[-2].item(), y.shape[-1].item()))
    (z,) = dispatch(BatchMatrixMultiply(), x, y)
    return z.reshape((*lead, z.shape[-2].item(), z.shape[-1].item()))
