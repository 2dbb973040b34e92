"""``matrix_multiply`` (minit/functional/linalg.py:9-20): the right operand is
2-D, leading dimensions of the left operand are folded into M and restored."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import MatrixMultiply


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
