"""``multiply`` (minit/functional/arith.py:21-24), the one arithmetic entry point
the hot path's callers use (``x * F.sigmoid(x)`` and ``silu(gate) * up``,
examples/llama3_70b.py:44-45,126-130).  Operands of one shape; the reference's
broadcast of Python constants is not part of this path."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import Multiply


def multiply(x: Tensor, y: Tensor):
    (z,) = dispatch(Multiply(), x, y)
    return z
