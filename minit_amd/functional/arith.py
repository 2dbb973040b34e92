"""``multiply`` and ``add`` (minit/functional/arith.py:9-24), the arithmetic entry
points the hot path's callers use (``x * F.sigmoid(x)``, ``silu(gate) * up`` and the
residual adds, examples/llama3_70b.py:44-45,126-130,159-162).  Operands of one
shape; the reference's broadcast of Python constants is not part of this path."""
from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import Add, Multiply


def multiply(x: Tensor, y: Tensor):
    (z,) = dispatch(Multiply(), x, y)
    return z


def add(x: Tensor, y: Tensor):
    (z,) = dispatch(Add(), x, y)
    return z
