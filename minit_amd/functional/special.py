"""``rms_norm`` / ``rope`` / ``softmax`` / ``sigmoid`` entry points with the
reference's signatures and argument checks (minit/functional/special.py:6-26).
``rope`` and ``softmax`` take optional keyword extensions (per-row positions; a
fused causal mask); the reference forms are the defaults."""
from typing import Optional

from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import RMSNorm, RoPE, Sigmoid, Softmax


def sigmoid(x: Tensor):
    (z,) = dispatch(Sigmoid(), x)
    return z


def rms_norm(x: Tensor, weight: Tensor, axis: int, eps: float) -> Tensor:
    assert isinstance(eps, float)
    assert eps > 0
    assert eps < 0.5
    (z,) = dispatch(RMSNorm(axis=axis, eps=eps), x, weight)
    return z


def rope(x: Tensor, freqs_cos: Tensor, freqs_sin: Tensor, positions: Optional[Tensor] = None) -> Tensor:
    if positions is None:
        (z,) = dispatch(RoPE(), x, freqs_cos, freqs_sin)
    else:
        (z,) = dispatch(RoPE(), x, freqs_cos, freqs_sin, positions)
    return z


def softmax(x: Tensor, axis: int) -> Tensor:
    (z,) = dispatch(Softmax(axis=axis), x)
    return z
