"""``rms_norm`` / ``rope`` / ``softmax`` / ``sigmoid``: the functional face of the
operators in ``minit_amd.operator`` with the reference's names, argument order and
argument checks (minit/functional/special.py:6-26).  ``rope`` takes an optional fourth
tensor (per-row positions); without it the call is the reference's."""
from typing import Optional

from ..core.dispatch import dispatch
from ..core.tensor import Tensor
from ..operator import RMSNorm, RoPE, Sigmoid, Softmax


def _single(outputs):
    """Every rule returns a tuple; these operators have one result."""
    assert len(outputs) == 1, f"expected one output, got {len(outputs)}"
    return outputs[0]


def sigmoid(x: Tensor) -> Tensor:
    return _single(dispatch(Sigmoid(), x))


def rms_norm(x: Tensor, weight: Tensor, axis: int, eps: float) -> Tensor:
    # the reference insists on a python float in (0, 0.5): an int or an array here is a slipped argument
    assert isinstance(eps, float) and 0.0 < eps < 0.5, f"eps must be a float in (0, 0.5), got {eps!r}"
    return _single(dispatch(RMSNorm(axis=axis, eps=eps), x, weight))


def rope(x: Tensor, freqs_cos: Tensor, freqs_sin: Tensor, positions: Optional[Tensor] = None) -> Tensor:
    operands = (x, freqs_cos, freqs_sin) if positions is None else (x, freqs_cos, freqs_sin, positions)
    return _single(dispatch(RoPE(), *operands))


def softmax(x: Tensor, axis: int) -> Tensor:
    return _single(dispatch(Softmax(axis=axis), x))
