"""``QLinear`` / ``QLinearWithBias`` (examples/qwen1_5_int8.py:270-317) over the
packed checkpoint tensors: ``forward(x) = x @ dequant(W) [+ bias]``.

The reference's modules unpack the sub-words into uint8 tensors for their
``weight`` property and call a fused kernel in ``forward``; here both go through
the operator API (``matrix_multiply`` on a :class:`QuantizedTensor`, which the
HIP rule serves from the packed words), and the bias is the library's in-place
broadcast add.
"""
from typing import Optional

from ..functional.linalg import matrix_multiply
from ..lib import DTYPE_CODES, call
from ..hip.tensor import HIPTensor
from .gptq import quantized_tensor_from_host
from .tensor import QuantizedTensor


class QLinear:
    def __init__(self, weight: QuantizedTensor, bias: Optional[HIPTensor] = None) -> None:
        if bias is not None:
            assert tuple(bias._shape) == (weight.out_features,), "bias must have N entries"
            assert bias.dtype == weight._scale.dtype, "bias and scales share one dtype"
        self.weight = weight
        self.bias = bias

    @classmethod
    def from_host(cls, w) -> "QLinear":
        """From :class:`minit_amd.quantize.checkpoint.GPTQLinearWeights`."""
        weight = quantized_tensor_from_host(w.qweight, w.qzeros, w.scales, w.g_idx)
        return cls(weight, None if w.bias is None else HIPTensor.from_numpy(w.bias))

    def forward(self, x):
        out = matrix_multiply(x, self.weight)
        if self.bias is not None:
            n = self.weight.out_features
            rows = 1
            for d in out._shape[:-1]:
                rows *= d
            call("mh_add_bias", None, out.data_ptr, self.bias.data_ptr, rows, n, DTYPE_CODES[out.dtype])
        return out

    __call__ = forward
