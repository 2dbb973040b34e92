"""``QLinear`` / ``QLinearWithBias`` (examples/qwen1_5_int8.py:270-317) over the
packed checkpoint tensors: ``forward(x) = x @ dequant(W) [+ bias]``.

The reference's modules unpack the sub-words into uint8 tensors for their
``weight`` property and call a fused kernel in ``forward``; here both go through
the packed words: ``weight`` is a :class:`QuantizedTensor` (the operator API's
``matrix_multiply`` serves it as well), and ``forward`` is one ``mh_gptq_linear``
call, the bias riding on the product kernel's stores.
"""
from typing import Optional

from ..lib import DTYPE_CODES, call
from ..hip import memory
from ..hip.tensor import HIPTensor
from .gptq import group_order, quantized_tensor_from_host, sort_rows_by_group_on_device
from .tensor import QuantizedTensor


class QLinear:
    def __init__(self, weight: QuantizedTensor, bias: Optional[HIPTensor] = None,
                 input_order: Optional[HIPTensor] = None) -> None:
        """``input_order`` (int32 ``[K]``): the activations' columns are gathered in
        this order before the product (a weight whose rows were sorted by group)."""
        if bias is not None:
            assert tuple(bias._shape) == (weight.out_features,), "bias must have N entries"
            assert bias.dtype == weight._scale.dtype, "bias and scales share one dtype"
        if input_order is not None:
            assert tuple(input_order._shape) == (weight.in_features,) and input_order.dtype == "int32"
        self.weight = weight
        self.bias = bias
        self.input_order = input_order

    @classmethod
    def from_host(cls, w, reorder: bool = True) -> "QLinear":
        """From :class:`minit_amd.quantize.checkpoint.GPTQLinearWeights`.

        An act-order weight (``g_idx`` not sequential) is repacked once on the device,
        rows sorted by group, so that the product runs on the MFMA kernels with the
        activations gathered to match; ``reorder=False`` (or groups of uneven size) keeps the
        checkpoint layout and the per-element kernel.
        """
        bias = None if w.bias is None else HIPTensor.from_numpy(w.bias)
        if w.g_idx is not None and reorder:
            geo = w.geometry
            perm = group_order(w.g_idx, geo.group_size)
            if perm is not None:
                order = HIPTensor.from_numpy(perm)
                weight = quantized_tensor_from_host(w.qweight, w.qzeros, w.scales, None)
                weight._data = sort_rows_by_group_on_device(weight._data, order, geo.bits)
                return cls(weight, bias, order)
        return cls(quantized_tensor_from_host(w.qweight, w.qzeros, w.scales, w.g_idx), bias)

    def forward(self, x):
        """``x [..., K] -> [..., N]``: one ``mh_gptq_linear`` call (product and bias in one launch,
        examples/qwen1_5_int8.py:311-317 runs them as two), after the gather of the activations'
        columns when the weight's rows were sorted by group at load time."""
        w = self.weight
        k, n = w.in_features, w.out_features
        assert x._shape[-1] == k, f"x has K={x._shape[-1]}, weight has K={k}"
        assert x.dtype == "float16" and w._scale.dtype == x.dtype
        rows = 1
        for d in x._shape[:-1]:
            rows *= d
        if self.input_order is not None:
            gathered = HIPTensor.allocate(x._shape, x.dtype)
            call("mh_gather_columns", None, x.data_ptr, self.input_order.data_ptr, gathered.data_ptr, rows, k,
                 DTYPE_CODES[x.dtype])
            x = gathered
        out = HIPTensor.allocate((*x._shape[:-1], n), x.dtype)
        if rows == 0:
            return out
        ws = memory.workspace(max(call("mh_gptq_workspace_bytes", rows, n, k, w.group_size, w.bits), 256))
        call("mh_gptq_linear", None, x.data_ptr, w._data.data_ptr, w._zero.data_ptr, w._scale.data_ptr,
             None if w._group is None else w._group.data_ptr, None if self.bias is None else self.bias.data_ptr,
             out.data_ptr, rows, n, k, w.group_size, w.bits, ws._pointer, ws._size)
        return out

    __call__ = forward
