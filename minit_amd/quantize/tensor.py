"""``QuantizedTensor(data, group, zero, scale)`` (minit/quantize/tensor.py:9-30).

The reference holds *unpacked* uint8 sub-words (examples/qwen1_5_int8.py:283-285);
this one holds the packed GPTQ checkpoint tensors as they are: ``data`` =
``qweight`` int32 ``[K/P, N]`` packed along K, ``zero`` = ``qzeros`` int32
``[G, N/P]`` packed along N, ``scale`` = ``scales`` fp16 ``[G, N]``, ``group`` =
``g_idx`` int32 ``[K]`` or ``None`` for ``k // group_size``; ``P = 32 / bits``.
"""
from typing import Optional

import numpy

from ..core.scalar import ScalarTensor
from ..core.tensor import Tensor
from .functional import dequantize


class _NoGroup(Tensor):
    """Placeholder for an absent ``g_idx`` so dispatch still sees a tensor."""

    @property
    def shape(self):
        return ()

    @property
    def dtype(self):
        return "int32"

    @property
    def device(self):
        return "host"


NO_GROUP = _NoGroup()


class QuantizedTensor(Tensor):
    def __init__(self, data: Tensor, group: Optional[Tensor], zero: Tensor, scale: Tensor) -> None:
        super().__init__()
        rows, n = (d.item() for d in data.shape)
        groups, packed_n = (d.item() for d in zero.shape)
        groups2, n2 = (d.item() for d in scale.shape)
        assert data.dtype == "int32" and zero.dtype == "int32", "packed tensors must be int32"
        assert groups == groups2 and n == n2, "qzeros / scales / qweight disagree"
        assert n % packed_n == 0
        per_word = n // packed_n
        assert per_word in (4, 8), f"unsupported pack size {per_word}"
        self.bits = 32 // per_word
        self.in_features = rows * per_word
        self.out_features = n
        assert self.in_features % groups == 0
        self.group_size = self.in_features // groups
        if group is not None:
            (klen,) = (d.item() for d in group.shape)
            # shape contract of the reference's fused path (qwen1_5_int8.py:247-254)
            assert klen == self.in_features, "g_idx must have K entries"
            host = group.numpy()
            trivial = numpy.arange(self.in_features, dtype=host.dtype) // self.group_size
            if numpy.array_equal(host, trivial):
                group = None  # sequential groups: the kernels compute k // group_size
        self._data = data
        self._group = group
        self._zero = zero
        self._scale = scale

    @property
    def shape(self):
        return (ScalarTensor(self.in_features, (), "int32"), ScalarTensor(self.out_features, (), "int32"))

    @property
    def dtype(self):
        return f"quint{self.bits}"

    @property
    def device(self):
        return self._data.device

    def dequantize(self) -> Tensor:
        group = self._group if self._group is not None else NO_GROUP
        return dequantize(self._data, group, self._zero, self._scale, 0)
