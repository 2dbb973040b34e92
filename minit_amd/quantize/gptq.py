"""Host-side helpers for the GPTQ checkpoint layout (numpy): packing synthetic
or converted weights into ``qweight`` / ``qzeros`` and building a
:class:`QuantizedTensor` from host arrays.

Layout (examples/qwen1_5_int8.py:276-285, generic in the bit width): sub-word
``i`` of a 32-bit word sits at bit ``i * bits``; ``qweight [K/P, N]`` packs P
consecutive k of one column, ``qzeros [G, N/P]`` packs P consecutive columns of
one group, ``P = 32 / bits``.
"""
import numpy

from ..hip.tensor import HIPTensor
from .tensor import QuantizedTensor


def pack_subwords(values: numpy.ndarray, axis: int, bits: int) -> numpy.ndarray:
    per_word = 32 // bits
    v = numpy.asarray(values)
    assert v.ndim == 2 and bits in (4, 8)
    assert v.min(initial=0) >= 0 and v.max(initial=0) < (1 << bits)
    v = numpy.moveaxis(v.astype(numpy.uint32), axis, -1)
    assert v.shape[-1] % per_word == 0
    v = v.reshape(v.shape[0], v.shape[1] // per_word, per_word)
    out = numpy.zeros(v.shape[:2], dtype=numpy.uint32)
    for i in range(per_word):
        out |= v[:, :, i] << numpy.uint32(i * bits)
    return numpy.ascontiguousarray(numpy.moveaxis(out, -1, axis)).view(numpy.int32)


def quantized_tensor_from_host(qweight, qzeros, scales, g_idx=None) -> QuantizedTensor:
    return QuantizedTensor(
        HIPTensor.from_numpy(numpy.ascontiguousarray(qweight)),
        None if g_idx is None else HIPTensor.from_numpy(numpy.ascontiguousarray(g_idx, dtype=numpy.int32)),
        HIPTensor.from_numpy(numpy.ascontiguousarray(qzeros)),
        HIPTensor.from_numpy(numpy.ascontiguousarray(scales)),
    )
