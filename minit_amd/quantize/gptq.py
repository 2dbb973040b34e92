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
from ..lib import call
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


def unpack_subwords(packed: numpy.ndarray, axis: int, bits: int) -> numpy.ndarray:
    """Inverse of :func:`pack_subwords` (examples/qwen1_5_int8.py:40-50): uint8 sub-words."""
    per_word = 32 // bits
    w = numpy.moveaxis(numpy.asarray(packed).view(numpy.uint32), axis, -1)
    shifts = (numpy.arange(per_word, dtype=numpy.uint32) * bits)[None, None, :]
    v = (w[:, :, None] >> shifts) & numpy.uint32((1 << bits) - 1)
    v = v.reshape(w.shape[0], w.shape[1] * per_word).astype(numpy.uint8)
    return numpy.ascontiguousarray(numpy.moveaxis(v, -1, axis))


def sort_rows_by_group(qweight: numpy.ndarray, g_idx: numpy.ndarray, bits: int, group_size: int):
    """One-time repack of an act-order weight: rows of ``W`` stably sorted by their group.

    Returns ``(qweight_sorted, perm)`` with ``W_sorted[j] = W[perm[j]]`` and
    ``g_idx[perm[j]] == j // group_size``, so ``x @ W == x[:, perm] @ W_sorted``
    and ``W_sorted`` has sequential groups (the layout the MFMA kernels read).
    ``None`` when some group does not hold exactly ``group_size`` rows: such a
    weight stays on the per-element path.
    """
    perm = group_order(g_idx, group_size)
    if perm is None:
        return None
    rows = unpack_subwords(qweight, 0, bits)          # [K, N] uint8
    return pack_subwords(rows[perm], 0, bits), perm


def group_order(g_idx: numpy.ndarray, group_size: int):
    """``perm`` with ``g_idx[perm[j]] == j // group_size`` (rows stably sorted by group), or
    ``None`` when some group does not hold exactly ``group_size`` rows."""
    g = numpy.asarray(g_idx, dtype=numpy.int64)
    k = g.shape[0]
    counts = numpy.bincount(g, minlength=k // group_size)
    if counts.shape[0] != k // group_size or (counts != group_size).any():
        return None
    return numpy.argsort(g, kind="stable").astype(numpy.int32)


def sort_rows_by_group_on_device(qweight: HIPTensor, perm: HIPTensor, bits: int) -> HIPTensor:
    """The repack of :func:`sort_rows_by_group` as one kernel over the packed words on the
    device (``mh_gptq_permute_rows``), with ``perm`` from :func:`group_order`."""
    packed_rows, n = qweight._shape
    k = packed_rows * (32 // bits)
    assert tuple(perm._shape) == (k,) and perm.dtype == "int32"
    out = HIPTensor.allocate((packed_rows, n), "int32")
    call("mh_gptq_permute_rows", None, qweight.data_ptr, perm.data_ptr, out.data_ptr, n, k, bits)
    return out


def quantized_tensor_from_host(qweight, qzeros, scales, g_idx=None) -> QuantizedTensor:
    return QuantizedTensor(
        HIPTensor.from_numpy(numpy.ascontiguousarray(qweight)),
        None if g_idx is None else HIPTensor.from_numpy(numpy.ascontiguousarray(g_idx, dtype=numpy.int32)),
        HIPTensor.from_numpy(numpy.ascontiguousarray(qzeros)),
        HIPTensor.from_numpy(numpy.ascontiguousarray(scales)),
    )


def quantized_tensor_from_unpacked(data, zero, scales, g_idx=None, bits: int = 8) -> QuantizedTensor:
    """From the *unpacked* form the reference's ``QuantizedTensor`` holds
    (examples/qwen1_5_int8.py:276-285: ``data`` uint8 ``[K, N]``, ``zero`` uint8
    ``[G, N]``, one sub-word per element): packed once on the host into the
    checkpoint layout the kernels read.  ``data`` / ``zero`` are numpy arrays or
    device tensors with a ``numpy()`` method.
    """
    def host(t):
        return t.numpy() if hasattr(t, "numpy") else numpy.asarray(t)
    d, z = host(data), host(zero)
    assert d.ndim == 2 and z.ndim == 2 and d.shape[1] == z.shape[1], "data [K, N] and zero [G, N] expected"
    return quantized_tensor_from_host(pack_subwords(d, 0, bits), pack_subwords(z, 1, bits), host(scales),
                                      None if g_idx is None else host(g_idx))
