"""GPTQ pack / unpack / dequantize / quantized matmul, restated on the CPU.

Test infrastructure only (see ``oracle/__init__.py``).

Follows, in the reference tree:

* ``examples/qwen1_5_int8.py:40-50``   ``unpack`` -- sub-words come out in
  memory (little-endian) order along the packed axis;
* ``examples/qwen1_5_int8.py:97-138``  ``RowPackedMatrix`` / ``ColPackedMatrix``
  accessors -- ``(pack >> ((idx % P) * b)) & mask`` with ``P = 32 / b``;
* ``examples/qwen1_5_int8.py:276-285`` buffer shapes: ``qweight [K/P, N]`` is
  packed along K, ``qzeros [G, N/P]`` along N, ``scales [G, N]``, ``g_idx [K]``;
* ``minit/quantize/dispatch.py:14-20``  ``W = (q - (z + 1)) * s`` evaluated in
  ``scale.dtype`` after gathering zero and scale rows by ``g_idx``;
* ``minit/quantize/dispatch.py:8-11``   matmul = dequantize, then a dense
  matmul with fp32 accumulation (``minit/cuda/kernel/cublas.py:116-127``) and
  one rounding to the activation dtype.

The reference instantiates these for 8-bit sub-words; the accessors are generic
in the bit width and the benchmark configurations use 4 bits, so ``bits`` is a
parameter here.
"""
import numpy as np


def _check_bits(bits):
    if bits not in (2, 4, 8):
        raise ValueError(f"unsupported bit width {bits}")
    return 32 // bits


def unpack(packed: np.ndarray, axis: int, bits: int = 4) -> np.ndarray:
    """Sub-word extraction; ``packed`` is int32 ``[R, C]``; returns uint8.

    ``axis == 0``: ``out[r * P + i, c] = (packed[r, c] >> (i * bits)) & mask``
    (the ColPackedMatrix accessor, qwen1_5_int8.py:119-138);
    ``axis == 1``: ``out[r, c * P + i] = (packed[r, c] >> (i * bits)) & mask``
    (the RowPackedMatrix accessor, qwen1_5_int8.py:97-116).
    """
    per_word = _check_bits(bits)
    if packed.dtype != np.int32 or packed.ndim != 2:
        raise ValueError("packed must be a 2-D int32 array")
    if axis not in (0, 1):
        raise ValueError("axis must be 0 or 1")
    words = packed.view(np.uint32)
    mask = np.uint32((1 << bits) - 1)
    shifts = (np.arange(per_word, dtype=np.uint32) * np.uint32(bits))
    rows, cols = packed.shape
    if axis == 0:
        out = (words[:, None, :] >> shifts[None, :, None]) & mask
        return out.reshape(rows * per_word, cols).astype(np.uint8)
    out = (words[:, :, None] >> shifts[None, None, :]) & mask
    return out.reshape(rows, cols * per_word).astype(np.uint8)


def unpack_by_views(packed: np.ndarray, axis: int) -> np.ndarray:
    """The reference's own 8-bit ``unpack`` spelled as view algebra.

    qwen1_5_int8.py:40-50: reinterpret int32 as uint8 (memory order), split the
    last axis into ``[last, 4]``, move the sub-word axis next to ``axis`` and
    fold.  Only meaningful for 8-bit sub-words on a little-endian host; used to
    cross-check ``unpack(..., bits=8)``.
    """
    assert packed.dtype == np.int32 and packed.ndim == 2
    last = packed.shape[-1]
    x = np.ascontiguousarray(packed).view(np.uint8)          # [R, C*4]
    x = x.reshape(packed.shape[0], last, 4)                   # expand
    x = np.expand_dims(x, axis + 1)                           # add_axis(axis+1)
    x = np.swapaxes(x, axis + 1, x.ndim - 1)                  # transpose
    x = np.squeeze(x, axis=x.ndim - 1)                        # remove_axis
    shape = list(x.shape)
    shape[axis:axis + 2] = [shape[axis] * shape[axis + 1]]    # fold
    return np.ascontiguousarray(x).reshape(shape)


def pack(values: np.ndarray, axis: int, bits: int = 4) -> np.ndarray:
    """Inverse of :func:`unpack` (sub-word ``i`` lands at bit ``i * bits``)."""
    per_word = _check_bits(bits)
    v = np.asarray(values)
    if v.ndim != 2:
        raise ValueError("values must be 2-D")
    if v.min(initial=0) < 0 or v.max(initial=0) >= (1 << bits):
        raise ValueError("value does not fit the bit width")
    v = v.astype(np.uint32)
    shifts = (np.arange(per_word, dtype=np.uint32) * np.uint32(bits))
    rows, cols = v.shape
    if axis == 0:
        if rows % per_word:
            raise ValueError("rows not a multiple of the pack size")
        w = v.reshape(rows // per_word, per_word, cols) << shifts[None, :, None]
        return np.bitwise_or.reduce(w, axis=1).astype(np.uint32).view(np.int32)
    if cols % per_word:
        raise ValueError("cols not a multiple of the pack size")
    w = v.reshape(rows, cols // per_word, per_word) << shifts[None, None, :]
    return np.bitwise_or.reduce(w, axis=2).astype(np.uint32).view(np.int32)


def dequantize(data: np.ndarray, group: np.ndarray, zero: np.ndarray,
               scale: np.ndarray) -> np.ndarray:
    """``Dequantize(axis=0)`` of the reference on *unpacked* operands.

    minit/quantize/dispatch.py:14-20::

        scale = scale.index(group, axis); zero = zero.index(group, axis)
        output = (data.cast(dtype) - (zero.cast(dtype) + 1)) * scale

    with ``dtype = scale.dtype`` (fp16 here).  ``data - (zero + 1)`` is an exact
    small integer in fp16 (|.| <= 256), so the only rounding is the multiply;
    numpy's fp16 multiply rounds to nearest-even once, as the device does.
    """
    dtype = scale.dtype
    s = scale[group]                       # [K, N]
    z = zero[group]                        # [K, N]
    one = np.array(1, dtype=dtype)
    return (data.astype(dtype) - (z.astype(dtype) + one)) * s


def dequantize_packed(qweight, qzeros, scales, g_idx=None, bits=4, group_size=None):
    """Dequantize straight from the packed checkpoint tensors -> ``[K, N]``."""
    per_word = _check_bits(bits)
    k = qweight.shape[0] * per_word
    if g_idx is None:
        if group_size is None:
            group_size = k // scales.shape[0]
        g_idx = (np.arange(k) // group_size).astype(np.int32)
    data = unpack(qweight, 0, bits)
    zero = unpack(qzeros, 1, bits)
    return dequantize(data, np.asarray(g_idx), zero, scales)


def dense_matmul(x: np.ndarray, w_kn: np.ndarray) -> np.ndarray:
    """``y[m, n] = round_to_x_dtype( sum_k fp32(x[m, k]) * fp32(w[k, n]) )``.

    The reference's dense product computes in fp32 and stores in the input
    dtype (minit/cuda/kernel/cublas.py:116-127, CUBLAS_COMPUTE_32F); the
    summation order is the library's, so the oracle accumulates in float64 and
    rounds once -- every fp32 summation order is within a few fp32 ulps of it.
    """
    acc = x.astype(np.float64) @ w_kn.astype(np.float64)
    return acc.astype(x.dtype)


def matmul_f64(x, qweight, qzeros, scales, g_idx=None, bits=4, group_size=None):
    """The un-rounded accumulator of :func:`matmul` (float64)."""
    w = dequantize_packed(qweight, qzeros, scales, g_idx, bits, group_size)
    return x.astype(np.float64) @ w.astype(np.float64)


def matmul(x, qweight, qzeros, scales, g_idx=None, bits=4, group_size=None):
    """``MatrixMultiply(Tensor, QuantizedTensor)``: ``x[M, K] @ dequant(W)[K, N]``.

    minit/quantize/dispatch.py:8-11; the fused kernel computes the same
    contraction (qwen1_5_int8.py:156-200) and enforces ``K == P * rows(qweight)
    == len(g_idx)`` and ``N == P * cols(qzeros) == cols(scales)`` (:247-254).
    """
    per_word = _check_bits(bits)
    k = qweight.shape[0] * per_word
    n = qweight.shape[1]
    if x.shape[-1] != k:
        raise ValueError("x and qweight disagree on K")
    if qzeros.shape[1] * per_word != n or scales.shape[1] != n:
        raise ValueError("qzeros / scales disagree with qweight on N")
    if qzeros.shape[0] != scales.shape[0]:
        raise ValueError("qzeros / scales disagree on the number of groups")
    if g_idx is not None and len(g_idx) != k:
        raise ValueError("g_idx must have K entries")
    lead = x.shape[:-1]
    y = matmul_f64(x.reshape(-1, k), qweight, qzeros, scales, g_idx, bits, group_size)
    return y.astype(x.dtype).reshape(*lead, n)


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """``silu(gate) * up`` as the models spell it, one launch per step.

    examples/llama3_70b.py:44-45,126-130 with the element-wise expressions of
    minit/cuda/dispatch.py:137,143: ``sig = T(1 / (1 + expf(-g)))``,
    ``a = g * sig`` (fp16 multiply), ``h = a * u`` (fp16 multiply) -- three
    roundings to fp16.
    """
    dtype = gate.dtype
    g32 = gate.astype(np.float32)
    sig = (1.0 / (1.0 + np.exp(-g32.astype(np.float64)))).astype(dtype)
    a = gate * sig
    return a * up


def silu_mul_f64(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """The same product without intermediate rounding (float64)."""
    g = gate.astype(np.float64)
    return g / (1.0 + np.exp(-g)) * up.astype(np.float64)
