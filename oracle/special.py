"""RMSNorm, RoPE, softmax (+ causal mask) and row reductions on the CPU.

Test infrastructure only.  Each function evaluates the reference kernel's
closed form in float64 and rounds once to the storage dtype, which is what the
reference kernels do in fp32 (they keep fp32 internally and round at the
store), up to fp32 round-off.
"""
import math

import numpy as np


def _abc(shape, axis):
    a = int(np.prod(shape[:axis], dtype=np.int64))
    b = int(shape[axis])
    c = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return a, b, c


def rms_norm(x: np.ndarray, weight: np.ndarray, axis: int, eps: float) -> np.ndarray:
    """minit/cuda/kernel/cuda/rms_norm.py:69-89 over the view ``[a, b, c]``.

    ``out = T( x / sqrt(sum(x^2) / b + eps) * w[b] )``; eps reaches the kernel
    as a float (rms_norm.py:94,98).
    """
    a, b, c = _abc(x.shape, axis)
    assert weight.shape == (b,)
    v = x.reshape(a, b, c).astype(np.float64)
    mean = (v * v).sum(axis=1, keepdims=True) / b
    rms = np.sqrt(mean + np.float64(np.float32(eps)))
    out = v / rms * weight.astype(np.float64)[None, :, None]
    return out.astype(x.dtype).reshape(x.shape)


def rope_tables(head_size: int, nr_positions: int, theta: float):
    """cos / sin tables ``[nr_positions, head_size / 2]`` in float32.

    examples/llama3_70b.py:206-212: ``freqs = (1/theta) ** (2 i / dim)``,
    ``angle = t * freqs``.  The example then casts the tables to fp16 although
    the operator asserts float32 (minit/cuda/dispatch.py:449-450); float32 is
    what the kernel signature takes (rope.py:58) and what is produced here.
    """
    i = np.arange(head_size // 2, dtype=np.float64)
    freqs = (1.0 / theta) ** (2.0 * i / head_size)
    t = np.arange(nr_positions, dtype=np.float64)
    ang = t[:, None] * freqs[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def rope(x: np.ndarray, freqs_cos: np.ndarray, freqs_sin: np.ndarray,
         positions: np.ndarray = None) -> np.ndarray:
    """Interleaved-pair rotary embedding, minit/cuda/kernel/cuda/rope.py:58-73.

    ``x`` is ``[bs, seq, nh, hs]``.  Reference form (``positions is None``):
    the tables are ``[seq, hs/2]`` and indexed by the sequence index.  With
    ``positions`` (int, ``[bs, seq]``) the tables are ``[P, hs/2]`` and row
    ``positions[b, s]`` is used; ``positions[b, s] = s`` on a table sliced at
    ``offset`` reduces to the reference form.
    """
    bs, seq, nh, hs = x.shape
    half = hs // 2
    if positions is None:
        assert freqs_cos.shape == (seq, half)
        cos = freqs_cos[None, :, None, :]
        sin = freqs_sin[None, :, None, :]
    else:
        positions = np.asarray(positions).reshape(bs, seq)
        cos = freqs_cos[positions][:, :, None, :]
        sin = freqs_sin[positions][:, :, None, :]
    cos = cos.astype(np.float64)
    sin = sin.astype(np.float64)
    v = x.astype(np.float64).reshape(bs, seq, nh, half, 2)
    real, imag = v[..., 0], v[..., 1]
    out = np.empty_like(v)
    out[..., 0] = real * cos - imag * sin
    out[..., 1] = imag * cos + real * sin
    return out.reshape(x.shape).astype(x.dtype)


def softmax(x: np.ndarray, axis: int) -> np.ndarray:
    """minit/cuda/kernel/cuda/softmax.py:71-105: max, sum of exp, normalise."""
    v = x.astype(np.float64)
    m = v.max(axis=axis, keepdims=True)
    # a fully masked row has max == -inf; the kernel then computes exp(nan)
    with np.errstate(invalid="ignore"):
        e = np.exp(v - m)
    return (e / e.sum(axis=axis, keepdims=True)).astype(x.dtype)


def causal_mask(seqlen: int, offset: int, dtype=np.float16) -> np.ndarray:
    """The additive mask the models build, ``[seqlen, offset + seqlen]``.

    examples/llama3_70b.py:103-107 with the predicate of
    minit/cuda/dispatch.py:393 (``row + diagonal <= col`` keeps ``-inf``,
    everything else becomes 0) and ``diagonal = 1``: ``m[s, t] = -inf`` iff
    ``t - offset > s``.
    """
    s = np.arange(seqlen)[:, None]
    t = np.arange(offset + seqlen)[None, :]
    return np.where(t - offset > s, -np.inf, 0.0).astype(dtype)


def masked_softmax(scores: np.ndarray, offset: int) -> np.ndarray:
    """softmax(scores + mask) over the last axis of ``[b, n, s, t]``.

    The mask is added in the storage dtype before the softmax
    (llama3_70b.py:108-112); adding 0 or -inf is exact.
    """
    b, n, s, t = scores.shape
    assert t == offset + s
    return softmax(scores + causal_mask(s, offset, scores.dtype)[None, None], 3)


def sigmoid(x: np.ndarray) -> np.ndarray:
    """minit/cuda/dispatch.py:143: ``1.0 / (1.0 + expf((float)-x))``, the sum and the
    quotient in double (the literals are doubles), one rounding to the storage type."""
    e = np.exp((-x.astype(np.float32)).astype(np.float32)).astype(np.float32)  # expf: float in, float out
    return (1.0 / (1.0 + e.astype(np.float64))).astype(x.dtype)


def add(x: np.ndarray, y: np.ndarray) -> np.ndarray:
    """minit/cuda/dispatch.py:135: ``{0} + {1}`` in the storage type (one rounding)."""
    return (x.astype(np.float64) + y.astype(np.float64)).astype(x.dtype)


def multiply(x: np.ndarray, y: np.ndarray) -> np.ndarray:
    """minit/cuda/dispatch.py:137: ``{0} * {1}`` in the storage type (one rounding)."""
    return (x.astype(np.float64) * y.astype(np.float64)).astype(x.dtype)


def reduce_sum(x: np.ndarray, axis: int) -> np.ndarray:
    """minit/cuda/kernel/cuda/reduce.py:76-92 with init 0: keepdim sum."""
    return x.astype(np.float64).sum(axis=axis, keepdims=True).astype(x.dtype)


def reduce_mean(x: np.ndarray, axis: int) -> np.ndarray:
    """minit/functional/reduce.py:14-18: ``sum(x) / fill(size)``, the sum rounded to
    the storage type, the length as a tensor of that type, and their quotient by the
    element-wise Divide (minit/cuda/dispatch.py:139, ``{0} / {1}`` in T)."""
    s = reduce_sum(x, axis)
    n = np.asarray(x.shape[axis]).astype(x.dtype)
    return (s.astype(np.float64) / np.float64(n)).astype(x.dtype)


def reduce_max(x: np.ndarray, axis: int) -> np.ndarray:
    """Same kernel with init -inf and max."""
    return x.max(axis=axis, keepdims=True)


def attention_scale(head_size: int) -> float:
    """``qk / sqrt(head_size)``, examples/llama3_70b.py:102."""
    return 1.0 / math.sqrt(head_size)
