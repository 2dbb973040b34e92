"""Seeded synthetic inputs for the benchmark configurations.

One ``numpy.random.Generator(PCG64(seed))`` per tensor, the seed derived from
(configuration, tensor name), so any tensor can be regenerated on its own.
Recipes: 4-bit weights uniform in [0, 15] packed 8 per int32 along K; zero
points uniform in [6, 9] packed along N; scales fp16 ``|N(0, 0.02)| + 1e-3``;
activations fp16 ``N(0, 1)``; int8 operands uniform in [-127, 127] with
per-token scale ``|N(0, 0.01)|`` and per-channel scale ``|N(0, 0.005)|``.
"""
import zlib

import numpy as np

from .quantize.gptq import pack_subwords


def rng(config: str, name: str) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(zlib.crc32(f"{config}/{name}".encode())))


def gptq_weights(config: str, name: str, k: int, n: int, group_size: int = 128, bits: int = 4,
                 zero_range=(6, 9)):
    """Returns ``(qweight, qzeros, scales)`` in the GPTQ checkpoint layout."""
    per_word = 32 // bits
    groups = k // group_size
    if bits == 4:
        # random words are uniform nibbles
        qweight = rng(config, name + ".qweight").integers(0, 1 << 32, size=(k // per_word, n), dtype=np.uint64)
        qweight = qweight.astype(np.uint32).view(np.int32)
    else:
        q = rng(config, name + ".qweight").integers(0, 1 << bits, size=(k, n), dtype=np.uint8)
        qweight = pack_subwords(q, 0, bits)
    z = rng(config, name + ".qzeros").integers(zero_range[0], zero_range[1] + 1, size=(groups, n), dtype=np.uint8)
    qzeros = pack_subwords(z, 1, bits)
    s = np.abs(rng(config, name + ".scales").normal(0.0, 0.02, size=(groups, n))) + 1e-3
    return qweight, qzeros, s.astype(np.float16)


def activations(config: str, name: str, shape, std: float = 1.0) -> np.ndarray:
    return rng(config, name).normal(0.0, std, size=shape).astype(np.float16)


def int8_operands(config: str, m: int, n: int, k: int):
    """``(A [M,K], W [N,K], a_scale [M], w_scale [N])`` for the W8A8 GEMM."""
    a = rng(config, "A").integers(-127, 128, size=(m, k), dtype=np.int8)
    w = rng(config, "W").integers(-127, 128, size=(n, k), dtype=np.int8)
    a_scale = np.abs(rng(config, "a_scale").normal(0.0, 0.01, size=m)).astype(np.float32)
    w_scale = np.abs(rng(config, "w_scale").normal(0.0, 0.005, size=n)).astype(np.float32)
    return a, w, a_scale, w_scale


def rope_tables(head_size: int, nr_positions: int, theta: float):
    """fp32 cos / sin tables ``[nr_positions, head_size/2]``; same recipe as the
    models (examples/llama3_70b.py:206-212), evaluated in float64 on the host."""
    i = np.arange(head_size // 2, dtype=np.float64)
    freqs = (1.0 / theta) ** (2.0 * i / head_size)
    ang = np.arange(nr_positions, dtype=np.float64)[:, None] * freqs[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
