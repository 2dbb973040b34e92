"""Writes tests/golden/kat.json: small known-answer vectors for the hot path.

The reference ships no tests or fixtures, and it cannot be run in this
environment, so these vectors are not its outputs: every expected value below is
derived by exact arithmetic on small integers and rationals (python ints and
fractions.Fraction, rounded once where the reference rounds once), written out
with explicit loops that share no code with oracle/ or with the kernels.  They
pin the oracle (CPU tests) and the HIP path (GPU tests) to the same answers.

Formulas restated: sub-word i of a word at bit i * bits
(examples/qwen1_5_int8.py:107-116,129-136); W = fp16((q - (z + 1)) * s)
(minit/quantize/dispatch.py:14-20); y = x[M,K] @ W[K,N]; int8 product with int32
accumulation and fp16(fp32(acc) * (a_scale * w_scale)); the special cases of
RMSNorm / RoPE / softmax / reductions where the closed form is exact
(minit/cuda/kernel/cuda/{rms_norm,rope,softmax,reduce}.py).

Run from the repository root:  python tests/golden/make_vectors.py
"""
import json
import os
import random
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f16_bits(value) -> int:
    return int(np.float16(value).view(np.uint16))


def f16_from_bits(bits: int) -> float:
    return float(np.uint16(bits).view(np.float16))


def round_fraction_to_f16(fr: Fraction) -> int:
    """One correct rounding of an exact rational to fp16 (bit pattern).  The
    rationals used here fit a double exactly, so double -> half rounds once."""
    as_double = float(fr)
    assert Fraction(as_double) == fr, "value does not fit a double exactly"
    return f16_bits(as_double)


def round_signed_sqrt_to_f16(sign: int, square: Fraction) -> float:
    """The fp16 value nearest to sign * sqrt(square), decided exactly: the candidate from double
    arithmetic is accepted only if the squares of the two midpoints to its fp16 neighbours
    bracket `square` (compared as rationals)."""
    cand = np.float16(float(square) ** 0.5)
    lo = Fraction(float(np.nextafter(cand, np.float16(0)))) + Fraction(float(cand))
    hi = Fraction(float(np.nextafter(cand, np.float16(np.inf)))) + Fraction(float(cand))
    assert (lo / 2) ** 2 < square < (hi / 2) ** 2, "candidate is not the nearest fp16 value"
    return sign * float(cand)


def pack_words(values, bits):
    """values: list of 32 // bits sub-words -> one signed 32-bit word."""
    word = 0
    for i, v in enumerate(values):
        assert 0 <= v < (1 << bits)
        word |= v << (i * bits)
    return word - (1 << 32) if word >= (1 << 31) else word


def gptq_case(rng, m, k, n, group, bits):
    per_word = 32 // bits
    q = [[rng.randrange(1 << bits) for _ in range(n)] for _ in range(k)]
    z = [[rng.randrange(1 << bits) for _ in range(n)] for _ in range(k // group)]
    # include the corners: zero point at its maximum (z + 1 must not wrap) and q == z + 1 (weight 0)
    z[0][0] = (1 << bits) - 1
    q[0][1] = min(z[0][1] + 1, (1 << bits) - 1)
    s_bits = [[f16_bits(abs(rng.gauss(0, 0.02)) + 1e-3) for _ in range(n)] for _ in range(k // group)]
    x_bits = [[f16_bits(rng.gauss(0, 1)) for _ in range(k)] for _ in range(m)]
    qweight = [[pack_words([q[r * per_word + i][c] for i in range(per_word)], bits) for c in range(n)]
               for r in range(k // per_word)]
    qzeros = [[pack_words([z[g][c * per_word + i] for i in range(per_word)], bits) for c in range(n // per_word)]
              for g in range(k // group)]
    w_bits = [[0] * n for _ in range(k)]
    w_exact = [[Fraction(0)] * n for _ in range(k)]
    for kk in range(k):
        g = kk // group
        for c in range(n):
            prod = Fraction(q[kk][c] - (z[g][c] + 1)) * Fraction(f16_from_bits(s_bits[g][c]))
            w_bits[kk][c] = round_fraction_to_f16(prod)
            w_exact[kk][c] = Fraction(f16_from_bits(w_bits[kk][c]))
    y = [[float(sum(Fraction(f16_from_bits(x_bits[r][kk])) * w_exact[kk][c] for kk in range(k))) for c in range(n)]
         for r in range(m)]
    return {"m": m, "k": k, "n": n, "group_size": group, "bits": bits, "q": q, "z": z, "qweight": qweight,
            "qzeros": qzeros, "scales_f16_bits": s_bits, "x_f16_bits": x_bits, "w_f16_bits": w_bits,
            "y_exact": y}


def int8_case(rng, m, n, k):
    a = [[rng.randrange(-127, 128) for _ in range(k)] for _ in range(m)]
    w = [[rng.randrange(-127, 128) for _ in range(k)] for _ in range(n)]
    a[0] = [-128] * k          # extremes: (-128) * (-128) * k and its negative
    w[0] = [-128] * k
    w[1] = [127] * k
    acc = [[sum(a[i][t] * w[j][t] for t in range(k)) for j in range(n)] for i in range(m)]
    assert all(-2**31 <= v < 2**31 for row in acc for v in row)
    a_scale = [float(np.float32(abs(rng.gauss(0, 0.01)) + 1e-4)) for _ in range(m)]
    w_scale = [float(np.float32(abs(rng.gauss(0, 0.005)) + 1e-4)) for _ in range(n)]
    out_bits = [[0] * n for _ in range(m)]
    for i in range(m):
        for j in range(n):
            scale = np.float32(a_scale[i]) * np.float32(w_scale[j])      # one fp32 rounding
            prod = np.float32(acc[i][j]) * scale                         # int -> fp32, then one fp32 rounding
            out_bits[i][j] = f16_bits(prod)                              # one fp16 rounding
    return {"m": m, "n": n, "k": k, "a": a, "w_nk": w, "acc": acc, "a_scale": a_scale, "w_scale": w_scale,
            "out_f16_bits": out_bits}


def special_cases():
    cases = {}
    # RMSNorm of a constant row c: c / sqrt(c^2 + eps) * w = sign(c) * w * (1 - eps / (2 c^2) ...); with
    # eps = 1e-6 the factor is within 1e-5 of 1, far inside half an fp16 step (2.4e-4), so the fp16 result is +-w
    w = [0.5, -1.25, 2.0, 1.0, 0.75, -3.0, 1.5, 0.125]
    cases["rms_norm_constant_rows"] = {
        "x": [[3.0] * 8, [-0.25] * 8], "weight": w, "eps": 1e-6,
        "out": [w, [-v for v in w]],
    }
    # RMSNorm where eps decides the answer: a constant row c with eps = c^2 normalises to sign(c) * w / sqrt(2),
    # and c = 3 * 2^-10 with the same eps to w * 3 / sqrt(10); eps left out gives +-w, eps added outside the
    # square root gives w * c / (|c| + eps) = 0.999 w.  out^2 = w^2 c^2 / (c^2 + eps), rounded to fp16 exactly.
    c0, eps = Fraction(1, 1024), Fraction(1, 1 << 20)
    rows = [c0, -c0, 3 * c0]
    cases["rms_norm_eps_rows"] = {
        "x": [[float(c)] * 8 for c in rows], "weight": w, "eps": float(eps),
        "out": [[round_signed_sqrt_to_f16((1 if c > 0 else -1) * (1 if v > 0 else -1),
                                          Fraction(v) ** 2 * c * c / (c * c + eps)) for v in w] for c in rows],
    }
    # softmax: uniform row of 8 -> 1/8; -inf entries -> exactly 0, the rest uniform
    ninf = "-inf"
    cases["softmax_rows"] = {
        "x": [[1.5] * 8, [2.0, ninf, 2.0, ninf, ninf, 2.0, 2.0, ninf], [ninf] * 7 + [-7.0]],
        "out": [[0.125] * 8, [0.25, 0.0, 0.25, 0.0, 0.0, 0.25, 0.25, 0.0], [0.0] * 7 + [1.0]],
    }
    # causal mask, s = 3 new rows on offset 2: row i sees t <= offset + i; equal scores -> uniform over the visible
    cases["softmax_causal"] = {
        "rows": 3, "t": 5, "offset": 2, "scale": 1.0, "score": 0.5,
        "out": [[1 / 3, 1 / 3, 1 / 3, 0.0, 0.0], [0.25, 0.25, 0.25, 0.25, 0.0], [0.2] * 5],
    }
    # RoPE: (cos, sin) = (1, 0) is the identity, (0, 1) maps (a, b) to (-b, a), (-1, 0) negates
    x = [1.0, 2.0, -3.0, 4.0, 0.5, -0.25]
    cases["rope_quarter_turns"] = {
        "x": x, "cos": [1.0, 0.0, -1.0], "sin": [0.0, 1.0, 0.0],
        "out": [1.0, 2.0, -4.0, -3.0, -0.5, 0.25],
    }
    # reductions over the middle axis of [2, 4, 3]
    t = [[[1, -2, 3], [4, 5, -6], [-7, 8, 9], [10, -11, 12]], [[0.5, 0.25, 0], [1, 1, 1], [-1, -1, -1], [2, 4, 8]]]
    cases["reduce_middle_axis"] = {
        "x": t,
        "sum": [[[8, 0, 18]], [[2.5, 4.25, 8]]],
        "max": [[[10, 8, 12]], [[2, 4, 8]]],
        # mean = sum / 4 (the reference divides the rounded sum by the rounded length: both exact here)
        "mean": [[[2, 0, 4.5]], [[0.625, 1.0625, 2]]],
    }
    # mean where the roundings show: 2049 ones sum to 2049, which fp16 rounds to 2048 (ties to even), and the
    # length 2049 rounds to 2048 as well: 2048 / 2048 = 1; 2050 halves: sum 1025, length 2050 -> 0.5
    cases["mean_roundings"] = {"ones": 2049, "ones_mean": 1.0, "halves": 2050, "halves_mean": 0.5}
    # the two element-wise kernels of the models' silu: sigmoid(0) = 1 / (1 + 1) = 0.5; products rounded once:
    # (1 + 2^-10)^2 = 1 + 2^-9 + 2^-20 -> 1 + 2^-9; 3 * 0.333251953125 = 0.999755859375 -> 1.0 (tie to even)
    cases["elementwise"] = {
        "sigmoid_in": [0.0], "sigmoid_out": [0.5],
        "a": [1.0009765625, 3.0, -0.5, 0.0], "b": [1.0009765625, 0.333251953125, 0.5, -7.0],
        "product": [1.001953125, 1.0, -0.25, -0.0],
    }
    # silu(g) * u with the three fp16 roundings of the models (sigmoid, g * sigmoid, * u) at g = 0: 0 * 0.5 = 0
    cases["silu_mul_zero_gate"] = {"gate": [0.0, 0.0], "up": [3.0, -2.0], "out": [0.0, -0.0]}
    return cases


def main():
    rng = random.Random(20240611)
    doc = {
        "gptq": [gptq_case(rng, 2, 64, 8, 32, 4), gptq_case(rng, 1, 64, 8, 32, 8), gptq_case(rng, 3, 256, 16, 128, 4)],
        "int8": [int8_case(rng, 3, 5, 64), int8_case(rng, 2, 4, 128)],
        "special": special_cases(),
    }
    path = os.path.join(HERE, "kat.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
