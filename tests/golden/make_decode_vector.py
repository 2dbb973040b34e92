"""Writes tests/golden/decode_step.json: one greedy decode step of a tiny
Llama-shaped GPTQ model, worked out with explicit python loops.

The reference ships no outputs for its models and cannot be run here, so the
expected values are not its outputs.  They restate examples/llama3_70b.py
(TransformerBlock.forward :157-162, Attention.forward :77-115, FeedForward.forward
:126-130, Llama3.forward :215-228, Llama3LM.forward :246-249) one scalar at a
time, in python floats (binary64) with exactly summed dot products
(math.fsum), and round to fp16 wherever the reference materialises an fp16
tensor.  Nothing is shared with oracle/ or with the kernels: no numpy
broadcasting, slicing or matrix product takes part in the expected values, so a
slip in the oracle's slices of q|k|v, its head mapping, its residual order or
its choice of norm shows as a mismatch.

Two rows with different positions, two layers, grouped-query attention with two
query heads per KV head, a prefilled cache.

Run from the repository root:  python tests/golden/make_decode_vector.py
"""
import json
import math
import os
import random

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

CFG = dict(n_layers=2, hidden=32, n_q_heads=4, n_kv_heads=2, head_dim=8, ffn=48, vocab=12,
           group_size=16, bits=4, rope_theta=100.0, rms_eps=1e-5, max_seq=8)


def h16(value: float) -> float:
    """One rounding to fp16, returned as a python float."""
    return float(np.float16(value))


def bits16(value: float) -> int:
    return int(np.float16(value).view(np.uint16))


def pack_word(values, bits):
    word = 0
    for i, v in enumerate(values):
        word |= v << (i * bits)
    return word - (1 << 32) if word >= (1 << 31) else word


def make_linear(rng, k, n, group, scale_div):
    q = [[rng.randrange(16) for _ in range(n)] for _ in range(k)]
    z = [[rng.randrange(6, 10) for _ in range(n)] for _ in range(k // group)]
    s = [[h16((abs(rng.gauss(0, 0.02)) + 1e-3) / scale_div) for _ in range(n)] for _ in range(k // group)]
    qweight = [[pack_word([q[r * 8 + i][c] for i in range(8)], 4) for c in range(n)] for r in range(k // 8)]
    qzeros = [[pack_word([z[g][c * 8 + i] for i in range(8)], 4) for c in range(n // 8)] for g in range(k // group)]
    # W = fp16((q - (z + 1)) * s), minit/quantize/dispatch.py:14-20
    w = [[h16((q[kk][c] - (z[kk // group][c] + 1)) * s[kk // group][c]) for c in range(n)] for kk in range(k)]
    return {"qweight": qweight, "qzeros": qzeros, "scales_f16_bits": [[bits16(v) for v in row] for row in s]}, w


def linear(x, w):
    """fp16(sum_k x[k] * W[k][n]) for one row."""
    k, n = len(w), len(w[0])
    return [h16(math.fsum(x[kk] * w[kk][c] for kk in range(k))) for c in range(n)]


def rms_norm(x, weight, eps):
    """fp16(x / sqrt(mean(x^2) + eps) * w), minit/cuda/kernel/cuda/rms_norm.py:69-89 (eps as a float)."""
    mean = math.fsum(v * v for v in x) / len(x)
    rms = math.sqrt(mean + float(np.float32(eps)))
    return [h16(v / rms * w) for v, w in zip(x, weight)]


def rope_head(x, position, head_dim, theta):
    """Interleaved pairs, fp32 tables, minit/cuda/kernel/cuda/rope.py:58-73 + llama3_70b.py:206-212."""
    out = [0.0] * head_dim
    for i in range(head_dim // 2):
        angle = position * (1.0 / theta) ** (2.0 * i / head_dim)
        c, s = float(np.float32(math.cos(angle))), float(np.float32(math.sin(angle)))
        a, b = x[2 * i], x[2 * i + 1]
        out[2 * i] = h16(a * c - b * s)
        out[2 * i + 1] = h16(b * c + a * s)
    return out


def main():
    rng = random.Random(70_2024)
    c = CFG
    hidden, qh, kvh, d, ffn, vocab = c["hidden"], c["n_q_heads"], c["n_kv_heads"], c["head_dim"], c["ffn"], c["vocab"]
    batch = 2
    tokens = [5, 9]
    positions = [3, 1]                      # index of the slot the new entry goes to = number of cached entries
    layers_doc, layers_w = [], []
    for _ in range(c["n_layers"]):
        doc, w = {}, {}
        for name, (k, n) in (("qkv", (hidden, (qh + 2 * kvh) * d)), ("o", (qh * d, hidden)),
                             ("gate_up", (hidden, 2 * ffn)), ("down", (ffn, hidden))):
            doc[name], w[name] = make_linear(rng, k, n, c["group_size"], 1.0)
        for name in ("input_norm", "post_norm"):
            w[name] = [h16(rng.gauss(1, 0.1)) for _ in range(hidden)]
            doc[name + "_f16_bits"] = [bits16(v) for v in w[name]]
        layers_doc.append(doc)
        layers_w.append(w)
    embed = [[h16(rng.gauss(0, 1.0)) for _ in range(hidden)] for _ in range(vocab)]
    lm_head = [[h16(rng.gauss(0, 0.3)) for _ in range(hidden)] for _ in range(vocab)]
    final_norm = [h16(rng.gauss(1, 0.1)) for _ in range(hidden)]
    # caches [layer][b][kv head][t][d]; entries at t >= positions[b] are never read
    k_cache = [[[[[h16(rng.gauss(0, 1)) for _ in range(d)] for _ in range(c["max_seq"])] for _ in range(kvh)]
                for _ in range(batch)] for _ in range(c["n_layers"])]
    v_cache = [[[[[h16(rng.gauss(0, 1)) for _ in range(d)] for _ in range(c["max_seq"])] for _ in range(kvh)]
                for _ in range(batch)] for _ in range(c["n_layers"])]
    k_in = json.loads(json.dumps(k_cache))
    v_in = json.loads(json.dumps(v_cache))

    rep = qh // kvh
    sqrt_d = h16(math.sqrt(d))             # the divisor becomes an fp16 scalar (llama3_70b.py:102)
    logits, new_k, new_v, hidden_after = [], [], [], []
    for b in range(batch):
        p = positions[b]
        h = list(embed[tokens[b]])
        row_k, row_v = [], []
        for l, w in enumerate(layers_w):
            xn = rms_norm(h, w["input_norm"], c["rms_eps"])
            qkv = linear(xn, w["qkv"])
            # q heads first, then k heads, then v heads (q_proj, k_proj, v_proj of llama3_70b.py:80-93)
            q = [rope_head(qkv[j * d:(j + 1) * d], p, d, c["rope_theta"]) for j in range(qh)]
            k_new = [rope_head(qkv[(qh + g) * d:(qh + g + 1) * d], p, d, c["rope_theta"]) for g in range(kvh)]
            v_new = [qkv[(qh + kvh + g) * d:(qh + kvh + g + 1) * d] for g in range(kvh)]
            for g in range(kvh):
                k_cache[l][b][g][p] = k_new[g]
                v_cache[l][b][g][p] = v_new[g]
            row_k.append(k_new)
            row_v.append(v_new)
            attn = []
            for j in range(qh):
                g = j // rep                 # "bs(hd)->bs(hr)d": KV head g serves query heads g*rep .. g*rep+rep-1
                scores = [h16(math.fsum(q[j][i] * k_cache[l][b][g][t][i] for i in range(d))) for t in range(p + 1)]
                scores = [h16(s / sqrt_d) for s in scores]
                top = max(scores)
                e = [math.exp(s - top) for s in scores]
                total = math.fsum(e)
                probs = [h16(v / total) for v in e]
                attn += [h16(math.fsum(probs[t] * v_cache[l][b][g][t][i] for t in range(p + 1))) for i in range(d)]
            o = linear(attn, w["o"])
            h = [h16(a + r) for a, r in zip(h, o)]                       # x + attention_output
            xn = rms_norm(h, w["post_norm"], c["rms_eps"])
            gu = linear(xn, w["gate_up"])
            act = []
            for i in range(ffn):
                gate, up = gu[i], gu[ffn + i]
                sig = h16(1.0 / (1.0 + math.exp(-gate)))                  # F.sigmoid, minit/cuda/dispatch.py:143
                act.append(h16(h16(gate * sig) * up))                     # x * sigmoid(x), then * up
            down = linear(act, w["down"])
            h = [h16(a + r) for a, r in zip(h, down)]
        hidden_after.append([bits16(v) for v in h])
        xn = rms_norm(h, final_norm, c["rms_eps"])
        logits.append([h16(math.fsum(xn[i] * lm_head[t][i] for i in range(hidden))) for t in range(vocab)])
        new_k.append(row_k)
        new_v.append(row_v)

    f16 = lambda nested: json.loads(json.dumps(nested), parse_float=lambda s: bits16(float(s)))  # noqa: E731
    doc = {
        "config": c, "tokens": tokens, "positions": positions, "layers": layers_doc,
        "embed_f16_bits": f16(embed), "lm_head_f16_bits": f16(lm_head), "final_norm_f16_bits": f16(final_norm),
        "k_cache_f16_bits": f16(k_in), "v_cache_f16_bits": f16(v_in),
        "expected": {
            "logits_f16_bits": f16(logits), "hidden_f16_bits": hidden_after,
            "argmax": [max(range(vocab), key=lambda t: row[t]) for row in logits],
            # appended cache rows [b][layer][kv head][d]
            "new_k_f16_bits": f16(new_k), "new_v_f16_bits": f16(new_v),
        },
    }
    path = os.path.join(HERE, "decode_step.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
