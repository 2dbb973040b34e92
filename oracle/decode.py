"""One greedy decode step of the reference's Llama-family models on the CPU.

Test infrastructure only.  Follows examples/llama3_70b.py:77-162,215-249 op by
op, rounding to fp16 wherever the reference materialises an fp16 tensor:
RMSNorm (eps from the model), q/k/v projections, interleaved RoPE at the row's
position, K/V appended to the cache, scores = q.k^T (fp32 accumulate, fp16
store), ``/ sqrt(d)`` in fp16, the additive causal mask (identically zero for a
single new token), softmax, P.V, output projection, residual adds in fp16,
``silu(gate) * up`` with its three roundings, and the lm_head product against
``[vocab, hidden]``; sampling is ``argmax`` (minit/chat/sample.py:11-14).

Every linear may carry a bias and an act-order ``g_idx`` (the reference's own GPTQ model,
examples/qwen1_5_int8.py:311-385, where gate is ``w2`` and up is ``w1``).

Grouped-query attention: query head j uses KV head ``j // (QH / KVH)``
(the reference repeats each KV head, llama3_70b.py:85-93).

Pinned by tests/test_oracle_decode.py: a known-answer step worked out scalar by
scalar (tests/golden/decode_step.json) and models whose projections are exact
zeros, identities or channel selections, for which the step has a closed form.
"""
import numpy as np

from . import gptq, special


def split_linear(w):
    """``w`` is ``(qweight, qzeros, scales, group_size[, bias[, g_idx]])``: the buffers of the reference's
    QLinear / QLinearWithBias (examples/qwen1_5_int8.py:276-305); ``bias`` and ``g_idx`` may be None."""
    qweight, qzeros, scales, group_size = w[:4]
    bias = w[4] if len(w) > 4 else None
    g_idx = w[5] if len(w) > 5 else None
    return qweight, qzeros, scales, group_size, bias, g_idx


def add_bias(y, bias):
    """``output += bias`` of QLinearWithBias.forward (examples/qwen1_5_int8.py:311-317): an fp16 add of the
    fp16 product and the bias broadcast over the rows, one more rounding."""
    return y if bias is None else (y + bias[None, :].astype(y.dtype))


def _linear(x, w, bits=4):
    """The quantized linear of the model code: the product (act-order ``g_idx`` included), then the bias."""
    qweight, qzeros, scales, group_size, bias, g_idx = split_linear(w)
    return add_bias(gptq.matmul(x, qweight, qzeros, scales, g_idx, bits, group_size), bias)


def attention(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, positions: np.ndarray) -> np.ndarray:
    """Attention of one new token per row over its cache, examples/llama3_70b.py:95-113.

    ``q [B, QH, D]``, caches ``[B, KVH, T, D]`` with the newest entry at
    ``positions[b]``; query head j reads KV head ``j // (QH / KVH)``.  Rounded to
    fp16 where the reference holds an fp16 tensor: the scores, their division by
    ``sqrt(D)``, the probabilities and the result.  The additive causal mask is zero
    for a single new token.
    """
    b, qh, d = q.shape
    rep = qh // k_cache.shape[1]
    sqrt_d = np.float16(np.sqrt(np.float64(d)))
    out = np.zeros((b, qh, d), np.float16)
    for i in range(b):
        p = int(positions[i])
        kk = k_cache[i, :, :p + 1].astype(np.float64)                  # [KVH, T, D]
        vv = v_cache[i, :, :p + 1].astype(np.float64)
        for j in range(qh):
            g = j // rep
            scores = (kk[g] @ q[i, j].astype(np.float64)).astype(np.float16)
            scores = (scores / sqrt_d).astype(np.float16)              # fp16 division
            probs = special.softmax(scores[None, :], 1)[0]
            out[i, j] = (probs.astype(np.float64) @ vv[g]).astype(np.float16)
    return out


def decode_step(model: dict, tokens: np.ndarray, positions: np.ndarray, k_cache: list, v_cache: list,
                linear=None):
    """Returns fp16 logits ``[B, vocab]``; caches ``[B, KVH, T, D]`` are updated in place.

    ``linear(x, (qweight, qzeros, scales, group_size), bits)`` replaces the numpy quantized
    product (full-width layers use the C restatement, which is held bit-exact to it)."""
    _linear = linear or globals()["_linear"]
    cfg = model["config"]
    qh, kvh, d = cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    rep = qh // kvh
    eps = cfg["rms_eps"]
    bits = cfg.get("bits", 4)
    b = len(tokens)
    h = model["embed"][tokens].astype(np.float16)                      # [B, H]
    cos, sin = model["cos"], model["sin"]
    inv_sqrt_d = np.float16(np.sqrt(np.float64(d)))
    for l, layer in enumerate(model["layers"]):
        xn = special.rms_norm(h, layer["input_norm"], 1, eps)
        qkv = _linear(xn, layer["qkv"], bits)
        q = qkv[:, :qh * d].reshape(b, 1, qh, d)
        k = qkv[:, qh * d:(qh + kvh) * d].reshape(b, 1, kvh, d)
        v = qkv[:, (qh + kvh) * d:].reshape(b, kvh, d)
        pos = positions.reshape(b, 1)
        q = special.rope(q, cos, sin, pos)[:, 0]                       # [B, QH, D]
        k = special.rope(k, cos, sin, pos)[:, 0]                       # [B, KVH, D]
        for i in range(b):
            p = int(positions[i])
            k_cache[l][i, :, p] = k[i]
            v_cache[l][i, :, p] = v[i]
        attn = attention(q, k_cache[l], v_cache[l], positions)
        o = _linear(attn.reshape(b, qh * d), layer["o"], bits)
        h = h + o                                                      # fp16 add
        xn = special.rms_norm(h, layer["post_norm"], 1, eps)
        gu = _linear(xn, layer["gate_up"], bits)
        f = gu.shape[1] // 2
        act = gptq.silu_mul(gu[:, :f], gu[:, f:])
        h = h + _linear(act, layer["down"], bits)
    xn = special.rms_norm(h, model["final_norm"], 1, eps)
    return gptq.dense_matmul(xn, model["lm_head"].T.astype(np.float16))


def greedy(model, tokens, positions, k_cache, v_cache, n_steps, linear=None):
    """Returns ``(out_tokens [n_steps, B], logits of every step)``."""
    tokens = np.array(tokens, np.int64)
    positions = np.array(positions, np.int64)
    out, all_logits = [], []
    for _ in range(n_steps):
        logits = decode_step(model, tokens, positions, k_cache, v_cache, linear)
        tokens = logits.astype(np.float32).argmax(axis=-1)
        positions = positions + 1
        out.append(tokens.copy())
        all_logits.append(logits)
    return np.stack(out), all_logits
