"""Pins ``oracle.decode.decode_step`` / ``greedy``, the checker of every decode
test on the GPU.

The reference holds no output of its models, so the composed step is pinned by

* a known-answer vector (tests/golden/decode_step.json, worked out scalar by
  scalar with python floats by tests/golden/make_decode_vector.py, sharing no
  code with the oracle): logits and the appended cache rows bit for bit;
* models built so that the mathematics fixes the answer: projections that are
  exactly zero (``q == z + 1``), exactly the identity or a selection of input
  channels (``q == z + 2`` on chosen entries, scale 1), norm weights that are
  zero.  Each one makes a different slip visible: a wrong q|k|v slice, a wrong
  KV head for a query head, RoPE at the wrong position, the wrong norm in
  front of a projection, gate and up exchanged, the residual taken from the
  wrong tensor, lm_head transposed, tokens or positions not fed back.
"""
import json
import math
import os

import numpy as np
from oracle import decode as OD
from oracle import gptq as OG
from oracle import special as OS

HERE = os.path.dirname(os.path.abspath(__file__))


def _f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16)


# ------------------------------------------------------------------ known-answer vector

def _kat_model():
    doc = json.load(open(os.path.join(HERE, "golden", "decode_step.json")))
    cfg = doc["config"]
    layers = []
    for l in doc["layers"]:
        layer = {name: (np.asarray(l[name]["qweight"], np.int32), np.asarray(l[name]["qzeros"], np.int32),
                        _f16(l[name]["scales_f16_bits"]), cfg["group_size"])
                 for name in ("qkv", "o", "gate_up", "down")}
        layer["input_norm"] = _f16(l["input_norm_f16_bits"])
        layer["post_norm"] = _f16(l["post_norm_f16_bits"])
        layers.append(layer)
    cos, sin = OS.rope_tables(cfg["head_dim"], cfg["max_seq"], cfg["rope_theta"])
    model = {"config": cfg, "layers": layers, "embed": _f16(doc["embed_f16_bits"]),
             "lm_head": _f16(doc["lm_head_f16_bits"]), "final_norm": _f16(doc["final_norm_f16_bits"]),
             "cos": cos, "sin": sin}
    return doc, model


def test_decode_step_known_answer():
    doc, model = _kat_model()
    cfg = doc["config"]
    k_cache = [_f16(c).copy() for c in doc["k_cache_f16_bits"]]      # [B, KVH, T, D] per layer
    v_cache = [_f16(c).copy() for c in doc["v_cache_f16_bits"]]
    before = [c.copy() for c in k_cache + v_cache]
    tokens, positions = np.asarray(doc["tokens"]), np.asarray(doc["positions"])
    logits = OD.decode_step(model, tokens, positions, k_cache, v_cache)
    exp = doc["expected"]
    assert logits.dtype == np.float16
    np.testing.assert_array_equal(logits.view(np.uint16), np.asarray(exp["logits_f16_bits"], np.uint16))
    assert logits.astype(np.float32).argmax(-1).tolist() == exp["argmax"]
    new_k, new_v = _f16(exp["new_k_f16_bits"]), _f16(exp["new_v_f16_bits"])   # [B, layer, KVH, D]
    for l in range(cfg["n_layers"]):
        for b, p in enumerate(positions):
            np.testing.assert_array_equal(k_cache[l][b, :, p].view(np.uint16), new_k[b, l].view(np.uint16))
            np.testing.assert_array_equal(v_cache[l][b, :, p].view(np.uint16), new_v[b, l].view(np.uint16))
            # nothing else in the cache moves
            for cache, old in ((k_cache[l], before[l]), (v_cache[l], before[cfg["n_layers"] + l])):
                keep = np.ones(cfg["max_seq"], bool)
                keep[p] = False
                np.testing.assert_array_equal(cache[b][:, keep].view(np.uint16), old[b][:, keep].view(np.uint16))


# ------------------------------------------------------------------ constructed models

H, QH, KVH, D, FFN, G = 64, 4, 2, 16, 64, 32           # hidden == QH * D == FFN == vocab where identities are needed
CFG = dict(n_layers=1, hidden=H, n_q_heads=QH, n_kv_heads=KVH, head_dim=D, ffn=FFN, vocab=H,
           group_size=G, bits=4, rope_theta=1e4, rms_eps=1e-5)
THETA = 1e4


def _linear_from_ints(w_int, scale=1.0):
    """GPTQ tensors whose dequantized matrix is exactly ``w_int * scale`` (zero point 7, so
    ``q - (z + 1) = q - 8``; entries in [-8, 7])."""
    w_int = np.asarray(w_int)
    k, n = w_int.shape
    assert w_int.min() >= -8 and w_int.max() <= 7
    qweight = OG.pack((w_int + 8).astype(np.uint8), 0, 4)
    qzeros = OG.pack(np.full((k // G, n), 7, np.uint8), 1, 4)
    scales = np.full((k // G, n), scale, np.float16)
    return (qweight, qzeros, scales, G)


def _random_linear(rng, k, n):
    return _linear_from_ints(rng.integers(-8, 8, (k, n)), 0.03)


def _zeros(k, n):
    return _linear_from_ints(np.zeros((k, n), np.int64))


def _eye(n, factor=1):
    return _linear_from_ints(np.eye(n, dtype=np.int64) * factor)


def _model(rng, **layer_overrides):
    layer = {"qkv": _random_linear(rng, H, (QH + 2 * KVH) * D), "o": _random_linear(rng, QH * D, H),
             "gate_up": _random_linear(rng, H, 2 * FFN), "down": _random_linear(rng, FFN, H),
             "input_norm": rng.normal(1, 0.2, H).astype(np.float16),
             "post_norm": rng.normal(1, 0.2, H).astype(np.float16)}
    layer.update(layer_overrides)
    cos, sin = OS.rope_tables(D, 32, THETA)
    return {"config": dict(CFG), "layers": [layer],
            "embed": rng.normal(0, 1, (H, H)).astype(np.float16),
            "lm_head": np.eye(H, dtype=np.float16),                     # logits = final-normed hidden state
            "final_norm": np.ones(H, np.float16), "cos": cos, "sin": sin}


def _caches(rng, batch, t=32):
    shape = (batch, KVH, t, D)
    return [rng.normal(0, 1, shape).astype(np.float16)], [rng.normal(0, 1, shape).astype(np.float16)]


def _norm(x, w, eps=1e-5):
    """fp16(x / sqrt(mean x^2 + eps) * w) of one row, in python floats."""
    x = [float(v) for v in x]
    rms = math.sqrt(math.fsum(v * v for v in x) / len(x) + float(np.float32(eps)))
    return np.asarray([np.float16(v / rms * float(wi)) for v, wi in zip(x, w)], np.float16)


def _logits_from_hidden(h):
    """lm_head = identity, final norm weight 1."""
    return _norm(h, np.ones(len(h)))


def _add16(a, b):
    return (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)


def test_layers_that_add_nothing_leave_lm_head_of_the_normed_embedding():
    """o and down exactly zero: h stays embed[token]; logits[v] = sum_h norm(h)[h] * lm_head[v, h]."""
    rng = np.random.default_rng(1)
    model = _model(rng, o=_zeros(QH * D, H), down=_zeros(FFN, H))
    vocab = 24
    model["lm_head"] = rng.normal(0, 0.3, (vocab, H)).astype(np.float16)    # [vocab, hidden], not square
    model["final_norm"] = rng.normal(1, 0.2, H).astype(np.float16)
    tokens, positions = np.array([3, 17, 40]), np.array([5, 0, 9])
    k, v = _caches(rng, 3)
    logits = OD.decode_step(model, tokens, positions, k, v)
    assert logits.shape == (3, vocab)
    for b, t in enumerate(tokens):
        xn = _norm(model["embed"][t], model["final_norm"])
        want = [np.float16(math.fsum(float(xn[i]) * float(model["lm_head"][j, i]) for i in range(H)))
                for j in range(vocab)]
        np.testing.assert_array_equal(logits[b], np.asarray(want, np.float16))


def _selecting_qkv(rng):
    """q columns random; k head g, dim i <- input channel 32 + g*16 + i; v head g, dim i <- channel g*16 + i."""
    w = rng.integers(-8, 8, (H, (QH + 2 * KVH) * D))
    w[:, QH * D:] = 0
    for g in range(KVH):
        for i in range(D):
            w[32 + g * D + i, (QH + g) * D + i] = 1
            w[g * D + i, (QH + KVH + g) * D + i] = 1
    return w


def test_single_visible_entry_returns_the_value_row_of_the_shared_kv_head():
    """Position 0: the only visible entry is the appended one, softmax over one score is 1, so query
    head j returns the new v row of KV head j // 2 whatever q is.  With v selecting channels of the
    normed input, o the identity and down zero: h = embed + [v0, v0, v1, v1]."""
    rng = np.random.default_rng(2)
    model = _model(rng, qkv=_linear_from_ints(_selecting_qkv(rng)), o=_eye(H), down=_zeros(FFN, H))
    layer = model["layers"][0]
    tokens, positions = np.array([7, 21]), np.array([0, 0])
    k, v = _caches(rng, 2)
    logits = OD.decode_step(model, tokens, positions, k, v)
    for b, t in enumerate(tokens):
        e = model["embed"][t]
        xn = _norm(e, layer["input_norm"])
        v_heads = [xn[g * D:(g + 1) * D] for g in range(KVH)]
        attn = np.concatenate([v_heads[j // (QH // KVH)] for j in range(QH)])
        np.testing.assert_array_equal(logits[b], _logits_from_hidden(_add16(e, attn)))
        # the appended rows: v as selected, k = the selected channels (RoPE at position 0 is the identity)
        np.testing.assert_array_equal(v[0][b, :, 0].reshape(-1), xn[:KVH * D])
        np.testing.assert_array_equal(k[0][b, :, 0].reshape(-1), xn[32:32 + KVH * D])


def test_appended_keys_are_rotated_at_the_row_s_own_position():
    rng = np.random.default_rng(3)
    model = _model(rng, qkv=_linear_from_ints(_selecting_qkv(rng)))
    layer = model["layers"][0]
    tokens, positions = np.array([1, 2, 3]), np.array([11, 4, 30])
    k, v = _caches(rng, 3)
    k_before = k[0].copy()
    OD.decode_step(model, tokens, positions, k, v)
    for b, (t, p) in enumerate(zip(tokens, positions)):
        xn = _norm(model["embed"][t], layer["input_norm"])
        for g in range(KVH):
            src = xn[32 + g * D:32 + (g + 1) * D].astype(np.float64)
            for i in range(D // 2):
                ang = float(p) * THETA ** (-2.0 * i / D)
                c, s = float(np.float32(math.cos(ang))), float(np.float32(math.sin(ang)))
                want = (np.float16(src[2 * i] * c - src[2 * i + 1] * s), np.float16(src[2 * i + 1] * c + src[2 * i] * s))
                assert (k[0][b, g, p, 2 * i], k[0][b, g, p, 2 * i + 1]) == want
        others = np.arange(32) != p
        np.testing.assert_array_equal(k[0][b][:, others], k_before[b][:, others])


def test_zero_input_norm_gives_the_mean_of_the_visible_values():
    """input_norm = 0: q = k = v = 0, all scores equal, so every head returns the mean of its KV head's
    visible value rows (the appended zero row included).  post_norm = 0 silences the feed-forward
    whatever its weights are: silu(0) * 0 = 0."""
    rng = np.random.default_rng(4)
    model = _model(rng, o=_eye(H), input_norm=np.zeros(H, np.float16), post_norm=np.zeros(H, np.float16))
    tokens, positions = np.array([9, 33]), np.array([3, 6])
    k, v = _caches(rng, 2)
    v_before = v[0].copy()
    logits = OD.decode_step(model, tokens, positions, k, v)
    for b, (t, p) in enumerate(zip(tokens, positions)):
        heads = []
        for j in range(QH):
            g = j // (QH // KVH)
            prob = float(np.float16(1.0 / (p + 1)))                       # probabilities are an fp16 tensor
            rows = [v_before[b, g, s].astype(np.float64) for s in range(p)] + [np.zeros(D)]
            heads.append(np.asarray([np.float16(math.fsum(prob * r[i] for r in rows)) for i in range(D)], np.float16))
        h = _add16(model["embed"][t], np.concatenate(heads))
        np.testing.assert_array_equal(logits[b], _logits_from_hidden(h))


def test_feed_forward_takes_post_norm_and_gate_before_up():
    """o zero, gate selects channel i, up selects channel i times 2, down the identity:
    h = embed + fp16(fp16(g * fp16(sigmoid(g))) * 2g) with g = norm(embed, post_norm)."""
    rng = np.random.default_rng(5)
    gate_up = np.concatenate([np.eye(H, dtype=np.int64), 2 * np.eye(H, dtype=np.int64)], axis=1)
    model = _model(rng, o=_zeros(QH * D, H), gate_up=_linear_from_ints(gate_up), down=_eye(FFN))
    layer = model["layers"][0]
    tokens, positions = np.array([12]), np.array([2])
    k, v = _caches(rng, 1)
    logits = OD.decode_step(model, tokens, positions, k, v)
    e = model["embed"][12]
    g = _norm(e, layer["post_norm"])
    act = []
    for gi in g:
        sig = np.float16(1.0 / (1.0 + math.exp(-float(gi))))
        act.append(np.float16(float(np.float16(float(gi) * float(sig))) * float(np.float16(2 * float(gi)))))
    np.testing.assert_array_equal(logits[0], _logits_from_hidden(_add16(e, np.asarray(act, np.float16))))
    # and it is the post-attention norm, not the input norm, that feeds it
    assert not np.array_equal(g, _norm(e, layer["input_norm"]))


def test_second_residual_adds_to_the_attention_output_sum():
    """o the identity and down the identity on a selecting gate/up: both residual adds stack,
    h = fp16(fp16(embed + attn) + ffn(norm(embed + attn)))."""
    rng = np.random.default_rng(6)
    gate_up = np.concatenate([np.eye(H, dtype=np.int64), np.eye(H, dtype=np.int64)], axis=1)
    model = _model(rng, qkv=_linear_from_ints(_selecting_qkv(rng)), o=_eye(H),
                   gate_up=_linear_from_ints(gate_up), down=_eye(FFN))
    layer = model["layers"][0]
    k, v = _caches(rng, 1)
    logits = OD.decode_step(model, np.array([30]), np.array([0]), k, v)
    e = model["embed"][30]
    xn = _norm(e, layer["input_norm"])
    attn = np.concatenate([xn[(j // 2) * D:(j // 2 + 1) * D] for j in range(QH)])
    h1 = _add16(e, attn)
    g = _norm(h1, layer["post_norm"])
    act = np.asarray([np.float16(float(np.float16(float(x) * float(np.float16(1.0 / (1.0 + math.exp(-float(x)))))))
                                 * float(x)) for x in g], np.float16)
    np.testing.assert_array_equal(logits[0], _logits_from_hidden(_add16(h1, act)))


def test_rows_are_independent_and_permute_with_their_caches():
    rng = np.random.default_rng(7)
    model = _model(rng)
    tokens, positions = np.array([4, 50, 23, 8]), np.array([7, 0, 19, 12])
    k, v = _caches(rng, 4)
    perm = np.array([2, 0, 3, 1])
    k2, v2 = [k[0][perm].copy()], [v[0][perm].copy()]
    a = OD.decode_step(model, tokens, positions, k, v)
    b = OD.decode_step(model, tokens[perm], positions[perm], k2, v2)
    np.testing.assert_array_equal(a[perm], b)
    np.testing.assert_array_equal(k[0][perm], k2[0])
    # a row alone gives what it gives in the batch
    rng = np.random.default_rng(7)
    model = _model(rng)
    kk, vv = _caches(rng, 4)
    single = OD.decode_step(model, tokens[2:3], positions[2:3], [kk[0][2:3].copy()], [vv[0][2:3].copy()])
    np.testing.assert_array_equal(single[0], a[2])


def test_entries_past_the_position_are_not_read():
    rng = np.random.default_rng(8)
    model = _model(rng)
    k, v = _caches(rng, 1)
    k2, v2 = [k[0].copy()], [v[0].copy()]
    k2[0][:, :, 6:] = 99.0
    v2[0][:, :, 6:] = -99.0
    a = OD.decode_step(model, np.array([3]), np.array([5]), k, v)
    b = OD.decode_step(model, np.array([3]), np.array([5]), k2, v2)
    np.testing.assert_array_equal(a, b)


def test_greedy_feeds_tokens_and_positions_back():
    """With layers that add nothing the next token is a function of the current one alone:
    T[t] = argmax_v lm_head[v] . norm(embed[t]); greedy must walk that table, and append one cache
    row per step at consecutive positions."""
    rng = np.random.default_rng(11)
    model = _model(rng, o=_zeros(QH * D, H), down=_zeros(FFN, H))
    vocab = H
    model["lm_head"] = rng.normal(0, 0.3, (vocab, H)).astype(np.float16)
    table = []
    for t in range(vocab):
        xn = _norm(model["embed"][t], np.ones(H))
        logit = [float(np.float16(math.fsum(float(xn[i]) * float(model["lm_head"][j, i]) for i in range(H))))
                 for j in range(vocab)]
        table.append(int(np.argmax(logit)))
    k = [np.zeros((2, KVH, 32, D), np.float16)]
    v = [np.zeros((2, KVH, 32, D), np.float16)]
    start, pos = [5, 41], [3, 10]
    out, logits = OD.greedy(model, start, pos, k, v, 4)
    assert out.shape == (4, 2) and len(logits) == 4
    for b in range(2):
        t = start[b]
        for step in range(4):
            t = table[t]
            assert out[step, b] == t
        written = np.abs(k[0][b].astype(np.float32)).sum(axis=(0, 2)) > 0
        assert written.tolist() == [pos[b] <= s < pos[b] + 4 for s in range(32)]


# ------------------------------------------------------------------ biases and act-order (examples/qwen1_5_int8.py:276-385)

def test_biases_are_added_to_the_rounded_product_in_fp16():
    """o and down exactly zero but biased: the residual stream is embed + b_o + b_down, two fp16 adds; a
    biased q|k|v that selects nothing appends k = RoPE(b_k) and v = b_v."""
    rng = np.random.default_rng(21)
    b_qkv = rng.normal(0, 1, (QH + 2 * KVH) * D).astype(np.float16)
    b_o = rng.normal(0, 1, H).astype(np.float16)
    b_down = rng.normal(0, 1, H).astype(np.float16)
    model = _model(rng, qkv=_zeros(H, (QH + 2 * KVH) * D) + (b_qkv,), o=_zeros(QH * D, H) + (b_o,),
                   down=_zeros(FFN, H) + (b_down,))
    tokens, positions = np.array([5, 9]), np.array([0, 3])
    k, v = _caches(rng, 2)
    logits = OD.decode_step(model, tokens, positions, k, v)
    for b, t in enumerate(tokens):
        h = _add16(_add16(model["embed"][t], b_o), b_down)
        np.testing.assert_array_equal(logits[b], _logits_from_hidden(h))
        p = int(positions[b])
        np.testing.assert_array_equal(v[0][b, :, p].reshape(-1), b_qkv[(QH + KVH) * D:])
        want_k = OS.rope(b_qkv[QH * D:(QH + KVH) * D].reshape(1, 1, KVH, D), model["cos"], model["sin"],
                         np.array([[p]]))[0, 0]
        np.testing.assert_array_equal(k[0][b, :, p], want_k)


def test_gate_and_up_biases_enter_before_the_activation():
    """gate|up exactly zero with biases (b_gate, b_up), down the identity: h = embed + silu(b_gate) * b_up
    with the three fp16 roundings of the models' silu (sigmoid, times the gate, times up)."""
    rng = np.random.default_rng(22)
    b_gate, b_up = rng.normal(0, 1, FFN).astype(np.float16), rng.normal(0, 1, FFN).astype(np.float16)
    model = _model(rng, o=_zeros(QH * D, H), gate_up=_zeros(H, 2 * FFN) + (np.concatenate([b_gate, b_up]),),
                   down=_eye(H))
    tokens, positions = np.array([2, 30]), np.array([1, 6])
    k, v = _caches(rng, 2)
    logits = OD.decode_step(model, tokens, positions, k, v)
    act = OG.silu_mul(b_gate, b_up)
    for b, t in enumerate(tokens):
        np.testing.assert_array_equal(logits[b], _logits_from_hidden(_add16(model["embed"][t], act)))


def test_act_order_rows_take_the_scale_and_zero_point_of_their_own_group():
    """A linear with a permuted g_idx (row k belongs to group g_idx[k]) against the dense product written
    out from the unpacked tensors, and invariance: the same rows listed group by group with a sequential
    g_idx, fed the activations in that order, give the same numbers."""
    rng = np.random.default_rng(23)
    k_dim, n = 2 * G, 24
    q = rng.integers(0, 16, (k_dim, n)).astype(np.uint8)
    z = rng.integers(0, 16, (k_dim // G, n)).astype(np.uint8)
    s = (rng.uniform(0.01, 0.05, (k_dim // G, n))).astype(np.float16)
    g_idx = rng.permutation(np.arange(k_dim) // G).astype(np.int32)
    bias = rng.normal(0, 1, n).astype(np.float16)
    x = rng.normal(0, 1, (3, k_dim)).astype(np.float16)
    w = (OG.pack(q, 0, 4), OG.pack(z, 1, 4), s, G, bias, g_idx)
    got = OD._linear(x, w)
    dense = np.empty((k_dim, n), np.float64)
    for r in range(k_dim):
        g = g_idx[r]
        dense[r] = ((q[r].astype(np.float64) - (z[g].astype(np.float64) + 1)) * s[g].astype(np.float64)).astype(np.float16)
    want = _add16((x.astype(np.float64) @ dense).astype(np.float16), np.broadcast_to(bias, (3, n)))
    np.testing.assert_array_equal(got, want)
    perm = np.argsort(g_idx, kind="stable")
    sorted_w = (OG.pack(q[perm], 0, 4), w[1], s, G, bias, None)
    same = OD._linear(np.ascontiguousarray(x[:, perm]), sorted_w)
    assert np.abs(same.astype(np.float64) - got.astype(np.float64)).max() <= 2 * np.spacing(np.abs(got).max())
