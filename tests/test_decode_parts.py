"""The parts of a decode step as entry points of their own (attention, RoPE and
cache append, residual add + RMSNorm, greedy sampling).  Decode attention: the restatement is pinned on the CPU by what the
mathematics fixes, and the HIP entry points (mh_rope_kv_append, mh_attn_decode)
are checked against it on the GPU.  The device keeps fp32 where the reference
rounds scores and probabilities to fp16, so outputs are compared under an
absolute bound of 4e-3 (values are averages of N(0, 1) entries) and a relative
L2 bound of 5e-3."""
import numpy as np
import pytest

from oracle import decode as OD
from oracle import special as OS


def test_oracle_attention_closed_forms():
    rng = np.random.default_rng(1)
    b, qh, kvh, t, d = 2, 4, 2, 9, 128
    q = rng.normal(0, 1, (b, qh, d)).astype(np.float16)
    k = rng.normal(0, 1, (b, kvh, t, d)).astype(np.float16)
    v = rng.normal(0, 1, (b, kvh, t, d)).astype(np.float16)
    pos = np.array([8, 3])
    out = OD.attention(q, k, v, pos)
    assert out.shape == (b, qh, d) and out.dtype == np.float16
    # a single visible entry: the output is that value row, whatever q is
    one = OD.attention(q, k, v, np.array([0, 0]))
    for h in range(qh):
        np.testing.assert_array_equal(one[:, h], v[:, h // 2, 0])
    # q = 0: uniform weights, the mean of the visible value rows
    zero = OD.attention(np.zeros_like(q), k, v, pos)
    for i in range(b):
        mean = v[i, :, :pos[i] + 1].astype(np.float64).mean(axis=1)
        np.testing.assert_allclose(zero[i, 0].astype(np.float64), mean[0], atol=2e-3)
        np.testing.assert_allclose(zero[i, 3].astype(np.float64), mean[1], atol=2e-3)
    # entries past positions[b] are not read
    k2, v2 = k.copy(), v.copy()
    k2[1, :, 4:] = 77
    v2[1, :, 4:] = -55
    np.testing.assert_array_equal(OD.attention(q, k2, v2, pos)[1], out[1])
    # against the float64 form without intermediate rounding
    for i, h in ((0, 0), (1, 3)):
        g = h // 2
        s = k[i, g, :pos[i] + 1].astype(np.float64) @ q[i, h].astype(np.float64) / np.sqrt(d)
        p = np.exp(s - s.max())
        ref = (p / p.sum()) @ v[i, g, :pos[i] + 1].astype(np.float64)
        np.testing.assert_allclose(out[i, h].astype(np.float64), ref, atol=4e-3)


def _t(arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


@pytest.mark.gpu
@pytest.mark.parametrize("batch,qh,kvh,max_seq,positions", [
    (1, 8, 1, 64, [0]),                     # one visible entry
    (3, 8, 2, 320, [5, 255, 319]),          # ragged rows, a chunk boundary, the last slot
    (2, 64, 8, 2112, [2047, 1000]),         # the 70B head geometry, several splits
    (5, 4, 4, 128, [17, 64, 63, 127, 1]),   # one query head per KV head
    (2, 4, 2, 576, [300, 575]),             # two query heads per KV head
    # a (row, KV head) pair per CU: one block of eight waves per pair, no merge across blocks;
    # rows shorter than one pass of the block, a ragged end, the last slot
    (32, 16, 8, 640, [(7 * i * i + 3) % 640 for i in range(29)] + [0, 511, 639]),
    # the decode benchmark's cache (context 2048 and the tokens after it): the first position of a
    # new chunk, the last slot, and in between, at the block counts of 2, 8 and 12 rows
    (2, 64, 8, 2176, [2048, 2175]),
    (8, 64, 8, 2176, [2048, 2049, 2111, 2112, 2113, 2174, 2175, 64]),
    (12, 64, 8, 2176, [2048 + 11 * i for i in range(12)]),
])
def test_attention_entry_points_match_oracle(hip, batch, qh, kvh, max_seq, positions):
    from minit_amd.hip.tensor import HIPTensor
    d = 128
    rng = np.random.default_rng(batch * 100 + qh)
    pos = np.asarray(positions, np.int32)
    k_cache = rng.normal(0, 1, (batch, kvh, max_seq, d)).astype(np.float16)
    v_cache = rng.normal(0, 1, (batch, kvh, max_seq, d)).astype(np.float16)
    # what lies past a row's position is not part of the result, whatever it holds: the kernel
    # requests whole chunks before it knows the length
    for i in range(batch):
        k_cache[i, :, pos[i] + 1:] = np.float16(np.nan)
        v_cache[i, :, pos[i] + 1:] = np.float16(np.inf)
    qkv = rng.normal(0, 1, (batch, (qh + 2 * kvh) * d)).astype(np.float16)
    cos, sin = OS.rope_tables(d, max_seq, 5e5)

    # oracle: rotate q and k, append k and v at positions[b], attend
    q_ref = OS.rope(qkv[:, :qh * d].reshape(batch, 1, qh, d), cos, sin, pos.reshape(batch, 1))[:, 0]
    k_new = OS.rope(qkv[:, qh * d:(qh + kvh) * d].reshape(batch, 1, kvh, d), cos, sin, pos.reshape(batch, 1))[:, 0]
    v_new = qkv[:, (qh + kvh) * d:].reshape(batch, kvh, d)
    k_ref, v_ref = k_cache.copy(), v_cache.copy()
    for i in range(batch):
        k_ref[i, :, pos[i]] = k_new[i]
        v_ref[i, :, pos[i]] = v_new[i]
    ref = OD.attention(q_ref, k_ref, v_ref, pos)

    from minit_amd.decode import tile_v_cache, untile_v_cache
    dk, dvt = _t(k_cache), _t(tile_v_cache(v_cache))
    dq = HIPTensor.allocate((batch, qh, d), "float16")
    dpos, dqkv, dcos, dsin = _t(pos), _t(qkv), _t(cos), _t(sin)   # named: the buffers must outlive the launch
    hip.call("mh_rope_kv_append", None, dqkv.data_ptr, dcos.data_ptr, dsin.data_ptr, dpos.data_ptr,
             dq.data_ptr, dk.data_ptr, dvt.data_ptr, batch, qh, kvh, d, max_seq)
    # the copy of v is exact; the rotation is fp32 on the device against float64 here, one
    # rounding each: equal except where the fp32 value sits on a rounding boundary (one step)
    np.testing.assert_array_equal(dvt.numpy().view(np.uint16), tile_v_cache(v_ref).view(np.uint16))
    np.testing.assert_array_equal(untile_v_cache(dvt.numpy()).view(np.uint16), v_ref.view(np.uint16))
    for got, want in ((dq.numpy(), q_ref), (dk.numpy(), k_ref)):
        live = np.isfinite(want)            # the poisoned tail of the K cache stays as it was
        np.testing.assert_array_equal(got.view(np.uint16)[~live], want.view(np.uint16)[~live])
        step = np.spacing(np.abs(want[live])).astype(np.float64)
        assert (np.abs(got[live].astype(np.float64) - want[live].astype(np.float64)) <= step).all()
        assert (got.view(np.uint16)[live] != want.view(np.uint16)[live]).mean() < 1e-3

    nbytes = hip.call("mh_attn_decode_workspace_bytes", batch, qh, kvh, d, max_seq)
    ws = HIPTensor.allocate((nbytes,), "int8")
    ws._memory.reset()
    out = HIPTensor.allocate((batch, qh, d), "float16")
    for _ in range(2):   # the second call finds the counters as the first one left them
        hip.call("mh_attn_decode", None, dq.data_ptr, dk.data_ptr, dvt.data_ptr, dpos.data_ptr, out.data_ptr,
                 batch, qh, kvh, d, max_seq, ws.data_ptr, nbytes)
    from minit_amd.decode import decode_attention
    bound = decode_attention(dq, dk, dvt, dpos, max_seq)      # the Python binding, its own workspace
    np.testing.assert_array_equal(bound.numpy().view(np.uint16), out.numpy().view(np.uint16))
    got = out.numpy().astype(np.float64)
    r = ref.astype(np.float64)
    assert np.abs(got - r).max() <= 4e-3, np.abs(got - r).max()
    assert np.linalg.norm(got - r) / np.linalg.norm(r) <= 5e-3


@pytest.mark.gpu
def test_attention_arguments_are_checked(hip):
    from minit_amd import lib
    from minit_amd.hip.tensor import HIPTensor
    t = HIPTensor.allocate((4096,), "float16")
    with pytest.raises(lib.HipError, match="head_dim"):
        hip.call("mh_attn_decode", None, t.data_ptr, t.data_ptr, t.data_ptr, t.data_ptr, t.data_ptr, 1, 8, 1, 64, 64,
                 t.data_ptr, 8192)
    with pytest.raises(lib.HipError, match="workspace"):
        hip.call("mh_attn_decode", None, t.data_ptr, t.data_ptr, t.data_ptr, t.data_ptr, t.data_ptr, 1, 8, 1, 128, 64,
                 None, 0)
    assert hip.call("mh_attn_decode_workspace_bytes", 1, 8, 1, 64, 64) == 0


@pytest.mark.gpu
def test_argmax_rows_first_maximum(hip):
    """mh_argmax against numpy's argmax (first maximum), ties and a vocabulary-sized
    row with an odd width included."""
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(4)
    for rows, cols in ((1, 7), (3, 1000), (2, 128257), (4, 4096)):
        x = rng.normal(0, 2, (rows, cols)).astype(np.float16)
        x[0, cols // 2] = x.max() + 1            # a clear winner
        if rows > 1:
            x[1, :] = 0.5                        # all tied: the first index wins
            x[-1, [cols - 1, cols // 3]] = 60.0  # a two-way tie
        dx = _t(x)
        out = HIPTensor.allocate((rows,), "int32")
        hip.call("mh_argmax", None, dx.data_ptr, out.data_ptr, rows, cols)
        np.testing.assert_array_equal(out.numpy(), x.argmax(axis=-1).astype(np.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,hidden", [(1, 8192), (5, 4096), (3, 264)])
def test_add_rms_norm_matches_add_then_norm(hip, rows, hidden):
    """h + delta rounded to fp16 first (bit for bit against the fp16 sum), then the
    norm of that sum within one fp16 step of the float64 closed form; delta = NULL
    leaves h alone."""
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(rows + hidden)
    h = rng.normal(0, 1, (rows, hidden)).astype(np.float16)
    delta = rng.normal(0, 1, (rows, hidden)).astype(np.float16)
    w = rng.normal(1, 0.1, hidden).astype(np.float16)
    dh, dd, dw = _t(h), _t(delta), _t(w)
    out = HIPTensor.allocate((rows, hidden), "float16")
    hip.call("mh_add_rms_norm", None, dh.data_ptr, dd.data_ptr, dw.data_ptr, out.data_ptr, rows, hidden, 1e-5)
    summed = h + delta                                      # numpy fp16 add: one rounding
    np.testing.assert_array_equal(dh.numpy().view(np.uint16), summed.view(np.uint16))
    ref = OS.rms_norm(summed, w, 1, 1e-5).astype(np.float64)
    err = np.abs(out.numpy().astype(np.float64) - ref)
    assert (err <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) + 1e-6).all()
    hip.call("mh_add_rms_norm", None, dh.data_ptr, None, dw.data_ptr, out.data_ptr, rows, hidden, 1e-5)
    np.testing.assert_array_equal(dh.numpy().view(np.uint16), summed.view(np.uint16))
    err = np.abs(out.numpy().astype(np.float64) - ref)
    assert (err <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) + 1e-6).all()


@pytest.mark.gpu
def test_one_step_composed_from_the_operator_api(hip):
    """One decode step written the way the reference's model code is written -- norm,
    quantized linears, rotary embedding and cache append, attention, silu(gate) * up
    as ``x * F.sigmoid(x)``, residual adds, lm_head, argmax -- from the operator API
    and the stand-alone entry points, against the oracle's step and against the
    native loop's logits."""
    import minit_amd.functional as F
    from minit_amd.decode import LlamaDecoder, decode_attention, tile_v_cache
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import quantized_tensor_from_host
    from test_decode_gpu import CFG, _host_model
    cfg = CFG
    batch, max_seq, context = 3, 64, 23
    qh, kvh, d, ffn, hidden = cfg["n_q_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"], cfg["hidden"]
    model = _host_model(cfg, seed=91)
    rng = np.random.default_rng(910)
    shape = (batch, kvh, max_seq, d)
    k_cache = [np.zeros(shape, np.float16) for _ in range(cfg["n_layers"])]
    v_cache = [np.zeros(shape, np.float16) for _ in range(cfg["n_layers"])]
    for c in k_cache + v_cache:
        c[:, :, :context] = rng.normal(0, 1, (batch, kvh, context, d))
    tokens = rng.integers(0, cfg["vocab"], batch)
    positions = np.array([context, context - 4, context - 9])
    ref_logits = OD.decode_step(model, tokens, positions, [c.copy() for c in k_cache], [c.copy() for c in v_cache])

    def qt(w, cols=None):
        qweight, qzeros, scales, _ = w
        if cols is not None:
            lo, hi = cols
            qweight, qzeros, scales = qweight[:, lo:hi], qzeros[:, lo // 8:hi // 8], scales[:, lo:hi]
        return quantized_tensor_from_host(*(np.ascontiguousarray(t) for t in (qweight, qzeros, scales)))

    cos, sin = _t(model["cos"]), _t(model["sin"])
    pos = _t(positions.astype(np.int32))
    eps = cfg["rms_eps"]
    h = _t(model["embed"][tokens])
    xn = F.rms_norm(h, _t(model["layers"][0]["input_norm"]), 1, eps)
    for l, layer in enumerate(model["layers"]):
        kc, vt = _t(k_cache[l]), _t(tile_v_cache(v_cache[l]))
        qkv = F.matrix_multiply(xn, qt(layer["qkv"]))
        q = HIPTensor.allocate((batch, qh, d), "float16")
        hip.call("mh_rope_kv_append", None, qkv.data_ptr, cos.data_ptr, sin.data_ptr, pos.data_ptr, q.data_ptr,
                 kc.data_ptr, vt.data_ptr, batch, qh, kvh, d, max_seq)
        attn = decode_attention(q, kc, vt, pos, max_seq)
        o = F.matrix_multiply(attn.reshape((batch, qh * d)), qt(layer["o"]))
        post = _t(layer["post_norm"])
        hip.call("mh_add_rms_norm", None, h.data_ptr, o.data_ptr, post.data_ptr, xn.data_ptr, batch, hidden, eps)
        gate = F.matrix_multiply(xn, qt(layer["gate_up"], (0, ffn)))
        up = F.matrix_multiply(xn, qt(layer["gate_up"], (ffn, 2 * ffn)))
        act = (gate * F.sigmoid(gate)) * up                       # silu(gate) * up as the models spell it
        down = F.matrix_multiply(act, qt(layer["down"]))
        nxt = _t(model["layers"][l + 1]["input_norm"] if l + 1 < cfg["n_layers"] else model["final_norm"])
        hip.call("mh_add_rms_norm", None, h.data_ptr, down.data_ptr, nxt.data_ptr, xn.data_ptr, batch, hidden, eps)
    # the residual add also exists as an operator of its own (`x = x + ...` in the models)
    np.testing.assert_array_equal((h + down).numpy().view(np.uint16), (h.numpy() + down.numpy()).view(np.uint16))
    logits = F.matrix_multiply(xn, _t(model["lm_head"]))          # dense rule: weight [vocab, hidden]
    token = HIPTensor.allocate((batch,), "int32")
    hip.call("mh_argmax", None, logits.data_ptr, token.data_ptr, batch, cfg["vocab"])

    g, r = logits.numpy().astype(np.float64), ref_logits.astype(np.float64)
    assert np.linalg.norm(g - r) / np.linalg.norm(r) <= 1e-2
    assert np.abs(g - r).max() <= 2e-2 * max(1.0, np.abs(r).max())
    np.testing.assert_array_equal(token.numpy(), logits.numpy().astype(np.float32).argmax(axis=-1))

    dec = LlamaDecoder(cfg, batch, max_seq)
    dec.load_host(model, k_cache, v_cache)
    _, native = dec.decode(tokens, positions, 1, want_logits=True)
    n = native.astype(np.float64)
    assert np.linalg.norm(g - n) / np.linalg.norm(n) <= 1e-2
