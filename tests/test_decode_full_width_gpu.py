"""GPU parity of the decode loop at the Llama-3-70B layer widths (config 4):
hidden 8192, 64 query / 8 KV heads of 128, ffn 28672, context 2048, batch 1, 8
and 32 -- the shapes the tokens-per-second figure is timed on, two layers deep so
that the second layer consumes what the fused epilogues of the first one wrote
(residual stream, sums of squares, cache rows).  At these widths the step runs
the norm-prologue + SiLU-epilogue gate|up product at 8192 x 57344, the
residual-epilogue down product at 28672 x 8192, the cut-tile q|k|v product with
its RoPE / cache-append epilogue and, above 8 rows, the second-stage kernels.

Checker: oracle.decode.decode_step (examples/llama3_70b.py:157-162,215-228 op by
op) with the C restatement of the quantized product (bit-exact to the numpy one,
tests/test_oracle_cport.py) so that it runs in seconds.  The vocabulary is small:
the lm_head product at its real size is covered in test_gptq_gpu.py.
"""
import numpy as np
import pytest

from oracle import cport
from oracle import decode as OD
from oracle import special as OS
from minit_amd.decode import untile_v_cache

pytestmark = pytest.mark.gpu

CFG = dict(n_layers=2, hidden=8192, n_q_heads=64, n_kv_heads=8, head_dim=128, ffn=28672, vocab=256,
           group_size=128, bits=4, rope_theta=5e5, rms_eps=1e-5)
CONTEXT, MAX_SEQ = 2048, 2048 + 64


def _c_linear(x, w, bits=4):
    qweight, qzeros, scales, group_size = w
    return cport.matmul(x, qweight, qzeros, scales, None, bits, group_size)


@pytest.fixture(scope="module")
def wide_model():
    from minit_amd import synthetic
    cport.lib()
    rng = np.random.default_rng(70)
    d = CFG["head_dim"]
    shapes = {"qkv": (CFG["hidden"], (CFG["n_q_heads"] + 2 * CFG["n_kv_heads"]) * d),
              "o": (CFG["n_q_heads"] * d, CFG["hidden"]),
              "gate_up": (CFG["hidden"], 2 * CFG["ffn"]),
              "down": (CFG["ffn"], CFG["hidden"])}
    layers = []
    for l in range(CFG["n_layers"]):
        layer = {}
        for name, (k, n) in shapes.items():
            qw, qz, sc = synthetic.gptq_weights("wide70b", f"{l}.{name}", k, n, CFG["group_size"], 4)
            # sums over 8192 / 28672 terms: keep the projections around unit size, or the reference's fp16
            # attention scores (q . k before the 1/sqrt(d) scale) overflow
            layer[name] = (qw, qz, (sc.astype(np.float32) / 16).astype(np.float16), CFG["group_size"])
        layer["input_norm"] = rng.normal(1, 0.1, CFG["hidden"]).astype(np.float16)
        layer["post_norm"] = rng.normal(1, 0.1, CFG["hidden"]).astype(np.float16)
        layers.append(layer)
    cos, sin = OS.rope_tables(d, MAX_SEQ, CFG["rope_theta"])
    return {"config": CFG, "layers": layers,
            "embed": rng.normal(0, 1.0, (CFG["vocab"], CFG["hidden"])).astype(np.float16),
            "lm_head": rng.normal(0, 0.02, (CFG["vocab"], CFG["hidden"])).astype(np.float16),
            "final_norm": rng.normal(1, 0.1, CFG["hidden"]).astype(np.float16), "cos": cos, "sin": sin}


def test_two_layers_at_70b_widths_eight_bit_weights(hip):
    """The same widths on 8-bit weights (what the reference's own example ships, examples/qwen1_5_int8.py)
    at 5 rows: gate|up (224 column tiles) then runs with the two K halves of a tile in one workgroup of
    eight waves, norm prologue and SiLU epilogue included, which 4-bit weights take only above 8 rows."""
    from minit_amd import synthetic
    from minit_amd.decode import LlamaDecoder
    cport.lib()
    cfg = dict(CFG, bits=8)
    batch, d = 5, CFG["head_dim"]
    rng = np.random.default_rng(78)
    shapes = {"qkv": (cfg["hidden"], (cfg["n_q_heads"] + 2 * cfg["n_kv_heads"]) * d),
              "o": (cfg["n_q_heads"] * d, cfg["hidden"]),
              "gate_up": (cfg["hidden"], 2 * cfg["ffn"]),
              "down": (cfg["ffn"], cfg["hidden"])}
    layers = []
    for l in range(cfg["n_layers"]):
        layer = {}
        for name, (k, n) in shapes.items():
            # zero points around the middle of the range and 16 times finer steps: the weight spread of the
            # 4-bit model above, then the same 1/16 that keeps the projections around unit size
            qw, qz, sc = synthetic.gptq_weights("wide70b8", f"{l}.{name}", k, n, cfg["group_size"], 8, zero_range=(120, 135))
            layer[name] = (qw, qz, (sc.astype(np.float32) / 256).astype(np.float16), cfg["group_size"])
        layer["input_norm"] = rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16)
        layer["post_norm"] = rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16)
        layers.append(layer)
    cos, sin = OS.rope_tables(d, MAX_SEQ, cfg["rope_theta"])
    model = {"config": cfg, "layers": layers,
             "embed": rng.normal(0, 1.0, (cfg["vocab"], cfg["hidden"])).astype(np.float16),
             "lm_head": rng.normal(0, 0.02, (cfg["vocab"], cfg["hidden"])).astype(np.float16),
             "final_norm": rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16), "cos": cos, "sin": sin}
    shape = (batch, cfg["n_kv_heads"], MAX_SEQ, d)
    k_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(cfg["n_layers"])]
    v_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(cfg["n_layers"])]
    tokens = rng.integers(0, cfg["vocab"], batch).astype(np.int32)
    positions = (CONTEXT - np.arange(batch) * 3).astype(np.int32)
    dec = LlamaDecoder(cfg, batch, MAX_SEQ)
    dec.load_host(model, k_cache, v_cache)
    _, got = dec.decode(tokens, positions, 1, want_logits=True)
    ref_k, ref_v = [c.copy() for c in k_cache], [c.copy() for c in v_cache]
    ref = OD.decode_step(model, tokens, positions, ref_k, ref_v, linear=_c_linear)
    g, r = got.astype(np.float64), ref.astype(np.float64)
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - r) / np.linalg.norm(r)
    print(f"[70B widths, 8 bit] logits rel L2 {rel:.3g}, worst |err| {np.abs(g - r).max():.3g} of {np.abs(r).max():.3g}", flush=True)
    assert rel <= 1e-2, f"relative L2 error of the logits {rel:.3g}"
    assert np.abs(g - r).max() <= 2e-2 * max(1.0, np.abs(r).max())
    for layer in range(cfg["n_layers"]):
        kc, vc = dec.k_cache[layer].numpy(), untile_v_cache(dec.v_cache[layer].numpy())
        tol = 2e-2 if layer == 0 else 6e-2
        for b in range(batch):
            pos = int(positions[b])
            assert np.abs(kc[b, :, pos].astype(np.float64) - ref_k[layer][b, :, pos].astype(np.float64)).max() <= tol
            assert np.abs(vc[b, :, pos].astype(np.float64) - ref_v[layer][b, :, pos].astype(np.float64)).max() <= tol


@pytest.mark.parametrize("batch", [1, 8, 32])
def test_two_layers_at_70b_widths(hip, wide_model, batch):
    from minit_amd.decode import LlamaDecoder
    model = wide_model
    rng = np.random.default_rng(700 + batch)
    shape = (batch, CFG["n_kv_heads"], MAX_SEQ, CFG["head_dim"])
    k_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(CFG["n_layers"])]
    v_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(CFG["n_layers"])]
    tokens = rng.integers(0, CFG["vocab"], batch).astype(np.int32)
    # context 2048, a few rows a little shorter: every row reads its own number of entries
    positions = (CONTEXT - (np.arange(batch) % 5) * 3).astype(np.int32)
    print(f"[70B widths] batch {batch}, positions {positions.min()}..{positions.max()}", flush=True)

    dec = LlamaDecoder(CFG, batch, MAX_SEQ)
    dec.load_host(model, k_cache, v_cache)
    got_tokens, got = dec.decode(tokens, positions, 1, want_logits=True)

    ref_k, ref_v = [c.copy() for c in k_cache], [c.copy() for c in v_cache]
    ref = OD.decode_step(model, tokens, positions, ref_k, ref_v, linear=_c_linear)
    g, r = got.astype(np.float64), ref.astype(np.float64)
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - r) / np.linalg.norm(r)
    worst = np.abs(g - r).max()
    print(f"[70B widths] batch {batch}: logits rel L2 {rel:.3g}, worst |err| {worst:.3g} of {np.abs(r).max():.3g}", flush=True)
    assert rel <= 1e-2, f"relative L2 error of the logits {rel:.3g}"
    assert worst <= 2e-2 * max(1.0, np.abs(r).max())
    ref_tok = ref.astype(np.float32).argmax(-1)
    for b in range(batch):
        if got_tokens[0, b] != ref_tok[b]:
            row = np.sort(r[b])
            assert row[-1] - row[-2] < 2e-2, f"row {b}: token differs with a clear margin"

    # appended keys and values, each row at its own position: layer 0 sees only the q|k|v product and RoPE,
    # layer 1 everything the first layer computed (attention, o + residual, gate|up + SiLU, down + residual, norm)
    for layer in range(CFG["n_layers"]):
        kc, vc = dec.k_cache[layer].numpy(), untile_v_cache(dec.v_cache[layer].numpy())   # both [B, KVH, T, D]
        tol = 2e-2 if layer == 0 else 6e-2
        for b in range(batch):
            p = int(positions[b])
            ek = np.abs(kc[b, :, p].astype(np.float64) - ref_k[layer][b, :, p].astype(np.float64)).max()
            ev = np.abs(vc[b, :, p].astype(np.float64) - ref_v[layer][b, :, p].astype(np.float64)).max()
            assert ek <= tol and ev <= tol, f"layer {layer} row {b}: appended k/v off by {ek:.3g} / {ev:.3g}"
        # what was already in the cache stays (row 0, below its position)
        p0 = int(positions[0])
        assert np.array_equal(kc[0, :, :p0].view(np.uint16), k_cache[layer][0, :, :p0].view(np.uint16))


def test_recorded_step_at_70b_widths_replays_like_the_eager_loop(hip, wide_model):
    """Three tokens at batch 32 (one unsplit attention block per row and KV head, second-stage kernels
    for q|k|v, gate|up and down): the recorded step, replayed, gives the eager loop's tokens, logits and
    caches bit for bit."""
    from minit_amd.decode import LlamaDecoder
    batch, steps = 32, 3
    rng = np.random.default_rng(732)
    shape = (batch, CFG["n_kv_heads"], MAX_SEQ, CFG["head_dim"])
    k_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(CFG["n_layers"])]
    v_cache = [rng.standard_normal(shape, np.float32).astype(np.float16) for _ in range(CFG["n_layers"])]
    tokens = rng.integers(0, CFG["vocab"], batch).astype(np.int32)
    positions = (CONTEXT - (np.arange(batch) % 7) * 11).astype(np.int32)
    runs = []
    for graph in (False, True):
        print(f"[70B widths] batch {batch}, {steps} steps, graph={graph}", flush=True)
        dec = LlamaDecoder(CFG, batch, MAX_SEQ)
        dec.load_host(wide_model, k_cache, v_cache)
        out, logits = dec.decode(tokens, positions, steps, want_logits=True, graph=graph)
        runs.append((out, logits, [t.numpy() for t in dec.k_cache + dec.v_cache]))
        del dec
    (out_e, logits_e, cache_e), (out_g, logits_g, cache_g) = runs
    np.testing.assert_array_equal(out_g, out_e)
    np.testing.assert_array_equal(logits_g.view(np.uint16), logits_e.view(np.uint16))
    for a, b in zip(cache_g, cache_e):
        np.testing.assert_array_equal(a.view(np.uint16), b.view(np.uint16))
