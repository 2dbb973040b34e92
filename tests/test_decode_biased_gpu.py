"""GPU parity of the native decode loop on the reference's own GPTQ model shape
(examples/qwen1_5_int8.py:320-400, Qwen-14B-Chat-Int8): 8-bit weights, hidden 5120 in 40 groups of 128,
40 heads of 128 without grouped queries, an MLP of 13696 (107 groups: K of the down projection is not a
multiple of the kernels' 256-k stages), a bias on every linear (QLinearWithBias) and act-order g_idx.
The bias is added to the fp16-rounded product before RoPE, before silu(gate) * up and before the
residual add; act-order weights are sorted by group at load time and the loop gathers the activations.
Checker: oracle.decode.decode_step with the C restatement of the quantized product."""
import numpy as np
import pytest

from oracle import cport
from oracle import decode as OD
from oracle import special as OS
from minit_amd.decode import untile_v_cache

pytestmark = pytest.mark.gpu

QWEN = dict(n_layers=2, hidden=5120, n_q_heads=40, n_kv_heads=40, head_dim=128, ffn=13696, vocab=256,
            group_size=128, bits=8, rope_theta=1e6, rms_eps=1e-6)
WIDE = dict(n_layers=2, hidden=8192, n_q_heads=64, n_kv_heads=8, head_dim=128, ffn=256, vocab=256,
            group_size=128, bits=4, rope_theta=5e5, rms_eps=1e-5)


def _c_linear(x, w, bits=4):
    qweight, qzeros, scales, group_size, bias, g_idx = OD.split_linear(w)
    return OD.add_bias(cport.matmul(x, qweight, qzeros, scales, g_idx, bits, group_size), bias)


def _model(cfg, seed, act_order):
    from minit_amd import synthetic
    cport.lib()
    rng = np.random.default_rng(seed)
    d, g = cfg["head_dim"], cfg["group_size"]
    shapes = {"qkv": (cfg["hidden"], (cfg["n_q_heads"] + 2 * cfg["n_kv_heads"]) * d),
              "o": (cfg["n_q_heads"] * d, cfg["hidden"]),
              "gate_up": (cfg["hidden"], 2 * cfg["ffn"]),
              "down": (cfg["ffn"], cfg["hidden"])}
    layers = []
    for l in range(cfg["n_layers"]):
        layer = {}
        for name, (k, n) in shapes.items():
            if cfg["bits"] == 8:
                qw, qz, sc = synthetic.gptq_weights(f"biased{seed}", f"{l}.{name}", k, n, g, 8, zero_range=(120, 135))
                sc = (sc.astype(np.float32) / 256).astype(np.float16)   # sums over 5120 / 13696 terms of unit size
            else:
                qw, qz, sc = synthetic.gptq_weights(f"biased{seed}", f"{l}.{name}", k, n, g, 4)
                sc = (sc.astype(np.float32) / 16).astype(np.float16)
            bias = rng.normal(0, 0.5, n).astype(np.float16)
            g_idx = None
            if act_order and (l == 0 or name in ("o", "down")):
                g_idx = rng.permutation(np.arange(k) // g).astype(np.int32)
            layer[name] = (qw, qz, sc, g, bias, g_idx)
        layer["input_norm"] = rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16)
        layer["post_norm"] = rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16)
        layers.append(layer)
    cos, sin = OS.rope_tables(d, 128, cfg["rope_theta"])
    return {"config": cfg, "layers": layers,
            "embed": rng.normal(0, 1.0, (cfg["vocab"], cfg["hidden"])).astype(np.float16),
            "lm_head": rng.normal(0, 0.02, (cfg["vocab"], cfg["hidden"])).astype(np.float16),
            "final_norm": rng.normal(1, 0.1, cfg["hidden"]).astype(np.float16), "cos": cos, "sin": sin}


@pytest.fixture(scope="module")
def qwen_model():
    return _model(QWEN, 14, act_order=True)


@pytest.fixture(scope="module")
def wide_model():
    return _model(WIDE, 15, act_order=False)


def _run_and_check(cfg, model, batch, context=40, max_seq=128):
    from minit_amd.decode import LlamaDecoder
    rng = np.random.default_rng(1400 + batch)
    shape = (batch, cfg["n_kv_heads"], max_seq, cfg["head_dim"])
    k_cache = [np.zeros(shape, np.float16) for _ in range(cfg["n_layers"])]
    v_cache = [np.zeros(shape, np.float16) for _ in range(cfg["n_layers"])]
    for c in k_cache + v_cache:
        c[:, :, :context] = rng.normal(0, 1, (batch, cfg["n_kv_heads"], context, cfg["head_dim"]))
    tokens = rng.integers(0, cfg["vocab"], batch).astype(np.int32)
    positions = (context - (np.arange(batch) % 4) * 5).astype(np.int32)
    print(f"[biased] hidden {cfg['hidden']}, {cfg['bits']} bit, batch {batch}", flush=True)
    dec = LlamaDecoder(cfg, batch, max_seq)
    dec.load_host(model, k_cache, v_cache)
    got_tokens, got = dec.decode(tokens, positions, 1, want_logits=True)
    ref_k, ref_v = [c.copy() for c in k_cache], [c.copy() for c in v_cache]
    ref = OD.decode_step(model, tokens, positions, ref_k, ref_v, linear=_c_linear)
    # the same model with the biases dropped must be far away, or the biases would not be tested
    bare = dict(model, layers=[{k: (v[:4] + (None,) + v[5:] if isinstance(v, tuple) else v) for k, v in layer.items()}
                               for layer in model["layers"]])
    off = OD.decode_step(bare, tokens, positions, [c.copy() for c in k_cache], [c.copy() for c in v_cache],
                         linear=_c_linear)
    g, r = got.astype(np.float64), ref.astype(np.float64)
    assert np.linalg.norm(off.astype(np.float64) - r) / np.linalg.norm(r) > 5e-2
    assert np.isfinite(g).all()
    rel = np.linalg.norm(g - r) / np.linalg.norm(r)
    worst = np.abs(g - r).max()
    print(f"[biased] batch {batch}: logits rel L2 {rel:.3g}, worst |err| {worst:.3g} of {np.abs(r).max():.3g}", flush=True)
    assert rel <= 1e-2, f"relative L2 error of the logits {rel:.3g}"
    assert worst <= 2e-2 * max(1.0, np.abs(r).max())
    ref_tok = ref.astype(np.float32).argmax(-1)
    for b in range(batch):
        if got_tokens[0, b] != ref_tok[b]:
            row = np.sort(r[b])
            assert row[-1] - row[-2] < 2e-2, f"row {b}: token differs with a clear margin"
    for layer in range(cfg["n_layers"]):
        kc, vc = dec.k_cache[layer].numpy(), untile_v_cache(dec.v_cache[layer].numpy())
        tol = 2e-2 if layer == 0 else 6e-2
        for b in range(batch):
            p = int(positions[b])
            ek = np.abs(kc[b, :, p].astype(np.float64) - ref_k[layer][b, :, p].astype(np.float64)).max()
            ev = np.abs(vc[b, :, p].astype(np.float64) - ref_v[layer][b, :, p].astype(np.float64)).max()
            assert ek <= tol and ev <= tol, f"layer {layer} row {b}: appended k/v off by {ek:.3g} / {ev:.3g}"


@pytest.mark.parametrize("batch", [1, 4, 9, 33])   # in-kernel reduction, second-stage epilogues, the unfused path
def test_qwen_14b_int8_shape_with_biases_and_act_order(hip, qwen_model, batch):
    _run_and_check(QWEN, qwen_model, batch)


@pytest.mark.parametrize("batch", [2, 9])
def test_biases_on_the_column_owner_kernel_at_70b_widths(hip, wide_model, batch):
    """q|k|v on the cut tiles with its RoPE / cache-append epilogue and o with the residual epilogue, biased."""
    _run_and_check(WIDE, wide_model, batch)
