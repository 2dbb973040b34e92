"""Greedy decode of a Llama-family GPTQ model on one GPU, driven through the
native loop ``mh_llama_decode`` (one call enqueues every kernel of the requested
steps).  Mirrors what the reference's cached server does per token
(examples/llama3_70b.py:394-398 -> Llama3LM.forward -> Top1Sampler) with a
preallocated KV cache, fused q|k|v and gate|up projections and on-device
sampling.
"""
import ctypes
import time
from ctypes import c_float, c_int, c_void_p

import numpy as np

from . import lib, synthetic
from .hip import memory
from .hip.tensor import HIPTensor


class LlamaConfig(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("n_layers", "hidden", "n_q_heads", "n_kv_heads", "head_dim", "ffn",
                                     "vocab", "group_size", "bits", "max_seq")] + [("rms_eps", c_float)]


class QLinear(ctypes.Structure):
    _fields_ = [("qweight", c_void_p), ("qzeros", c_void_p), ("scales", c_void_p), ("bias", c_void_p),
                ("perm", c_void_p)]


class LlamaLayer(ctypes.Structure):
    _fields_ = [("qkv", QLinear), ("o", QLinear), ("gate_up", QLinear), ("down", QLinear),
                ("input_norm", c_void_p), ("post_norm", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p)]


LLAMA3_70B = dict(n_layers=80, hidden=8192, n_q_heads=64, n_kv_heads=8, head_dim=128, ffn=28672,
                  vocab=128256, group_size=128, bits=4, rope_theta=5e5, rms_eps=1e-5)


def interleave_gate_up(qweight, qzeros, scales, bits=4):
    """Column order of the fused gate|up projection that the device path expects.

    ``[gate (ffn) | up (ffn)]`` becomes blocks of 256 columns holding 128 gate
    columns followed by the 128 up columns of the same positions, so one column
    tile of the product kernel sees both operands of ``silu(gate) * up``.  128 is
    a multiple of the 8 (or 4) columns packed into a ``qzeros`` word, so whole
    words move and nothing is repacked.
    """
    n = qweight.shape[1]
    ffn = n // 2
    assert ffn % 128 == 0, "ffn must be a multiple of 128"
    t = np.arange(ffn // 128)[:, None, None]
    c = np.arange(128)[None, None, :]
    part = np.arange(2)[None, :, None]            # 0 = gate, 1 = up
    cols = (part * ffn + t * 128 + c).reshape(-1)  # new column j takes old column cols[j]
    per = 32 // bits
    words = cols.reshape(-1, per)[:, 0] // per
    return qweight[:, cols], qzeros[:, words], scales[:, cols]


V_TILE = 64


def tile_v_cache(v: np.ndarray) -> np.ndarray:
    """``[B, KVH, T, D]`` (T a multiple of 64) to the layout the attention kernel reads,
    ``[B, KVH, T / 64, D, 64]``: positions contiguous, in tiles of 64, so that the 64
    positions x D values of one step of a wave are one piece of memory."""
    b, h, t, d = v.shape
    assert t % V_TILE == 0, f"cache length {t} must be a multiple of {V_TILE}"
    return np.ascontiguousarray(v.reshape(b, h, t // V_TILE, V_TILE, d).transpose(0, 1, 2, 4, 3))


def untile_v_cache(vt: np.ndarray) -> np.ndarray:
    """Inverse of :func:`tile_v_cache`: ``[B, KVH, T / 64, D, 64]`` to ``[B, KVH, T, D]``."""
    b, h, tiles, d, w = vt.shape
    return np.ascontiguousarray(vt.transpose(0, 1, 2, 4, 3).reshape(b, h, tiles * w, d))


def decode_attention(q, k_cache, vt_cache, positions, max_seq: int):
    """Attention of one new token per row over a preallocated cache (the core of
    examples/llama3_70b.py:77-113 for a decode step) through ``mh_attn_decode``.

    ``q [B, QH, 128]``, ``k_cache [B, KVH, max_seq, 128]``, ``vt_cache [B, KVH, max_seq / 64,
    128, 64]`` (:func:`tile_v_cache`), ``positions [B]`` int32 = index of the newest entry;
    all :class:`HIPTensor`.  Returns ``[B, QH, 128]``.
    """
    batch, qh, d = q._shape
    kvh = k_cache._shape[1]
    nbytes = lib.call("mh_attn_decode_workspace_bytes", batch, qh, kvh, d, max_seq)
    ws = _attention_workspace(nbytes, (batch, qh, kvh, d, max_seq))
    out = HIPTensor.allocate((batch, qh, d), q.dtype)
    lib.call("mh_attn_decode", None, q.data_ptr, k_cache.data_ptr, vt_cache.data_ptr, positions.data_ptr,
             out.data_ptr, batch, qh, kvh, d, max_seq, ws._pointer, ws._size)
    return out


_ATTN_WS = {}


def _attention_workspace(nbytes: int, key):
    """One workspace per call geometry, zero-filled once: the kernel leaves its counters at zero,
    but where the counters end and the records begin depends on the geometry, so a buffer shared
    between geometries would hand one call's records to the next as counters."""
    if key not in _ATTN_WS:
        mem = memory.HIPMemory(max(nbytes, 256))
        mem.reset()
        memory.synchronize()
        _ATTN_WS[key] = mem
    return _ATTN_WS[key]


class LlamaDecoder:
    """Owns the device tensors of one model and its KV cache."""

    def __init__(self, config: dict, batch_max: int, max_seq: int):
        self.config = dict(config)
        # the V cache is kept in tiles of 64 positions
        max_seq = (max_seq + 63) // 64 * 64
        self.batch_max, self.max_seq = batch_max, max_seq
        c = self.config
        self._cfg = LlamaConfig(c["n_layers"], c["hidden"], c["n_q_heads"], c["n_kv_heads"], c["head_dim"],
                                c["ffn"], c["vocab"], c["group_size"], c["bits"], max_seq, c["rms_eps"])
        h = c_void_p()
        lib.call("mh_llama_create", ctypes.byref(h), ctypes.byref(self._cfg))
        self._handle = h.value
        self._keep = []          # device tensors referenced by the native model
        self.k_cache, self.v_cache = [], []
        self._scratch = {}
        self._graph_io = {}      # batch -> (tokens, positions, out_tokens) a recorded step is bound to
        self._graph_stream = None
        cos, sin = synthetic.rope_tables(c["head_dim"], max_seq, c["rope_theta"])
        self.cos, self.sin = HIPTensor.from_numpy(cos), HIPTensor.from_numpy(sin)

    def __del__(self):
        try:
            lib.call("mh_llama_destroy", self._handle)
        except Exception:
            pass

    # ---- weights ------------------------------------------------------------------------------
    def _alloc_cache(self):
        c = self.config
        # K is [B, KVH, T, D]; V is kept with positions contiguous, in tiles of 64 (tile_v_cache), for the
        # P.V matrix product
        k_shape = (self.batch_max, c["n_kv_heads"], self.max_seq, c["head_dim"])
        v_shape = (self.batch_max, c["n_kv_heads"], self.max_seq // V_TILE, c["head_dim"], V_TILE)
        kc, vc = HIPTensor.allocate(k_shape, "float16"), HIPTensor.allocate(v_shape, "float16")
        kc._memory.reset()
        vc._memory.reset()
        return kc, vc

    def _set_layer(self, index, linears, input_norm, post_norm, k_cache, v_cache):
        def ql(t):   # (qweight, qzeros, scales[, bias[, perm]]); None where absent
            extra = [e.data_ptr if e is not None else None for e in t[3:5]] + [None, None]
            return QLinear(t[0].data_ptr, t[1].data_ptr, t[2].data_ptr, extra[0], extra[1])
        layer = LlamaLayer(ql(linears["qkv"]), ql(linears["o"]), ql(linears["gate_up"]), ql(linears["down"]),
                           input_norm.data_ptr, post_norm.data_ptr, k_cache.data_ptr, v_cache.data_ptr)
        lib.call("mh_llama_set_layer", self._handle, index, ctypes.byref(layer))
        self._keep.append((linears, input_norm, post_norm))
        self.k_cache.append(k_cache)
        self.v_cache.append(v_cache)

    def _set_globals(self, embed, lm_head, final_norm):
        lib.call("mh_llama_set_globals", self._handle, embed.data_ptr, lm_head.data_ptr, final_norm.data_ptr,
                 self.cos.data_ptr, self.sin.data_ptr)
        self._keep.append((embed, lm_head, final_norm))
        self.embed, self.lm_head, self.final_norm = embed, lm_head, final_norm

    def linear_shapes(self):
        c = self.config
        d = c["head_dim"]
        return {"qkv": (c["hidden"], (c["n_q_heads"] + 2 * c["n_kv_heads"]) * d),
                "o": (c["n_q_heads"] * d, c["hidden"]),
                "gate_up": (c["hidden"], 2 * c["ffn"]),
                "down": (c["ffn"], c["hidden"])}

    def load_synthetic(self, seed: int = 0, prefill: int = 0, scale_std: float = 0.02, zero_range=(6, 9)):
        """Random-init weights generated on the device; KV cache prefilled with N(0, 1).  ``scale_std``,
        ``zero_range``: spread of the group scales and range of the zero points.  The defaults are the
        benchmark recipe, whose weights have a mean of -1 step (sub-words uniform in 0..15 against zero
        points 6..9) and sums over 8192 terms in the hundreds: fine for timing, but over 80 layers the
        common-mode part of the residual stream grows by about 2000 per layer until fp16 overflows, so a
        run that is checked for its values takes finer scales and zero points 6..7 (mean-free weights)."""
        c = self.config
        per = 32 // c["bits"]
        g = c["group_size"]
        for l in range(c["n_layers"]):
            linears = {}
            for j, (name, (k, n)) in enumerate(self.linear_shapes().items()):
                s0 = (seed * 100003 + l) * 16 + j * 3
                qw = HIPTensor.allocate((k // per, n), "int32")
                qz = HIPTensor.allocate((k // g, n // per), "int32")
                sc = HIPTensor.allocate((k // g, n), "float16")
                lib.call("mh_synth_u32", None, qw.data_ptr, (k // per) * n, s0)
                lib.call("mh_synth_subwords", None, qz.data_ptr, (k // g) * (n // per), c["bits"], zero_range[0],
                         zero_range[1], s0 + 1)
                lib.call("mh_synth_normal", None, sc.data_ptr, (k // g) * n, 0.0, scale_std, 1, scale_std / 20, s0 + 2, 0)
                linears[name] = (qw, qz, sc)
            norms = []
            for j in range(2):
                w = HIPTensor.allocate((c["hidden"],), "float16")
                lib.call("mh_synth_normal", None, w.data_ptr, c["hidden"], 1.0, 0.1, 0, 0.0, s0 + 10 + j, 0)
                norms.append(w)
            kc, vc = self._alloc_cache()
            if prefill:
                for t, sd in ((kc, 13), (vc, 14)):
                    lib.call("mh_synth_normal", None, t.data_ptr, int(np.prod(t._shape)), 0.0, 1.0, 0, 0.0,
                             s0 + sd, 0)
            self._set_layer(l, linears, norms[0], norms[1], kc, vc)
        embed = HIPTensor.allocate((c["vocab"], c["hidden"]), "float16")
        lm_head = HIPTensor.allocate((c["vocab"], c["hidden"]), "float16")
        final_norm = HIPTensor.allocate((c["hidden"],), "float16")
        n = c["vocab"] * c["hidden"]
        lib.call("mh_synth_normal", None, embed.data_ptr, n, 0.0, 0.02, 0, 0.0, seed * 7 + 1, 0)
        lib.call("mh_synth_normal", None, lm_head.data_ptr, n, 0.0, 0.02, 0, 0.0, seed * 7 + 2, 0)
        lib.call("mh_synth_normal", None, final_norm.data_ptr, c["hidden"], 1.0, 0.1, 0, 0.0, seed * 7 + 3, 0)
        self._set_globals(embed, lm_head, final_norm)
        memory.synchronize()

    def load_host(self, model: dict, k_cache=None, v_cache=None):
        """Uploads a model given as numpy arrays (the layout of ``oracle.decode``)."""
        from .quantize import gptq as host_gptq
        bits, group = self.config["bits"], self.config["group_size"]
        for l, layer in enumerate(model["layers"]):
            linears = {}
            for name in ("qkv", "o", "gate_up", "down"):
                # (qweight, qzeros, scales, group_size[, bias[, g_idx]]): the buffers of the reference's
                # QLinear / QLinearWithBias (examples/qwen1_5_int8.py:276-305)
                w = layer[name]
                qweight, qzeros, scales = w[:3]
                bias = w[4] if len(w) > 4 else None
                g_idx = w[5] if len(w) > 5 else None
                perm = None
                if g_idx is not None and not np.array_equal(np.asarray(g_idx), np.arange(len(g_idx)) // group):
                    # act-order: rows sorted by group once, here on the host; the loop gathers the activations
                    res = host_gptq.sort_rows_by_group(qweight, np.asarray(g_idx), bits, group)
                    assert res is not None, f"{name}: groups of uneven size are not served by the decode loop"
                    qweight, perm = res
                if name == "gate_up":
                    cols_before = qweight.shape[1]
                    qweight, qzeros, scales = interleave_gate_up(qweight, qzeros, scales, bits=bits)
                    if bias is not None:   # the same column order
                        ffn = cols_before // 2
                        bias = np.stack([bias[:ffn].reshape(-1, 128), bias[ffn:].reshape(-1, 128)], axis=1).reshape(-1)
                dev = [HIPTensor.from_numpy(np.ascontiguousarray(a)) for a in (qweight, qzeros, scales)]
                dev.append(None if bias is None else HIPTensor.from_numpy(np.ascontiguousarray(bias, np.float16)))
                dev.append(None if perm is None else HIPTensor.from_numpy(np.ascontiguousarray(perm, np.int32)))
                linears[name] = tuple(dev)
            kc, vc = self._alloc_cache()
            if k_cache is not None:   # host caches are [B, KVH, T, D] with T <= max_seq
                t = k_cache[l].shape[2]
                kpad = np.zeros(kc._shape, np.float16)
                kpad[:, :, :t] = k_cache[l]
                vpad = np.zeros(kc._shape, np.float16)
                vpad[:, :, :t] = v_cache[l]
                kc.copy_from_numpy(kpad)
                vc.copy_from_numpy(tile_v_cache(vpad))
            self._set_layer(l, linears, HIPTensor.from_numpy(layer["input_norm"]),
                            HIPTensor.from_numpy(layer["post_norm"]), kc, vc)
        self._set_globals(HIPTensor.from_numpy(model["embed"]), HIPTensor.from_numpy(model["lm_head"]),
                          HIPTensor.from_numpy(model["final_norm"]))

    # ---- decode ---------------------------------------------------------------------------------
    def _scratch_for(self, batch):
        if batch not in self._scratch:
            nbytes = lib.call("mh_llama_scratch_bytes", self._handle, batch)
            mem = memory.HIPMemory(nbytes)
            mem.reset()
            memory.synchronize()
            self._scratch[batch] = mem
        return self._scratch[batch]

    def decode(self, tokens, positions, n_steps: int, want_logits: bool = False, stream=None, graph: bool = False):
        """Greedy-decodes ``n_steps`` tokens for ``len(tokens)`` rows.

        With ``graph`` one step is recorded into a HIP graph the first time a batch
        size is seen and replayed per token (``mh_llama_decode_graph``), on a stream
        and on token / position / output buffers the decoder keeps for that batch size.
        Returns ``(out_tokens [n_steps, B] int32, logits of the last step or None)``.
        """
        batch = len(tokens)
        assert batch <= self.batch_max
        assert int(np.max(positions)) + n_steps <= self.max_seq, "KV cache too short"
        logits = HIPTensor.allocate((batch, self.config["vocab"]), "float16") if want_logits else None
        scratch = self._scratch_for(batch)
        if graph:
            if batch not in self._graph_io:
                self._graph_io[batch] = (HIPTensor.allocate((batch,), "int32"), HIPTensor.allocate((batch,), "int32"),
                                         HIPTensor.allocate((self.max_seq, batch), "int32"))
            if self._graph_stream is None:
                self._graph_stream = memory.create_stream()
            tok, pos, out = self._graph_io[batch]
            tok.copy_from_numpy(np.asarray(tokens, np.int32))
            pos.copy_from_numpy(np.asarray(positions, np.int32))
            lib.call("mh_llama_decode_graph", self._handle, stream or self._graph_stream, batch, tok.data_ptr,
                     pos.data_ptr, n_steps, out.data_ptr, logits.data_ptr if logits else None, scratch._pointer,
                     scratch._size)
            result = out.numpy()[:n_steps].copy()
        else:
            tok = HIPTensor.from_numpy(np.asarray(tokens, np.int32))
            pos = HIPTensor.from_numpy(np.asarray(positions, np.int32))
            out = HIPTensor.allocate((n_steps, batch), "int32")
            lib.call("mh_llama_decode", self._handle, stream, batch, tok.data_ptr, pos.data_ptr, n_steps,
                     out.data_ptr, logits.data_ptr if logits else None, scratch._pointer, scratch._size)
            result = out.numpy()
        return result, (logits.numpy() if logits else None)

    def norm_clamped(self, batch: int) -> bool:
        """True when a fused residual + norm launch at this batch size has held an ``h * norm_weight``
        at the fp16 limit since the decoder was built (``mh_llama_norm_clamped``): the steps since
        then differ from the reference's in that channel and carry no parity claim."""
        flag = ctypes.c_int(0)
        lib.call("mh_llama_norm_clamped", self._handle, None, batch, self._scratch_for(batch)._pointer,
                 ctypes.byref(flag))
        return bool(flag.value)

    def weight_bytes_per_token(self, batch: int, context: int) -> int:
        """Algorithmic HBM bytes one decode step has to move."""
        c = self.config
        g, bits = c["group_size"], c["bits"]
        total = 0
        for k, n in self.linear_shapes().values():
            total += k * n * bits // 8 + (k // g) * n * 2 + (k // g) * (n * bits // 32) * 4
        total *= c["n_layers"]
        total += c["vocab"] * c["hidden"] * 2                                   # lm_head
        total += c["n_layers"] * batch * 2 * context * c["n_kv_heads"] * c["head_dim"] * 2   # KV read
        return total


def bench_tokens_per_second(batches=(1, 8, 32), context=2048, tokens=128, log=print, config=None, graph=False,
                            finite=True):
    """Config 4: 70B-shape GPTQ decode, prefilled KV cache, greedy decode.

    ``finite``: group scales 16 times finer than the benchmark recipe and zero points 6..7, so that the
    activations of all 80 layers stay finite (with the recipe as given the residual stream overflows fp16
    after a few layers and the rest of the run multiplies NaNs: the same launches and bytes, but not the
    operand values a model would have).  False times the recipe as given."""
    cfg = dict(config or LLAMA3_70B)
    bmax = max(batches)
    t0 = time.time()
    dec = LlamaDecoder(cfg, bmax, context + tokens + 8)
    if finite and cfg["bits"] == 8:
        # 8-bit sub-words: zero points in the middle of the range and steps 16 times finer again
        dec.load_synthetic(seed=1, prefill=context, scale_std=0.02 / 256, zero_range=(126, 127))
    elif finite:
        dec.load_synthetic(seed=1, prefill=context, scale_std=0.02 / 16, zero_range=(6, 7))
    else:
        dec.load_synthetic(seed=1, prefill=context)
    log(f"decode: model + cache resident after {time.time() - t0:.1f} s")
    results = []
    for b in batches:
        toks = np.arange(b, dtype=np.int32) * 17 + 5
        pos = np.full(b, context, np.int32)
        dec.decode(toks, pos, 12, graph=graph)         # warm-up: the recording of the step, and the part's clocks
        memory.synchronize()
        # host clock around a call that ends in a device synchronisation: the graph
        # variant runs on the decoder's own stream, where null-stream events do not see it
        t0 = time.perf_counter()
        out, _ = dec.decode(toks, pos, tokens, graph=graph)
        ms = (time.perf_counter() - t0) * 1e3
        tps = b * tokens / (ms * 1e-3)
        gb = dec.weight_bytes_per_token(b, context + tokens // 2) / 1e9
        results.append({"batch": b, "context": context, "tokens": tokens, "graph": bool(graph),
                        "finite_activations": bool(finite), "distinct_tokens": int(len(np.unique(out))),
                        "ms_per_token": round(ms / tokens, 3),
                        "tok_s": round(tps, 1), "algorithmic_gb_per_step": round(gb, 2),
                        "hbm_gbps": round(gb / (ms / tokens * 1e-3), 1)})
        log(f"decode batch {b}: {ms / tokens:.3f} ms/token, {tps:.1f} tok/s")
    return results


if __name__ == "__main__":
    import argparse
    import json

    ap = argparse.ArgumentParser(description="Llama-3-70B-shape GPTQ decode on one GPU: tokens per second")
    ap.add_argument("--batches", default="1,8,32")
    ap.add_argument("--tokens", type=int, default=64)
    ap.add_argument("--graph", action="store_true", help="replay one recorded step per token (HIP graph)")
    ap.add_argument("--recipe-as-given", action="store_true",
                    help="weights exactly as the benchmark recipe draws them (activations overflow fp16 after a few layers)")
    ap.add_argument("--bits", type=int, default=4, choices=(4, 8),
                    help="bit width of the packed weights (8: what the reference's own example ships)")
    cli = ap.parse_args()
    print(json.dumps(bench_tokens_per_second(batches=tuple(int(b) for b in cli.batches.split(",")),
                                             tokens=cli.tokens, log=lambda *a: print(*a, flush=True),
                                             graph=cli.graph, finite=not cli.recipe_as_given,
                                             config=dict(LLAMA3_70B, bits=cli.bits))))
