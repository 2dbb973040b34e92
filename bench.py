#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One *step* is one pass of the decode hot path over one layer's worth of
Llama-3-70B-shape GPTQ 4-bit weights at M = 1: the four quantized linears
(qkv 8192x10240, o 8192x8192, gate|up 8192x57344, down 28672x8192, group 128)
through ``mh_gptq_matmul`` (the library's dispatch; ``--entry`` times the VALU
GEMV or the MFMA kernel explicitly).  ``--layers`` distinct weight sets (default 6,
2.6 GB -- ten times the 256 MB Infinity Cache) are generated on the device and
cycled, so every step streams its weights from HBM.  The value reported is
algorithmic bytes per second: packed weights + scales + zero points +
activations + outputs, each counted once.

Prints ONE JSON line with the headline metric, its roofline fraction (HBM,
8 TB/s) and the CPU baseline: the C restatement of the reference's arithmetic
(``oracle/c``) timed on this machine's host cores on the same layer, whose
result the GPU output is also checked against.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# HBM bytes per launch of the dominant kernel (the gate|up product) come from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE, in KiB per
# dispatch, scaled by what the same counters read for the 1 GiB copy kernel of
# --calibrate-copy).  A process cannot read those counters itself, so the figure is
# read from the committed summary of those runs, which carries a line
#   bench-traffic: entry=<entry point> kernel=<name> bytes_per_launch=<n> commit=<hash>
# and is reported with the commit it was measured at (null if the line is missing).
TRAFFIC_SUMMARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                               "gptq_decode_gemvs_llama70b_m1.md")


def measured_traffic(entry):
    import re
    try:
        text = open(TRAFFIC_SUMMARY).read()
    except OSError:
        return None, None
    for m in re.finditer(r"bench-traffic:\s*entry=(\S+)\s+kernel=(\S+)\s+bytes_per_launch=(\d+)\s+commit=(\S+)", text):
        if m.group(1) == entry:
            return int(m.group(3)), m.group(4)
    return None, None


HBM_PEAK_GBPS = 8000.0
INT8_PEAK_TOPS = 5000.0

# (name, K, N) of the fused per-layer projections at Llama-3-70B shape
HIDDEN, Q_HEADS, KV_HEADS, HEAD, FFN = 8192, 64, 8, 128, 28672
LINEARS = [
    ("qkv_proj", HIDDEN, (Q_HEADS + 2 * KV_HEADS) * HEAD),
    ("o_proj", Q_HEADS * HEAD, HIDDEN),
    ("gate_up_proj", HIDDEN, 2 * FFN),
    ("down_proj", FFN, HIDDEN),
]
GROUP, BITS = 128, 4


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def linear_bytes(m, k, n, group=GROUP, bits=BITS):
    """Algorithmic bytes of one quantized linear (every operand once)."""
    groups = k // group
    return k * n * bits // 8 + groups * n * 2 + groups * (n * bits // 32) * 4 + m * k * 2 + m * n * 2


class DeviceLinear:
    """One GPTQ weight set generated on the device."""

    def __init__(self, lib, HIPTensor, k, n, seed, bits=BITS):
        per = 32 // bits
        groups = k // GROUP
        self.k, self.n, self.bits = k, n, bits
        self.qweight = HIPTensor.allocate((k // per, n), "int32")
        self.qzeros = HIPTensor.allocate((groups, n // per), "int32")
        self.scales = HIPTensor.allocate((groups, n), "float16")
        zlo, zhi = (6, 9) if bits == 4 else (120, 135)
        lib.call("mh_synth_u32", None, self.qweight.data_ptr, (k // per) * n, seed * 3 + 0)
        lib.call("mh_synth_subwords", None, self.qzeros.data_ptr, groups * (n // per), bits, zlo, zhi, seed * 3 + 1)
        lib.call("mh_synth_normal", None, self.scales.data_ptr, groups * n, 0.0, 0.02, 1, 1e-3, seed * 3 + 2, 0)


def run_gemv(lib, x, lin, out, ws, m=1, entry="mh_gptq_matmul"):
    lib.call(entry, None, x.data_ptr, lin.qweight.data_ptr, lin.qzeros.data_ptr, lin.scales.data_ptr, None,
             out.data_ptr, m, lin.n, lin.k, GROUP, getattr(lin, "bits", BITS), ws._pointer, ws._size)


def bench_int8(lib, HIPTensor, memory, n, iters=20):
    """W8A8 GEMM, M = 2048, K = 4096 (fp16 output + scale epilogue)."""
    m, k = 2048, 4096
    a = HIPTensor.allocate((m, k), "int8")
    sa = HIPTensor.allocate((m,), "float32")
    sw = HIPTensor.allocate((n,), "float32")
    out = HIPTensor.allocate((m, n), "float16")
    lib.call("mh_synth_i8", None, a.data_ptr, m * k, -127, 127, 11)
    lib.call("mh_synth_normal", None, sa.data_ptr, m, 0.0, 0.01, 1, 0.0, 12, 2)
    lib.call("mh_synth_normal", None, sw.data_ptr, n, 0.0, 0.005, 1, 0.0, 13, 2)
    ws = []
    for i in range(4):  # rotate weight buffers
        w = HIPTensor.allocate((n, k), "int8")
        lib.call("mh_synth_i8", None, w.data_ptr, n * k, -127, 127, 20 + i)
        ws.append(w)

    def go(i):
        lib.call("mh_i8_gemm", None, a.data_ptr, ws[i % 4].data_ptr, sa.data_ptr, sw.data_ptr, out.data_ptr,
                 None, m, n, k)
    us = _time_launches(memory, go, iters=iters, warmup=4)
    tops = 2.0 * m * n * k / us / 1e6
    return {"M": m, "N": n, "K": k, "us": round(us, 2), "tops": round(tops, 1),
            "frac_of_peak": round(tops / INT8_PEAK_TOPS, 4)}


def _settle(memory, fn, ms):
    """Runs fn(0), fn(1), ... for at least `ms` milliseconds, untimed: the part needs some tens of
    milliseconds of load to reach its steady clocks (the headline step measures 99.7 us when timed
    right after 20 warm-up steps and 92.1-92.7 us after 0.3 s of the same work)."""
    t0, i = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(16):
            fn(i)
            i += 1
        memory.synchronize()
    return i


SETTLE_MS = 150.0   # untimed load before every timed section (--settle-ms)


def _time_launches(memory, fn, iters=200, warmup=10):
    _settle(memory, fn, SETTLE_MS)
    for i in range(warmup):
        fn(i)
    memory.synchronize()
    e0, e1 = memory.Event(), memory.Event()
    e0.record()
    for i in range(iters):
        fn(i)
    e1.record()
    e1.synchronize()
    return e0.elapsed_ms(e1) * 1e3 / iters


def bench_rowwise(lib, HIPTensor, memory):
    """Config 3: RMSNorm [16, 4096], RoPE [16, 1, 32, 128] at random positions, softmax
    and row-sum over [512, ctx]; microseconds per launch and algorithmic GB/s (every
    operand once).  The working sets are a few MB and stay in cache: these lines show
    launch latency, not HBM."""
    import numpy as np
    from minit_amd import synthetic
    out = []

    def add(name, us, nbytes):
        out.append({"kernel": name, "us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1)})

    f16 = 0
    x = HIPTensor.allocate((16, 4096), "float16")
    w = HIPTensor.allocate((4096,), "float16")
    y = HIPTensor.allocate((16, 4096), "float16")
    lib.call("mh_synth_normal", None, x.data_ptr, 16 * 4096, 0.0, 1.0, 0, 0.0, 31, 0)
    lib.call("mh_synth_normal", None, w.data_ptr, 4096, 1.0, 0.1, 0, 0.0, 32, 0)
    us = _time_launches(memory, lambda i: lib.call("mh_rms_norm", None, x.data_ptr, w.data_ptr, y.data_ptr,
                                                    16, 4096, 1, 1e-6, f16))
    add("rms_norm [16,4096]", us, 2 * 16 * 4096 * 2 + 4096 * 2)

    cos, sin = synthetic.rope_tables(128, 4096, 1e6)
    dcos, dsin = HIPTensor.from_numpy(cos), HIPTensor.from_numpy(sin)
    pos = HIPTensor.from_numpy(np.random.default_rng(33).integers(0, 4096, size=(16, 1)).astype(np.int32))
    q = HIPTensor.allocate((16, 1, 32, 128), "float16")
    qo = HIPTensor.allocate((16, 1, 32, 128), "float16")
    lib.call("mh_synth_normal", None, q.data_ptr, 16 * 32 * 128, 0.0, 1.0, 0, 0.0, 34, 0)
    us = _time_launches(memory, lambda i: lib.call("mh_rope", None, q.data_ptr, dcos.data_ptr, dsin.data_ptr,
                                                    pos.data_ptr, qo.data_ptr, 16, 1, 32, 128, f16))
    add("rope [16,1,32,128]", us, 2 * 16 * 32 * 128 * 2 + 16 * 64 * 4 * 2)

    for ctx in (1024, 4096):
        sc = HIPTensor.allocate((512, ctx), "float16")
        so = HIPTensor.allocate((512, ctx), "float16")
        rs = HIPTensor.allocate((512, 1), "float16")
        lib.call("mh_synth_normal", None, sc.data_ptr, 512 * ctx, 0.0, 3.0, 0, 0.0, 35, 0)
        us = _time_launches(memory, lambda i: lib.call("mh_softmax", None, sc.data_ptr, so.data_ptr, 512, ctx, 1, f16))
        add(f"softmax [512,{ctx}]", us, 2 * 512 * ctx * 2)
        us = _time_launches(memory, lambda i: lib.call("mh_sum", None, sc.data_ptr, rs.data_ptr, 512, ctx, 1, f16))
        add(f"row_sum [512,{ctx}]", us, 512 * ctx * 2 + 512 * 2)
    del sc, so, rs

    # The same kernels on operands beyond the 256 MB Infinity Cache (512 MB each): these
    # lines are the HBM-bound ones.
    rows, width = 32768, 8192
    big = HIPTensor.allocate((rows, width), "float16")
    big_out = HIPTensor.allocate((rows, width), "float16")
    w8 = HIPTensor.allocate((width,), "float16")
    col = HIPTensor.allocate((rows, 1), "float16")
    lib.call("mh_synth_normal", None, big.data_ptr, rows * width, 0.0, 1.0, 0, 0.0, 36, 0)
    lib.call("mh_synth_normal", None, w8.data_ptr, width, 1.0, 0.1, 0, 0.0, 37, 0)
    nb = rows * width * 2
    us = _time_launches(memory, lambda i: lib.call("mh_rms_norm", None, big.data_ptr, w8.data_ptr, big_out.data_ptr,
                                                    rows, width, 1, 1e-6, f16), iters=20, warmup=3)
    add(f"rms_norm [{rows},{width}]", us, 2 * nb + width * 2)
    us = _time_launches(memory, lambda i: lib.call("mh_softmax", None, big.data_ptr, big_out.data_ptr, rows, width, 1,
                                                    f16), iters=20, warmup=3)
    add(f"softmax [{rows},{width}]", us, 2 * nb)
    us = _time_launches(memory, lambda i: lib.call("mh_sum", None, big.data_ptr, col.data_ptr, rows, width, 1, f16),
                        iters=20, warmup=3)
    add(f"row_sum [{rows},{width}]", us, nb + rows * 2)
    toks, heads = rows * width // (64 * 128), 64
    pos = HIPTensor.from_numpy(np.random.default_rng(38).integers(0, 4096, size=(toks, 1)).astype(np.int32))
    us = _time_launches(memory, lambda i: lib.call("mh_rope", None, big.data_ptr, dcos.data_ptr, dsin.data_ptr,
                                                    pos.data_ptr, big_out.data_ptr, toks, 1, heads, 128, f16),
                        iters=20, warmup=3)
    add(f"rope [{toks},1,{heads},128]", us, 2 * nb + toks * 64 * 4 * 2)
    return out


def bench_small_configs(lib, HIPTensor, memory, ws):
    """Config 0 (GEMV 4096x4096) and config 1 (Mistral-7B MLP block: gate|up 4096 ->
    2 x 14336 with the SiLU*up epilogue, down 14336 -> 4096) at M in {1, 8, 32, 128};
    weight sets rotated over more than the 256 MB Infinity Cache."""
    res = {}
    hidden, ffn = 4096, 14336
    sets = 16  # x 8.7 MB (config 0) / x 91.5 MB (config 1)
    lin0 = [DeviceLinear(lib, HIPTensor, hidden, hidden, 500 + i) for i in range(32)]
    x0 = HIPTensor.allocate((1, hidden), "float16")
    lib.call("mh_synth_normal", None, x0.data_ptr, hidden, 0.0, 1.0, 0, 0.0, 41, 0)
    y0 = HIPTensor.allocate((1, hidden), "float16")
    us = _time_launches(memory, lambda i: run_gemv(lib, x0, lin0[i % 32], y0, ws), iters=128, warmup=32)
    res["gemv_cfg0"] = {"M": 1, "K": hidden, "N": hidden, "us": round(us, 2),
                        "gbps": round(linear_bytes(1, hidden, hidden) / us / 1e3, 1)}
    del lin0
    gate_up = [DeviceLinear(lib, HIPTensor, hidden, 2 * ffn, 600 + i) for i in range(sets // 4)]
    down = [DeviceLinear(lib, HIPTensor, ffn, hidden, 700 + i) for i in range(sets // 4)]
    block = []
    for m in (1, 8, 32, 128):
        x = HIPTensor.allocate((m, hidden), "float16")
        lib.call("mh_synth_normal", None, x.data_ptr, m * hidden, 0.0, 1.0, 0, 0.0, 42, 0)
        h = HIPTensor.allocate((m, ffn), "float16")
        y = HIPTensor.allocate((m, hidden), "float16")

        # gate|up through mh_gptq_matmul_silu_pairs: up to 32 rows one launch with SiLU*up in its
        # reduction, above that the fused product and one pass over it; then down
        ws_pairs = memory.workspace(max(lib.call("mh_gptq_silu_pairs_workspace_bytes", m, 2 * ffn, hidden, GROUP, BITS),
                                        ws._size))

        def step(i, ws_pairs=ws_pairs):
            gu, dn = gate_up[i % len(gate_up)], down[i % len(down)]
            lib.call("mh_gptq_matmul_silu_pairs", None, x.data_ptr, gu.qweight.data_ptr, gu.qzeros.data_ptr,
                     gu.scales.data_ptr, h.data_ptr, m, 2 * ffn, hidden, GROUP, BITS, ws_pairs._pointer, ws_pairs._size)
            run_gemv(lib, h, dn, y, ws_pairs, m=m)
        us = _time_launches(memory, step, iters=40, warmup=4)
        nbytes = linear_bytes(m, hidden, 2 * ffn) - m * ffn * 2 + linear_bytes(m, ffn, hidden)
        block.append({"M": m, "us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                      "tflops": round(2.0 * m * 3 * hidden * ffn / us / 1e6, 2)})
    res["mlp_block_cfg1"] = block
    del gate_up, down
    # the unquantized lm_head of the decode loop: fp16 [vocab, hidden] (2.1 GB, streamed once per launch)
    vocab, hid = 128256, 8192
    w = HIPTensor.allocate((vocab, hid), "float16")
    lib.call("mh_synth_normal", None, w.data_ptr, vocab * hid, 0.0, 0.02, 0, 0.0, 43, 0)
    head = []
    for m in (1, 4, 8, 32):
        x = HIPTensor.allocate((m, hid), "float16")
        lib.call("mh_synth_normal", None, x.data_ptr, m * hid, 0.0, 1.0, 0, 0.0, 44, 0)
        y = HIPTensor.allocate((m, vocab), "float16")
        us = _time_launches(memory, lambda i: lib.call("mh_f16_matmul_nk", None, x.data_ptr, w.data_ptr, y.data_ptr,
                                                       m, vocab, hid), iters=10, warmup=2)
        nbytes = 2 * (vocab * hid + m * hid + m * vocab)
        head.append({"M": m, "us": round(us, 1), "gbps": round(nbytes / us / 1e3, 1)})
    res["lm_head_f16"] = head
    del w
    # the decode attention on its own at the 70B head geometry, cache filled to 2048 positions
    # (K and V read once per launch; six cache sets cycled, more than the 256 MB of the last-level cache
    # from 8 rows on)
    qh, kvh, d, ctx, max_seq, sets = 64, 8, 128, 2048, 2112, 6
    attn = []
    for batch in (1, 8, 32):
        n = batch * kvh * max_seq * d
        ks = [HIPTensor.allocate((batch, kvh, max_seq, d), "float16") for _ in range(sets)]
        vs = [HIPTensor.allocate((batch, kvh, max_seq // 64, d, 64), "float16") for _ in range(sets)]
        for i in range(sets):
            lib.call("mh_synth_normal", None, ks[i].data_ptr, n, 0.0, 1.0, 0, 0.0, 50 + i, 0)
            lib.call("mh_synth_normal", None, vs[i].data_ptr, n, 0.0, 1.0, 0, 0.0, 60 + i, 0)
        q = HIPTensor.allocate((batch, qh, d), "float16")
        lib.call("mh_synth_normal", None, q.data_ptr, batch * qh * d, 0.0, 1.0, 0, 0.0, 70, 0)
        pos = HIPTensor.from_numpy(np.full(batch, ctx - 1, np.int32))
        out = HIPTensor.allocate((batch, qh, d), "float16")
        nws = lib.call("mh_attn_decode_workspace_bytes", batch, qh, kvh, d, max_seq)
        aws = HIPTensor.allocate((nws,), "int8")
        aws._memory.reset()
        memory.synchronize()
        us = _time_launches(memory, lambda i: lib.call("mh_attn_decode", None, q.data_ptr, ks[i % sets].data_ptr,
                                                       vs[i % sets].data_ptr, pos.data_ptr, out.data_ptr, batch, qh,
                                                       kvh, d, max_seq, aws.data_ptr, nws), iters=200, warmup=10)
        nbytes = batch * 2 * ctx * kvh * d * 2
        attn.append({"batch": batch, "context": ctx, "us": round(us, 1), "gbps": round(nbytes / us / 1e3, 1)})
        del ks, vs
    res["attention_70b"] = attn
    return res


def bench_int8_library(n, iters=50):
    """The vendor library's int8 GEMM (torch._int_mm, int32 output, no scale epilogue)
    on the W8A8 shapes and operand layout of bench_int8, as a yardstick for what this
    problem size allows on the part.  Comparison only: nothing of the library's path."""
    import torch
    m, k = 2048, 4096
    a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda:0")
    ws = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda:0").t() for _ in range(4)]
    for w in ws:
        torch._int_mm(a, w)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        torch._int_mm(a, ws[i % 4])
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / iters
    tops = 2.0 * m * n * k / us / 1e6
    return {"M": m, "N": n, "K": k, "us": round(us, 2), "tops": round(tops, 1),
            "frac_of_peak": round(tops / INT8_PEAK_TOPS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--layers", type=int, default=6, help="distinct weight sets cycled through")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--shapes-only", action="store_true",
                    help="of the extras, keep only the per-shape GEMV breakdown")
    ap.add_argument("--entry", default="mh_gptq_matmul", choices=["mh_gptq_matmul", "mh_gptq_gemv", "mh_gptq_gemm"],
                    help="C-ABI entry point timed: the library's own dispatch (default), the VALU GEMV, "
                         "or the MFMA kernel")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only the plain copy kernel (1 GiB read + 1 GiB write per launch) that the "
                         "FETCH_SIZE / WRITE_SIZE counters are scaled against, then exit")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed load (the step itself) before the warm-up steps, so that the timed steps run at the "
                         "part's steady clocks; half of it before every timed section of the extras; 0 switches it off")
    ap.add_argument("--int8-library", action="store_true",
                    help="time the vendor library's int8 GEMM (torch._int_mm) on the W8A8 shapes, then exit")
    ap.add_argument("--rowwise-only", action="store_true",
                    help="time only the row-wise kernels (RMSNorm, RoPE, softmax, row sum) and print their lines")
    ap.add_argument("--small-configs-only", action="store_true",
                    help="run only config 0 (GEMV 4096x4096), config 1 (Mistral-shape MLP block at 1 to 128 rows) and "
                         "the lm_head and decode-attention lines, then exit")
    ap.add_argument("--int8-only", action="store_true",
                    help="run only the W8A8 GEMM lines (M=2048, K=4096, N in {4096, 11008}), then exit")
    args = ap.parse_args()
    if args.int8_library:  # before this repository's library is loaded: torch brings a HIP runtime of its own
        print(json.dumps({"int8_gemm_vendor_library": [bench_int8_library(n) for n in (4096, 11008)]}))
        return
    ENTRY = args.entry
    global SETTLE_MS
    SETTLE_MS = args.settle_ms / 2
    if args.gpus != 1:
        log(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
            "(no collectives or sharding in this path).")
        sys.exit(2)

    from minit_amd import lib
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor

    lib.cdll()
    if lib.device_count() < 1:
        log("bench.py: no HIP device visible")
        sys.exit(1)
    info = lib.device_info()
    log("device:", info)

    if args.calibrate_copy:
        nbytes = 1 << 30
        src, dst = memory.HIPMemory(nbytes), memory.HIPMemory(nbytes)
        src.reset()
        dst.reset()
        memory.synchronize()
        e0, e1 = memory.Event(), memory.Event()
        e0.record()
        for _ in range(5):
            lib.call("mh_copy_kernel", None, src._pointer, dst._pointer, nbytes)
        e1.record()
        e1.synchronize()
        us = e0.elapsed_ms(e1) * 1e3 / 5
        print(json.dumps({"kernel": "copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes,
                          "us": round(us, 1), "gbps_read_plus_write": round(2 * nbytes / us / 1e3, 1)}))
        return

    if args.rowwise_only:
        print(json.dumps({"rowwise_cfg3": bench_rowwise(lib, HIPTensor, memory)}))
        return

    if args.small_configs_only:
        print(json.dumps(bench_small_configs(lib, HIPTensor, memory, memory.workspace(64 << 20))))
        return

    if args.int8_only:
        print(json.dumps({"int8_gemm": [bench_int8(lib, HIPTensor, memory, n, iters=50) for n in (4096, 11008)]}))
        return

    # ---- inputs, resident in HBM before the timed region ------------------------------------
    t0 = time.time()
    layers = []
    for layer in range(args.layers):
        layers.append([DeviceLinear(lib, HIPTensor, k, n, 1000 * layer + j) for j, (_, k, n) in enumerate(LINEARS)])
    xs, outs = {}, {}
    for _, k, n in LINEARS:
        if k not in xs:
            xs[k] = HIPTensor.allocate((1, k), "float16")
            lib.call("mh_synth_normal", None, xs[k].data_ptr, k, 0.0, 1.0, 0, 0.0, 7 + k, 0)
        outs[n] = HIPTensor.allocate((1, n), "float16")
    ws_bytes = max(lib.call("mh_gptq_workspace_bytes", 1, n, k, GROUP, BITS) for _, k, n in LINEARS)
    ws = memory.workspace(max(ws_bytes, 256))
    memory.synchronize()
    weight_bytes = sum(linear_bytes(0, k, n) for _, k, n in LINEARS)
    log(f"generated {args.layers} layers x {weight_bytes / 1e6:.1f} MB in {time.time() - t0:.1f} s")

    def step(i):
        for lin in layers[i % args.layers]:
            run_gemv(lib, xs[lin.k], lin, outs[lin.n], ws, entry=ENTRY)

    def timed_steps(fn, count):
        e0, e1 = memory.Event(), memory.Event()
        e0.record()                      # null stream: the stream the kernels run on
        for i in range(count):
            fn(i)
        e1.record()
        e1.synchronize()
        return e0.elapsed_ms(e1)

    step_bytes = sum(linear_bytes(1, k, n) for _, k, n in LINEARS)
    # the same K steps right after the warm-up, before the clocks have settled: the figure earlier
    # versions of this benchmark reported as `value`, kept so that results stay comparable
    for i in range(args.warmup):
        step(i)
    memory.synchronize()
    unsettled_ms = timed_steps(step, args.steps)
    gbps_unsettled = step_bytes / (unsettled_ms / args.steps * 1e-3) / 1e9
    if args.settle_ms > 0:
        settled = _settle(memory, step, args.settle_ms)
        log(f"settled the clocks with {settled} untimed steps ({args.settle_ms:.0f} ms)")
    for i in range(args.warmup):
        step(i)
    memory.synchronize()
    wall0 = time.perf_counter()
    dev_ms = timed_steps(step, args.steps)
    memory.synchronize()
    wall = time.perf_counter() - wall0
    ms_per_step = dev_ms / args.steps
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    launches = args.steps * len(LINEARS)
    log(f"{args.steps} steps: {dev_ms:.2f} ms on device ({wall * 1e3:.2f} ms wall), "
        f"{ms_per_step * 1e3:.1f} us/step, {gbps:.0f} GB/s ({gbps_unsettled:.0f} GB/s before the clocks settled)")

    # ---- the dominant kernel (gate|up: 55 % of the step's bytes).  Its average launch duration is measured
    # directly: max(K, 200) launches of it back to back over the cycled weight sets between one pair of HIP
    # events on the stream it runs on (the gaps between the launches, well under a microsecond, are part of
    # the figure, so it reads slightly above the kernel trace of the same command, never below).  Two other
    # readings are reported beside it and are not the roofline figure: what the step loses when that launch
    # is left out (`marginal_us_in_step`: a difference of two passes, which also drops one launch boundary),
    # and the mean of an event pair around every such launch inside the step (two more packets per launch,
    # 2-3 us above the trace).
    dom = max(range(len(LINEARS)), key=lambda j: linear_bytes(1, LINEARS[j][1], LINEARS[j][2]))
    dom_name, dom_k, dom_n = LINEARS[dom]
    dom_count = max(args.steps, 200)

    def dom_only(i):
        lin = layers[i % args.layers][dom]
        run_gemv(lib, xs[lin.k], lin, outs[lin.n], ws, entry=ENTRY)

    def step_without(i):
        for j, lin in enumerate(layers[i % args.layers]):
            if j != dom:
                run_gemv(lib, xs[lin.k], lin, outs[lin.n], ws, entry=ENTRY)

    for i in range(20):
        dom_only(i)
    memory.synchronize()
    dom_us = timed_steps(dom_only, dom_count) * 1e3 / dom_count
    for i in range(20):
        step(i)
    memory.synchronize()
    with_ms = timed_steps(step, dom_count)
    for i in range(20):
        step_without(i)
    memory.synchronize()
    marginal_us = (with_ms - timed_steps(step_without, dom_count)) * 1e3 / dom_count
    pairs = [(memory.Event(), memory.Event()) for _ in range(min(dom_count, 400))]
    for i in range(len(pairs)):
        for j, lin in enumerate(layers[i % args.layers]):
            if j == dom:
                pairs[i][0].record()
            run_gemv(lib, xs[lin.k], lin, outs[lin.n], ws, entry=ENTRY)
            if j == dom:
                pairs[i][1].record()
    memory.synchronize()
    dom_pair_us = float(np.mean([a.elapsed_ms(b) for a, b in pairs])) * 1e3
    dom_bytes = linear_bytes(1, dom_k, dom_n)
    dom_gbps = dom_bytes / dom_us / 1e3
    traffic, traffic_commit = measured_traffic(ENTRY)
    log(f"dominant kernel ({dom_name} {dom_k}x{dom_n}): {dom_us:.2f} us per launch back to back ({dom_count} launches), "
        f"{dom_gbps:.0f} GB/s; marginal in the step {marginal_us:.2f} us, event pair per launch {dom_pair_us:.2f} us")

    result = {
        "metric": "w4a16_gemv_hbm_gbps",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        # the same steps timed before the untimed settle_ms of load (clocks not yet steady)
        "value_unsettled": round(gbps_unsettled, 1),
        "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
        "config": {
            "workload": "llama3-70b-shape GPTQ w4a16 decode GEMVs, M=1, group 128: qkv 8192x10240, "
                        "o 8192x8192, gate_up 8192x57344, down 28672x8192; one step = one layer",
            "layers_cycled": args.layers,
            "bytes_per_step": step_bytes,
            "settle_ms": args.settle_ms,
            "device": info["name"].strip(),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": ("gptq_gemv_kernel<4,1,8>" if ENTRY == "mh_gptq_gemv" else "gptq_gemm_small_kernel<4,1,4,false,true>")
                      + f" ({dom_name} {dom_k}x{dom_n}, M=1)",
            "entry": ENTRY,
            "achieved": round(dom_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dom_gbps / HBM_PEAK_GBPS, 4),
            "avg_launch_us": round(dom_us, 3),
            "launches_timed": dom_count,
            "marginal_us_in_step": round(marginal_us, 3),
            "avg_launch_us_event_pair_per_launch": round(dom_pair_us, 3),
            "bytes_per_launch": dom_bytes,
            "traffic": traffic,
            "traffic_measured_at_commit": traffic_commit,
            # the whole step (four launches, launch gaps included) on the same scale: the headline value
            "step_achieved": round(gbps, 1),
            "step_frac": round(gbps / HBM_PEAK_GBPS, 4),
            "step_avg_launch_us": round(dev_ms * 1e3 / launches, 3),
        },
    }

    # ---- per-shape breakdown and the other metrics named by the baseline --------------------
    if not args.no_extras:
        per_shape = {}
        for j, (name, k, n) in enumerate(LINEARS):
            for i in range(3):
                run_gemv(lib, xs[k], layers[i % args.layers][j], outs[n], ws, entry=ENTRY)
            memory.synchronize()
            a, b = memory.Event(), memory.Event()
            a.record()
            for i in range(50):
                run_gemv(lib, xs[k], layers[i % args.layers][j], outs[n], ws, entry=ENTRY)
            b.record()
            b.synchronize()
            us = a.elapsed_ms(b) * 1e3 / 50
            per_shape[name] = {"us": round(us, 2), "gbps": round(linear_bytes(1, k, n) / us / 1e3, 1)}
        # the same launches on one weight set each: what fits the 256 MB Infinity Cache stays there
        cached = {}
        for j, (name, k, n) in enumerate(LINEARS):
            us = _time_launches(memory, lambda i: run_gemv(lib, xs[k], layers[0][j], outs[n], ws, entry=ENTRY),
                                iters=50, warmup=5)
            cached[name] = {"us": round(us, 2), "gbps": round(linear_bytes(1, k, n) / us / 1e3, 1),
                            "weight_mb": round(linear_bytes(1, k, n) / 1e6, 1)}
        result["extra"] = {"gemv_per_shape": per_shape, "gemv_per_shape_cache_resident": cached}
        # What the launch boundaries cost: the same step with its four launches alternated over two
        # streams (a workspace each).  The four products of the benchmark step do not depend on each
        # other, so the launches overlap freely, which the products of a decode layer cannot: a figure
        # for comparison, not a way the hot path is run.
        two = [memory.create_stream() for _ in range(2)]
        ws2 = [memory.HIPMemory(max(ws_bytes, 256)) for _ in range(2)]
        for mem in ws2:
            mem.reset()
        memory.synchronize()

        def step_two_streams(i):
            for j, lin in enumerate(layers[i % args.layers]):
                t = (i * len(LINEARS) + j) & 1
                lib.call(ENTRY, two[t], xs[lin.k].data_ptr, lin.qweight.data_ptr, lin.qzeros.data_ptr,
                         lin.scales.data_ptr, None, outs[lin.n].data_ptr, 1, lin.n, lin.k, GROUP, BITS,
                         ws2[t]._pointer, ws2[t]._size)
        for i in range(200):
            step_two_streams(i)
        memory.synchronize()
        t0 = time.perf_counter()
        for i in range(1000):
            step_two_streams(i)
        memory.synchronize()
        two_us = (time.perf_counter() - t0) * 1e3
        for st in two:
            lib.call("mh_stream_destroy", st)
        result["extra"]["gemv_step_two_independent_streams"] = {
            "us": round(two_us, 2), "gbps": round(step_bytes / two_us / 1e3, 1),
            "note": "host clock around 1000 steps; launches of a step overlap, which dependent products cannot"}
        if not args.shapes_only:
            # the same four shapes on 8-bit weights (the bit width the reference's own example ships,
            # examples/qwen1_5_int8.py): half the arithmetic per byte
            w8 = {}
            for j, (name, k, n) in enumerate(LINEARS):
                sets = [DeviceLinear(lib, HIPTensor, k, n, 900 + 10 * j + i, bits=8) for i in range(3)]
                ws8 = memory.workspace(max(lib.call("mh_gptq_workspace_bytes", 1, n, k, GROUP, 8), ws._size))
                us = _time_launches(memory, lambda i: run_gemv(lib, xs[k], sets[i % 3], outs[n], ws8), iters=30, warmup=3)
                w8[name] = {"us": round(us, 2), "gbps": round(linear_bytes(1, k, n, bits=8) / us / 1e3, 1)}
                del sets
            result["extra"]["gemv_w8a16_per_shape"] = w8
        try:
            if not args.shapes_only:
                result["extra"]["int8_gemm"] = [bench_int8(lib, HIPTensor, memory, n) for n in (4096, 11008)]
        except Exception as exc:  # report, do not hide
            result["extra"]["int8_gemm_error"] = str(exc)
        try:
            if not args.shapes_only:
                result["extra"]["rowwise_cfg3"] = bench_rowwise(lib, HIPTensor, memory)
                big = lib.call("mh_gptq_workspace_bytes", 128, 2 * 14336, 4096, GROUP, BITS)
                result["extra"].update(bench_small_configs(lib, HIPTensor, memory, memory.workspace(max(big, ws._size))))
        except Exception as exc:
            result["extra"]["small_configs_error"] = str(exc)
        try:
            if args.shapes_only:
                raise RuntimeError("skipped (--shapes-only)")
            from minit_amd import decode
            result["extra"]["decode_70b"] = decode.bench_tokens_per_second(batches=(1, 8, 32), tokens=128, log=log)
            # the same model on 8-bit weights, the bit width of the reference's own example
            result["extra"]["decode_70b_w8a16"] = decode.bench_tokens_per_second(
                batches=(1, 32), tokens=64, log=log, config=dict(decode.LLAMA3_70B, bits=8))
        except Exception as exc:
            result["extra"]["decode_70b_error"] = str(exc)

    # ---- CPU baseline: the C restatement on this host's cores, same layer ---------------------
    if not args.no_cpu_baseline:
        from oracle import cport
        cport.build()
        threads = cport.threads()
        host = []
        for lin in layers[0]:
            host.append((lin.qweight.numpy(), lin.qzeros.numpy(), lin.scales.numpy()))
        hx = {k: t.numpy() for k, t in xs.items()}
        # GPU results for layer 0, to check against what the CPU computes
        gpu_out = []
        for lin in layers[0]:
            run_gemv(lib, xs[lin.k], lin, outs[lin.n], ws, entry=ENTRY)
            gpu_out.append(outs[lin.n].numpy().copy())
        times, worst = [], 0.0
        reps = 5
        for rep in range(reps):
            t = time.perf_counter()
            cpu_out = [cport.matmul(hx[lin.k], *h, None, BITS, GROUP) for lin, h in zip(layers[0], host)]
            times.append(time.perf_counter() - t)
        # one thread: the smallest linear of the layer (o_proj), scaled by its own bytes
        small = min(range(len(LINEARS)), key=lambda j: linear_bytes(1, LINEARS[j][1], LINEARS[j][2]))
        cport.set_threads(1)
        times1 = []
        for rep in range(reps):
            t = time.perf_counter()
            cport.matmul(hx[layers[0][small].k], *host[small], None, BITS, GROUP)
            times1.append(time.perf_counter() - t)
        cport.set_threads(threads)
        small_bytes = linear_bytes(1, LINEARS[small][1], LINEARS[small][2])
        n_out = n_one_step = n_coarse = 0
        for g, c in zip(gpu_out, cpu_out):
            d = np.abs(g.astype(np.float64) - c.astype(np.float64))
            spacing = np.spacing(np.abs(c)).astype(np.float64)
            tol = np.maximum(1e-2, spacing)
            worst = max(worst, float((d / tol).max()))
            n_out += d.size
            n_one_step += int((d > 1e-2).sum())      # outputs that needed the one-fp16-step allowance
            n_coarse += int((spacing > 1e-2).sum())  # outputs large enough (|y| >= 16) to be granted it
        cpu_s = float(np.median(times))
        cpu1_s = float(np.median(times1))
        cpu_model = "unknown"
        try:
            for line in open("/proc/cpuinfo"):
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
        except OSError:
            pass
        result["cpu_baseline"] = {
            "value": round(step_bytes / cpu_s / 1e9, 2),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"one layer (4 GEMVs, {step_bytes / 1e6:.0f} MB), median of {reps} runs, "
                      f"{cpu_s:.2f} s per run, OpenMP over output columns",
            "cpu_model": cpu_model,
            "one_thread": {"value": round(small_bytes / cpu1_s / 1e9, 3), "unit": "GB/s", "cores": 1,
                           "sample": f"{LINEARS[small][0]} alone ({small_bytes / 1e6:.0f} MB), median of {reps} runs, "
                                     f"{cpu1_s:.2f} s per run"},
            "gpu_vs_cpu_worst_err_over_tol": round(worst, 3),
            "gpu_vs_cpu_outputs": n_out,
            "gpu_vs_cpu_outputs_fp16_coarser_than_1e-2": n_coarse,
            "gpu_vs_cpu_outputs_one_fp16_step_off": n_one_step,
        }
        log(f"cpu baseline ({cpu_model}): {cpu_s:.2f} s per layer on {threads} threads, {cpu1_s:.2f} s for "
            f"{LINEARS[small][0]} on one; "
            f"GPU vs CPU worst error / tolerance = {worst:.3f}")

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
