"""Known-answer vectors (tests/golden/kat.json, written by
tests/golden/make_vectors.py with exact integer / rational arithmetic that
shares no code with oracle/ or the kernels): the oracle against them on the CPU,
the HIP path against the same vectors on the GPU."""
import json
import os

import numpy as np
import pytest

from oracle import gptq as OG
from oracle import int8 as OI
from oracle import special as OS

KAT = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat.json")))


def _f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16)


def _gptq_arrays(c):
    return (np.asarray(c["qweight"], dtype=np.int32), np.asarray(c["qzeros"], dtype=np.int32),
            _f16(c["scales_f16_bits"]), _f16(c["x_f16_bits"]))


def _close_to_exact(got, exact, what):
    """fp16 result of an fp32-accumulated sum against the exact sum: within one
    fp16 step of the exact value (the sum's own rounding) plus the fp32 noise."""
    got = got.astype(np.float64)
    tol = np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64) + 1e-4
    assert (np.abs(got - exact) <= tol).all(), f"{what}: worst {np.abs(got - exact).max()}"


def _inf(rows):
    return np.asarray([[-np.inf if v == "-inf" else v for v in r] for r in rows], dtype=np.float16)


# ------------------------------------------------------------------ oracle (CPU)

@pytest.mark.parametrize("idx", range(len(KAT["gptq"])))
def test_oracle_gptq_known_answers(idx):
    c = KAT["gptq"][idx]
    qweight, qzeros, scales, x = _gptq_arrays(c)
    bits, g = c["bits"], c["group_size"]
    np.testing.assert_array_equal(OG.unpack(qweight, 0, bits), np.asarray(c["q"], dtype=np.uint8))
    np.testing.assert_array_equal(OG.unpack(qzeros, 1, bits), np.asarray(c["z"], dtype=np.uint8))
    w = OG.dequantize_packed(qweight, qzeros, scales, None, bits, g)
    np.testing.assert_array_equal(w.view(np.uint16), np.asarray(c["w_f16_bits"], dtype=np.uint16))
    y = OG.matmul(x, qweight, qzeros, scales, None, bits, g)
    _close_to_exact(y, np.asarray(c["y_exact"]), f"oracle matmul {idx}")


@pytest.mark.parametrize("idx", range(len(KAT["int8"])))
def test_oracle_int8_known_answers(idx):
    c = KAT["int8"][idx]
    a, w = np.asarray(c["a"], dtype=np.int8), np.asarray(c["w_nk"], dtype=np.int8)
    acc = OI.gemm_i32(a, w)
    np.testing.assert_array_equal(acc, np.asarray(c["acc"], dtype=np.int32))
    out = OI.dequant_epilogue(acc, np.asarray(c["a_scale"], dtype=np.float32), np.asarray(c["w_scale"], dtype=np.float32))
    np.testing.assert_array_equal(out.view(np.uint16), np.asarray(c["out_f16_bits"], dtype=np.uint16))


def test_oracle_special_known_answers():
    s = KAT["special"]
    c = s["rms_norm_constant_rows"]
    got = OS.rms_norm(np.asarray(c["x"], np.float16), np.asarray(c["weight"], np.float16), 1, c["eps"])
    np.testing.assert_array_equal(got, np.asarray(c["out"], np.float16))
    c = s["rms_norm_eps_rows"]   # eps as large as the mean square: its place in the formula decides the answer
    got = OS.rms_norm(np.asarray(c["x"], np.float16), np.asarray(c["weight"], np.float16), 1, c["eps"])
    np.testing.assert_array_equal(got, np.asarray(c["out"], np.float16))
    c = s["softmax_rows"]
    np.testing.assert_array_equal(OS.softmax(_inf(c["x"]), 1), np.asarray(c["out"], np.float16))
    c = s["softmax_causal"]
    scores = np.full((1, 1, c["rows"], c["t"]), c["score"], np.float16)
    np.testing.assert_array_equal(OS.masked_softmax(scores, c["offset"])[0, 0], np.asarray(c["out"], np.float16))
    c = s["rope_quarter_turns"]
    x = np.asarray(c["x"], np.float16).reshape(1, 1, 1, 6)
    got = OS.rope(x, np.asarray([c["cos"]], np.float32), np.asarray([c["sin"]], np.float32))
    np.testing.assert_array_equal(got.reshape(-1), np.asarray(c["out"], np.float16))
    c = s["reduce_middle_axis"]
    x = np.asarray(c["x"], np.float16)
    np.testing.assert_array_equal(OS.reduce_sum(x, 1), np.asarray(c["sum"], np.float16))
    np.testing.assert_array_equal(OS.reduce_max(x, 1), np.asarray(c["max"], np.float16))
    np.testing.assert_array_equal(OS.reduce_mean(x, 1), np.asarray(c["mean"], np.float16))
    c = s["mean_roundings"]
    assert OS.reduce_mean(np.ones((1, c["ones"]), np.float16), 1)[0, 0] == c["ones_mean"]
    assert OS.reduce_mean(np.full((1, c["halves"]), 0.5, np.float16), 1)[0, 0] == c["halves_mean"]
    c = s["elementwise"]
    np.testing.assert_array_equal(OS.sigmoid(np.asarray(c["sigmoid_in"], np.float16)), np.asarray(c["sigmoid_out"], np.float16))
    got = OS.multiply(np.asarray(c["a"], np.float16), np.asarray(c["b"], np.float16))
    np.testing.assert_array_equal(got.view(np.uint16), np.asarray(c["product"], np.float16).view(np.uint16))
    c = s["silu_mul_zero_gate"]
    got = OG.silu_mul(np.asarray(c["gate"], np.float16), np.asarray(c["up"], np.float16))
    np.testing.assert_array_equal(got.view(np.uint16), np.asarray(c["out"], np.float16).view(np.uint16))


# ------------------------------------------------------------------ HIP path (GPU)

def _t(arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(len(KAT["gptq"])))
def test_hip_gptq_known_answers(hip, idx):
    import minit_amd.functional as F
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import quantized_tensor_from_host
    c = KAT["gptq"][idx]
    qweight, qzeros, scales, x = _gptq_arrays(c)
    bits, k, n = c["bits"], c["k"], c["n"]
    for axis, packed, key in ((0, qweight, "q"), (1, qzeros, "z")):
        out = HIPTensor.allocate(np.asarray(c[key]).shape, "uint8")
        dp = _t(packed)  # held until the result has been read back
        hip.call("mh_gptq_unpack", None, dp.data_ptr, out.data_ptr, packed.shape[0], packed.shape[1], axis, bits)
        np.testing.assert_array_equal(out.numpy(), np.asarray(c[key], dtype=np.uint8))
    w = quantized_tensor_from_host(qweight, qzeros, scales, None)
    np.testing.assert_array_equal(w.dequantize().numpy().view(np.uint16), np.asarray(c["w_f16_bits"], dtype=np.uint16))
    y = F.matrix_multiply(_t(x), w).numpy()
    _close_to_exact(y, np.asarray(c["y_exact"]), f"hip matmul {idx}")


@pytest.mark.gpu
@pytest.mark.parametrize("idx", range(len(KAT["int8"])))
def test_hip_int8_known_answers(hip, idx):
    from minit_amd.hip.tensor import HIPTensor
    c = KAT["int8"][idx]
    a, w = np.asarray(c["a"], dtype=np.int8), np.asarray(c["w_nk"], dtype=np.int8)
    m, n, k = c["m"], c["n"], c["k"]
    out, acc = HIPTensor.allocate((m, n), "float16"), HIPTensor.allocate((m, n), "int32")
    da, dw = _t(a), _t(w)  # device buffers stay referenced until the results have been read back
    dsa, dsw = _t(np.asarray(c["a_scale"], np.float32)), _t(np.asarray(c["w_scale"], np.float32))
    hip.call("mh_i8_gemm", None, da.data_ptr, dw.data_ptr, dsa.data_ptr, dsw.data_ptr, out.data_ptr, acc.data_ptr,
             m, n, k)
    np.testing.assert_array_equal(acc.numpy(), np.asarray(c["acc"], dtype=np.int32))
    np.testing.assert_array_equal(out.numpy().view(np.uint16), np.asarray(c["out_f16_bits"], dtype=np.uint16))


@pytest.mark.gpu
def test_hip_special_known_answers(hip):
    import minit_amd.functional as F
    from minit_amd.hip.tensor import HIPTensor
    s = KAT["special"]
    c = s["rms_norm_constant_rows"]
    got = F.rms_norm(_t(np.asarray(c["x"], np.float16)), _t(np.asarray(c["weight"], np.float16)), 1, c["eps"]).numpy()
    np.testing.assert_array_equal(got, np.asarray(c["out"], np.float16))
    c = s["rms_norm_eps_rows"]
    x, w, ref = (np.asarray(c[key], np.float16) for key in ("x", "weight", "out"))
    step = np.spacing(np.abs(ref)).astype(np.float64)
    got = F.rms_norm(_t(x), _t(w), 1, c["eps"]).numpy()
    assert (np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= step).all(), "mh_rms_norm: eps term"
    # the same rows through the fused residual add + norm, without and with a delta that sums to the row
    for delta in (None, x / 2):
        h = _t(x if delta is None else x / 2)
        d = None if delta is None else _t(np.ascontiguousarray(delta))
        out, dw = HIPTensor.allocate(x.shape, "float16"), _t(w)
        hip.call("mh_add_rms_norm", None, h.data_ptr, d.data_ptr if d else None, dw.data_ptr, out.data_ptr,
                 x.shape[0], x.shape[1], c["eps"])
        assert (np.abs(out.numpy().astype(np.float64) - ref.astype(np.float64)) <= step).all(), "mh_add_rms_norm: eps term"
        np.testing.assert_array_equal(h.numpy(), x)
    c = s["softmax_rows"]
    np.testing.assert_array_equal(F.softmax(_t(_inf(c["x"])), 1).numpy(), np.asarray(c["out"], np.float16))
    c = s["softmax_causal"]
    scores = _t(np.full((1, 1, c["rows"], c["t"]), c["score"], np.float16))
    out = HIPTensor.allocate((1, 1, c["rows"], c["t"]), "float16")
    hip.call("mh_softmax_causal", None, scores.data_ptr, out.data_ptr, 1, c["rows"], c["t"], c["offset"], c["scale"], 0)
    ref = np.asarray(c["out"], np.float64)
    assert (np.abs(out.numpy()[0, 0].astype(np.float64) - ref) <= np.spacing(ref.astype(np.float16))).all()
    assert (out.numpy()[0, 0][ref == 0] == 0).all()
    c = s["rope_quarter_turns"]
    got = F.rope(_t(np.asarray(c["x"], np.float16).reshape(1, 1, 1, 6)), _t(np.asarray([c["cos"]], np.float32)),
                 _t(np.asarray([c["sin"]], np.float32))).numpy()
    np.testing.assert_array_equal(got.reshape(-1), np.asarray(c["out"], np.float16))
    c = s["reduce_middle_axis"]
    x = _t(np.asarray(c["x"], np.float16))
    np.testing.assert_array_equal(F.sum(x, 1).numpy(), np.asarray(c["sum"], np.float16))
    np.testing.assert_array_equal(F.max(x, 1).numpy(), np.asarray(c["max"], np.float16))
    np.testing.assert_array_equal(F.mean(x, 1).numpy(), np.asarray(c["mean"], np.float16))
    c = s["mean_roundings"]
    assert F.mean(_t(np.ones((1, c["ones"]), np.float16)), 1).numpy()[0, 0] == c["ones_mean"]
    assert F.mean(_t(np.full((1, c["halves"]), 0.5, np.float16)), 1).numpy()[0, 0] == c["halves_mean"]
    c = s["elementwise"]
    np.testing.assert_array_equal(F.sigmoid(_t(np.asarray(c["sigmoid_in"], np.float16))).numpy(),
                                  np.asarray(c["sigmoid_out"], np.float16))
    got = F.multiply(_t(np.asarray(c["a"], np.float16)), _t(np.asarray(c["b"], np.float16))).numpy()
    np.testing.assert_array_equal(got.view(np.uint16), np.asarray(c["product"], np.float16).view(np.uint16))
    c = s["silu_mul_zero_gate"]
    g, u = _t(np.asarray(c["gate"], np.float16)), _t(np.asarray(c["up"], np.float16))
    out = HIPTensor.allocate((2,), "float16")
    hip.call("mh_silu_mul", None, g.data_ptr, u.data_ptr, out.data_ptr, 2, 1, 0)
    np.testing.assert_array_equal(out.numpy().view(np.uint16), np.asarray(c["out"], np.float16).view(np.uint16))
