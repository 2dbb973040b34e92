"""GPU parity at the full sizes of the benchmark configurations.

Config 1 (Mistral-7B MLP block, M in {1, 8, 32, 128}) is small enough for the
float64 oracle and is checked stage by stage against it.  The Llama-3-70B
linears of config 4 are too large for that in seconds, so they are checked
through properties that do not depend on size: one-hot activations must return
rows of the dequantized matrix bit for bit (the dequantize kernel itself is
bit-exact against the oracle in test_gptq_gpu.py), the product must be linear in
the activations, and weights equal to their zero point must give exactly zero.
"""
import numpy as np
import pytest

from helpers import assert_fp16_close, fp16_spacing
from oracle import gptq as O

pytestmark = pytest.mark.gpu

GROUP, BITS = 128, 4


def _dev(arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


def _linear(hip, x, qweight, qzeros, scales, m, n, k, entry="mh_gptq_matmul"):
    """x, qweight, qzeros, scales: device tensors."""
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    out = HIPTensor.allocate((m, n), "float16")
    nbytes = hip.call("mh_gptq_workspace_bytes", m, n, k, GROUP, BITS)
    ws = memory.workspace(max(nbytes, 256))
    hip.call(entry, None, x.data_ptr, qweight.data_ptr, qzeros.data_ptr, scales.data_ptr, None,
             out.data_ptr, m, n, k, GROUP, BITS, ws._pointer, ws._size)
    return out


@pytest.fixture(scope="module")
def mistral_weights():
    from minit_amd import synthetic
    hidden, ffn = 4096, 14336
    host = {
        "gate": synthetic.gptq_weights("cfg1", "gate", hidden, ffn, GROUP, BITS),
        "up": synthetic.gptq_weights("cfg1", "up", hidden, ffn, GROUP, BITS),
        "down": synthetic.gptq_weights("cfg1", "down", ffn, hidden, GROUP, BITS),
    }
    dense = {name: O.dequantize_packed(*w, None, BITS, GROUP).astype(np.float64) for name, w in host.items()}
    return host, dense


def test_mistral_prefill_rows(hip, mistral_weights):
    """The same gate and down products over a prefill's worth of rows (2000: blocks of 256 rows, the last
    one ragged; 896 and 256 workgroups), every output against the float64 oracle."""
    from minit_amd import synthetic
    host, dense = mistral_weights
    hidden, ffn, m = 4096, 14336, 2000
    x = synthetic.activations("cfg1", f"x{m}", (m, hidden))
    gate = _linear(hip, _dev(x), *(_dev(t) for t in host["gate"]), m, ffn, hidden).numpy()
    assert_fp16_close(gate, x.astype(np.float64) @ dense["gate"], what=f"gate M={m}")
    h = (gate[:, :ffn] * np.float16(0.125)).astype(np.float16)   # activations of the size the block produces
    y = _linear(hip, _dev(h), *(_dev(t) for t in host["down"]), m, hidden, ffn).numpy()
    assert_fp16_close(y, h.astype(np.float64) @ dense["down"], what=f"down M={m}")


@pytest.mark.parametrize("m", [1, 8, 32, 128])
def test_mistral_mlp_block(hip, mistral_weights, m):
    """h = SiLU(x Wg) * (x Wu), y = h Wd with K = 4096 -> 14336 -> 4096."""
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    host, dense = mistral_weights
    hidden, ffn = 4096, 14336
    x = synthetic.activations("cfg1", f"x{m}", (m, hidden))
    dx = _dev(x)
    dw = {name: tuple(_dev(t) for t in w) for name, w in host.items()}

    gate = _linear(hip, dx, *dw["gate"], m, ffn, hidden)
    up = _linear(hip, dx, *dw["up"], m, ffn, hidden)
    x64 = x.astype(np.float64)
    assert_fp16_close(gate.numpy(), x64 @ dense["gate"], what=f"gate M={m}")
    assert_fp16_close(up.numpy(), x64 @ dense["up"], what=f"up M={m}")

    h = HIPTensor.allocate((m, ffn), "float16")
    hip.call("mh_silu_mul", None, gate.data_ptr, up.data_ptr, h.data_ptr, m * ffn, 1, 0)
    h_host = h.numpy()
    ref_h = O.silu_mul(gate.numpy(), up.numpy())
    mism = (h_host.view(np.uint16) != ref_h.view(np.uint16)).mean()
    assert mism < 1e-3, f"SiLU*up M={m}: {mism:.2%} of elements differ from the three-rounding form"

    # the down projection is checked on the activations the device actually produced
    y = _linear(hip, h, *dw["down"], m, hidden, ffn)
    assert_fp16_close(y.numpy(), h_host.astype(np.float64) @ dense["down"], what=f"down M={m}")


@pytest.mark.parametrize("m", [1, 8, 32, 128])
def test_mistral_mlp_block_fused_entry_points(hip, mistral_weights, m):
    """The same block through the two calls the benchmark times: mh_gptq_matmul_silu_pairs on
    the interleaved gate|up weight (4096 -> 2 x 14336, SiLU*up inside the product: in the
    reduction of the small-M kernel up to 32 rows, in the store of the 128-row blocks above),
    then mh_gptq_matmul 14336 -> 4096, each stage against the float64 oracle."""
    from minit_amd import synthetic
    from minit_amd.decode import interleave_gate_up
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    host, dense = mistral_weights
    hidden, ffn = 4096, 14336
    x = synthetic.activations("cfg1", f"x{m}", (m, hidden))
    fused = interleave_gate_up(*(np.concatenate([g, u], axis=1) for g, u in zip(host["gate"], host["up"])))
    dq, dz, ds = (_dev(t) for t in fused)
    dx = _dev(x)
    h = HIPTensor.allocate((m, ffn), "float16")
    ws = memory.workspace(max(hip.call("mh_gptq_silu_pairs_workspace_bytes", m, 2 * ffn, hidden, GROUP, BITS),
                              hip.call("mh_gptq_workspace_bytes", m, hidden, ffn, GROUP, BITS), 256))
    hip.call("mh_gptq_matmul_silu_pairs", None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, h.data_ptr,
             m, 2 * ffn, hidden, GROUP, BITS, ws._pointer, ws._size)
    h_host = h.numpy()
    assert np.isfinite(h_host.astype(np.float64)).all()
    x64 = x.astype(np.float64)
    gate = (x64 @ dense["gate"]).astype(np.float16)
    up = (x64 @ dense["up"]).astype(np.float16)
    ref = O.silu_mul_f64(gate, up)
    # gate and up are rounded to fp16 before the epilogue; the device's fp32 sums may round to the
    # neighbouring fp16 value, which moves the result by |d silu / d gate| <= 1.1 times a step of
    # gate times |up|, and by |silu(gate)| times a step of up
    g64, u64 = gate.astype(np.float64), up.astype(np.float64)
    step_h = fp16_spacing(ref)
    # (sums that nearly cancel differ between fp32 and float64 accumulation by far more than their own
    # fp16 spacing: an absolute term for that, `hidden` terms of unit size in fp32)
    order = 4.0 * hidden * 2.0 ** -24
    slack = (1.1 * np.abs(u64) * (fp16_spacing(gate) + order)
             + np.abs(g64 / (1.0 + np.exp(-g64))) * (fp16_spacing(up) + order))
    err = np.abs(h_host.astype(np.float64) - ref)
    assert (err <= step_h + slack + 1e-7).all(), f"SiLU*up M={m}: worst {(err - slack).max():.4g}"
    # and that allowance is the exception: nearly all outputs sit within one step of their own
    share = float((err > step_h).mean())
    assert share < 0.02, f"SiLU*up M={m}: {share:.2%} of the outputs needed the operand-step allowance"
    assert np.linalg.norm(h_host.astype(np.float64) - ref) <= 1e-3 * np.linalg.norm(ref)

    y = HIPTensor.allocate((m, hidden), "float16")
    dd = tuple(_dev(t) for t in host["down"])
    hip.call("mh_gptq_matmul", None, h.data_ptr, dd[0].data_ptr, dd[1].data_ptr, dd[2].data_ptr, None, y.data_ptr,
             m, hidden, ffn, GROUP, BITS, ws._pointer, ws._size)
    assert_fp16_close(y.numpy(), h_host.astype(np.float64) @ dense["down"], what=f"down after fused gate|up M={m}")


LLAMA70B_LINEARS = [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 57344), ("down", 28672, 8192)]


class _DeviceLinear:
    """A weight set generated on the device (the host generator would take minutes at these sizes)."""

    def __init__(self, hip, k, n, seed, zeros=(6, 9)):
        from minit_amd.hip.tensor import HIPTensor
        per, groups = 32 // BITS, k // GROUP
        self.k, self.n = k, n
        self.qweight = HIPTensor.allocate((k // per, n), "int32")
        self.qzeros = HIPTensor.allocate((groups, n // per), "int32")
        self.scales = HIPTensor.allocate((groups, n), "float16")
        hip.call("mh_synth_u32", None, self.qweight.data_ptr, (k // per) * n, seed * 3)
        hip.call("mh_synth_subwords", None, self.qzeros.data_ptr, groups * (n // per), BITS, zeros[0], zeros[1],
                 seed * 3 + 1)
        hip.call("mh_synth_normal", None, self.scales.data_ptr, groups * n, 0.0, 0.02, 1, 1e-3, seed * 3 + 2, 0)

    def dense(self, hip):
        from minit_amd.hip.tensor import HIPTensor
        w = HIPTensor.allocate((self.k, self.n), "float16")
        hip.call("mh_gptq_dequant", None, self.qweight.data_ptr, self.qzeros.data_ptr, self.scales.data_ptr, None,
                 w.data_ptr, self.n, self.k, GROUP, BITS)
        return w


@pytest.mark.parametrize("name,k,n", LLAMA70B_LINEARS)
@pytest.mark.parametrize("m", [1, 4, 8, 32])
def test_llama70b_linear_one_hot_rows(hip, name, k, n, m):
    """x = e_k returns row k of the dequantized matrix, bit for bit, at full size."""
    lin = _DeviceLinear(hip, k, n, seed=31)
    rows = np.random.default_rng(k + n + m).choice(k, size=m, replace=False)
    rows[0] = k - 1  # the last row exercises the end of the K walk
    x = np.zeros((m, k), dtype=np.float16)
    x[np.arange(m), rows] = 1.0
    got = _linear(hip, _dev(x), lin.qweight, lin.qzeros, lin.scales, m, n, k).numpy()
    w = lin.dense(hip).numpy()
    np.testing.assert_array_equal(got.view(np.uint16), w[rows].view(np.uint16))


@pytest.mark.parametrize("name,k,n", LLAMA70B_LINEARS)
def test_llama70b_linear_is_linear(hip, name, k, n):
    """f(a + b) = f(a) + f(b) within the product tolerance; a, b carry few
    mantissa bits so that a + b is exact in fp16."""
    lin = _DeviceLinear(hip, k, n, seed=32)
    rng = np.random.default_rng(k * 3 + n)
    a = (rng.integers(-64, 65, size=(1, k)) / 64.0).astype(np.float16)
    b = (rng.integers(-64, 65, size=(1, k)) / 32.0).astype(np.float16)
    s = (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
    assert np.array_equal(s.astype(np.float32), a.astype(np.float32) + b.astype(np.float32))
    ya, yb, ys = (_linear(hip, _dev(v), lin.qweight, lin.qzeros, lin.scales, 1, n, k).numpy() for v in (a, b, s))
    # three fp16 roundings are involved instead of one: allow two fp16 steps
    ref = ya.astype(np.float64) + yb.astype(np.float64)
    err = np.abs(ys.astype(np.float64) - ref)
    tol = np.maximum(2e-2, 2 * fp16_spacing(ref))
    assert (err <= tol).all(), f"{name}: linearity off by {err.max():.4g} at {err.argmax()}"
    assert np.linalg.norm(ys - ref) <= 1e-3 * np.linalg.norm(ref)


@pytest.mark.parametrize("name,k,n", LLAMA70B_LINEARS)
def test_llama70b_linear_zero_point_weights_give_zero(hip, name, k, n):
    """q == z + 1 everywhere dequantizes to 0, so any activation gives exactly 0."""
    from minit_amd.hip.tensor import HIPTensor
    lin = _DeviceLinear(hip, k, n, seed=33, zeros=(6, 6))
    lin.qweight = _dev(np.full((k // 8, n), 0x77777777, dtype=np.uint32).view(np.int32))
    x = HIPTensor.allocate((4, k), "float16")
    hip.call("mh_synth_normal", None, x.data_ptr, 4 * k, 0.0, 1.0, 0, 0.0, 5, 0)
    got = _linear(hip, x, lin.qweight, lin.qzeros, lin.scales, 4, n, k).numpy()
    assert not got.any(), f"{name}: {np.count_nonzero(got)} non-zero outputs"


@pytest.mark.parametrize("m,shares", [(1, None), (5, None), (5, "1")])
def test_eight_bit_gate_up_shape_one_hot_rows(hip, monkeypatch, m, shares):
    """8-bit weights at the gate|up shape, two packed rows per 8 k: one workgroup of eight
    waves per column tile whose two K halves meet in LDS (what 8-bit weights take at any
    row count), and, with that switched off, the balanced plan of the small-M kernel (a
    workgroup finishes one tile and begins the next); one-hot rows return rows of the
    dequantized matrix bit for bit."""
    from minit_amd.hip import memory
    if shares is not None:
        monkeypatch.setenv("MH_GEMM_SMALL_KW", shares)  # read at every call
    from minit_amd.hip.tensor import HIPTensor
    k, n, bits = 8192, 57344, 8
    per, groups = 32 // bits, k // GROUP
    qweight = HIPTensor.allocate((k // per, n), "int32")
    qzeros = HIPTensor.allocate((groups, n // per), "int32")
    scales = HIPTensor.allocate((groups, n), "float16")
    hip.call("mh_synth_u32", None, qweight.data_ptr, (k // per) * n, 97)
    hip.call("mh_synth_subwords", None, qzeros.data_ptr, groups * (n // per), bits, 0, 255, 98)
    hip.call("mh_synth_normal", None, scales.data_ptr, groups * n, 0.0, 0.02, 1, 1e-3, 99, 0)
    rows = np.random.default_rng(m).choice(k, size=m, replace=False)
    rows[0] = k - 1
    x = np.zeros((m, k), dtype=np.float16)
    x[np.arange(m), rows] = 1.0
    dx = _dev(x)
    out = HIPTensor.allocate((m, n), "float16")
    ws = memory.workspace(max(hip.call("mh_gptq_workspace_bytes", m, n, k, GROUP, bits), 256))
    hip.call("mh_gptq_matmul", None, dx.data_ptr, qweight.data_ptr, qzeros.data_ptr, scales.data_ptr, None,
             out.data_ptr, m, n, k, GROUP, bits, ws._pointer, ws._size)
    w = HIPTensor.allocate((k, n), "float16")
    hip.call("mh_gptq_dequant", None, qweight.data_ptr, qzeros.data_ptr, scales.data_ptr, None, w.data_ptr, n, k,
             GROUP, bits)
    np.testing.assert_array_equal(out.numpy().view(np.uint16), w.numpy()[rows].view(np.uint16))


@pytest.mark.parametrize("m", [1, 4, 8, 16, 32, 64])
def test_lm_head_shape_dense_product(hip, m):
    """The unquantized lm_head of the decode loop at its full shape (fp16 [128256, 8192]):
    one-hot activations return columns of the weight bit for bit (every output index of
    the dot-product kernel at 1-8 rows and of the LDS-streaming MFMA kernel above), and a random
    activation agrees with float64 on a sample of the outputs."""
    from minit_amd.hip.tensor import HIPTensor
    vocab, hidden = 128256, 8192
    w = HIPTensor.allocate((vocab, hidden), "float16")
    hip.call("mh_synth_normal", None, w.data_ptr, vocab * hidden, 0.0, 0.05, 0, 0.0, 77, 0)
    wh = w.numpy()
    rng = np.random.default_rng(100 + m)
    ks = rng.choice(hidden, size=m, replace=False)
    ks[0] = hidden - 1
    x = np.zeros((m, hidden), dtype=np.float16)
    x[np.arange(m), ks] = 1.0
    out = HIPTensor.allocate((m, vocab), "float16")
    dx = _dev(x)
    hip.call("mh_f16_matmul_nk", None, dx.data_ptr, w.data_ptr, out.data_ptr, m, vocab, hidden)
    # bit for bit, except that a weight of -0 comes back as the +0 the accumulators start from
    zero = np.float16(0)
    np.testing.assert_array_equal((out.numpy() + zero).view(np.uint16),
                                  (np.ascontiguousarray(wh[:, ks].T) + zero).view(np.uint16))
    x = rng.normal(0, 1, size=(m, hidden)).astype(np.float16)
    dx = _dev(x)
    hip.call("mh_f16_matmul_nk", None, dx.data_ptr, w.data_ptr, out.data_ptr, m, vocab, hidden)
    cols = np.concatenate([rng.choice(vocab, size=509, replace=False), [0, vocab - 1, vocab - 4]])
    ref = x.astype(np.float64) @ wh[cols].astype(np.float64).T
    assert_fp16_close(out.numpy()[:, cols], ref, what="lm_head dense")
