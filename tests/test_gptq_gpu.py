"""GPU parity: GPTQ unpack / dequantize / quantized linear against the oracle.

Integer work (unpack) and the dequantized matrix are bit-exact; products are
within the fp16 tolerance stated in ``helpers.py``.  One-hot activations turn
the product kernels into exact row-pickers of the dequantized matrix, which
pins their k-ordering bit for bit.
"""
import ctypes

import numpy as np
import pytest

from helpers import assert_fp16_close
from oracle import gptq as O

pytestmark = pytest.mark.gpu


def _dev(hip, arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


def _weights(k, n, group_size, bits, seed, zero_range=(6, 9)):
    from minit_amd import synthetic
    return synthetic.gptq_weights(f"test{seed}", "w", k, n, group_size, bits, zero_range)


def _run_linear(hip, entry, x, qweight, qzeros, scales, group_size, bits, g_idx=None):
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    m, k = x.shape
    n = qweight.shape[1]
    dx, dq, dz, ds = _dev(hip, x), _dev(hip, qweight), _dev(hip, qzeros), _dev(hip, scales)
    dg = None if g_idx is None else _dev(hip, g_idx.astype(np.int32))
    out = HIPTensor.allocate((m, n), "float16")
    nbytes = hip.call("mh_gptq_workspace_bytes", m, n, k, group_size, bits)
    ws = memory.workspace(max(nbytes, 256))
    hip.call(entry, None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr,
             None if dg is None else dg.data_ptr, out.data_ptr, m, n, k, group_size, bits,
             ws._pointer, ws._size)
    return out.numpy()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("axis", [0, 1])
def test_unpack_bit_exact(hip, bits, axis):
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(bits * 10 + axis)
    packed = rng.integers(-2**31, 2**31, size=(37, 53), dtype=np.int64).astype(np.int32)
    per_word = 32 // bits
    shape = (37 * per_word, 53) if axis == 0 else (37, 53 * per_word)
    out = HIPTensor.allocate(shape, "uint8")
    dp = _dev(hip, packed)
    hip.call("mh_gptq_unpack", None, dp.data_ptr, out.data_ptr, 37, 53, axis, bits)
    np.testing.assert_array_equal(out.numpy(), O.unpack(packed, axis, bits))


@pytest.mark.parametrize("k,n,group_size,bits", [
    (4096, 4096, 128, 4),     # config 0
    (256, 136, 32, 4),        # N not a multiple of the column tile
    (512, 64, 64, 8),         # the reference's own 8-bit layout
    (384, 72, 128, 4),
])
def test_dequant_bit_exact(hip, k, n, group_size, bits):
    from minit_amd.hip.tensor import HIPTensor
    qweight, qzeros, scales = _weights(k, n, group_size, bits, seed=1, zero_range=(0, (1 << bits) - 1))
    out = HIPTensor.allocate((k, n), "float16")
    dq, dz, ds = _dev(hip, qweight), _dev(hip, qzeros), _dev(hip, scales)
    hip.call("mh_gptq_dequant", None, dq.data_ptr, dz.data_ptr, ds.data_ptr, None, out.data_ptr,
             n, k, group_size, bits)
    ref = O.dequantize_packed(qweight, qzeros, scales, None, bits, group_size)
    np.testing.assert_array_equal(out.numpy().view(np.uint16), ref.view(np.uint16))


def test_dequant_act_order_bit_exact(hip):
    from minit_amd.hip.tensor import HIPTensor
    k, n, g = 512, 128, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=2)
    g_idx = np.random.default_rng(3).permutation(k).astype(np.int32) // g
    out = HIPTensor.allocate((k, n), "float16")
    dq, dz, ds, dg = _dev(hip, qweight), _dev(hip, qzeros), _dev(hip, scales), _dev(hip, g_idx)
    hip.call("mh_gptq_dequant", None, dq.data_ptr, dz.data_ptr, ds.data_ptr, dg.data_ptr, out.data_ptr,
             n, k, g, 4)
    ref = O.dequantize_packed(qweight, qzeros, scales, g_idx, 4)
    np.testing.assert_array_equal(out.numpy().view(np.uint16), ref.view(np.uint16))


LINEAR_SHAPES = [
    # m, k, n, group_size, bits
    (1, 4096, 4096, 128, 4),    # config 0
    (2, 1024, 520, 128, 4),     # ragged N
    (3, 768, 256, 64, 4),
    (4, 512, 1032, 32, 4),
    (1, 1024, 256, 128, 8),
    (4, 512, 264, 64, 8),
]


@pytest.mark.parametrize("m,k,n,group_size,bits", LINEAR_SHAPES)
def test_gemv_matches_oracle(hip, m, k, n, group_size, bits):
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, group_size, bits, seed=4)
    x = synthetic.activations("test4", "x", (m, k))
    got = _run_linear(hip, "mh_gptq_gemv", x, qweight, qzeros, scales, group_size, bits)
    ref = O.matmul_f64(x, qweight, qzeros, scales, None, bits, group_size)
    assert_fp16_close(got, ref, what=f"gemv {m}x{k}x{n}")


@pytest.mark.parametrize("entry,m", [("mh_gptq_gemv", 1), ("mh_gptq_gemv", 4), ("mh_gptq_gemm", 1),
                                     ("mh_gptq_gemm", 16), ("mh_gptq_gemm", 40)])
@pytest.mark.parametrize("bits", [4, 8])
def test_one_hot_rows_are_exact(hip, entry, m, bits):
    """x = e_k picks row k of dequant(W): any wrong k-ordering or zero/scale
    indexing changes bits."""
    k, n, g = 512, 520, 128
    qweight, qzeros, scales = _weights(k, n, g, bits, seed=5, zero_range=(0, (1 << bits) - 1))
    w = O.dequantize_packed(qweight, qzeros, scales, None, bits, g)
    rows = np.random.default_rng(6).choice(k, size=m, replace=False)
    x = np.zeros((m, k), dtype=np.float16)
    x[np.arange(m), rows] = 1.0
    got = _run_linear(hip, entry, x, qweight, qzeros, scales, g, bits)
    np.testing.assert_array_equal(got.view(np.uint16), w[rows].view(np.uint16))


@pytest.mark.parametrize("m,k,n,g,bits", [
    (1, 256, 32, 128, 4), (1, 4096, 4096, 128, 4), (2, 768, 96, 128, 4), (3, 2304, 160, 128, 4),
    (5, 1280, 8192, 128, 4), (8, 8192, 64, 128, 4), (8, 512, 1024, 128, 4),
    # 8-bit words (two packed rows per lane and step) and the other group sizes
    (1, 4096, 4096, 128, 8), (2, 768, 96, 64, 8), (8, 1024, 1024, 256, 8), (4, 512, 2048, 32, 8),
    (1, 2048, 4096, 32, 4), (3, 2304, 160, 64, 4), (5, 1280, 8192, 256, 4), (8, 768, 512, 64, 4),
])
def test_narrow_outputs_match_oracle(hip, m, k, n, g, bits):
    """Shapes served by the kernel whose workgroups own 32 columns over all of K
    (groups of 32 to 256, at most 8 rows, K a multiple of 256, N of 32): K ranges
    that leave waves idle or half used, every zero point, one-hot rows bit for bit."""
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, g, bits, seed=31, zero_range=(0, (1 << bits) - 1))
    x = synthetic.activations("test31", f"x{m}_{k}", (m, k))
    got = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, g, bits)
    assert_fp16_close(got, O.matmul_f64(x, qweight, qzeros, scales, None, bits, g), what=f"narrow {m}x{k}x{n}")
    rows = np.random.default_rng(32).choice(k, size=m, replace=False)
    rows[0] = k - 1
    onehot = np.zeros((m, k), dtype=np.float16)
    onehot[np.arange(m), rows] = 1.0
    got = _run_linear(hip, "mh_gptq_matmul", onehot, qweight, qzeros, scales, g, bits)
    w = O.dequantize_packed(qweight, qzeros, scales, None, bits, g)
    np.testing.assert_array_equal(got.view(np.uint16), w[rows].view(np.uint16))


@pytest.mark.parametrize("m", [1, 5, 8, 16, 17, 32, 64, 128, 200])
def test_gemm_matches_oracle(hip, m):
    from minit_amd import synthetic
    k, n, g = 1024, 776, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=7)
    x = synthetic.activations("test7", f"x{m}", (m, k))
    got = _run_linear(hip, "mh_gptq_gemm", x, qweight, qzeros, scales, g, 4)
    ref = O.matmul_f64(x, qweight, qzeros, scales, None, 4, g)
    assert_fp16_close(got, ref, what=f"gemm M={m}")


@pytest.mark.parametrize("m,k,n,group_size,bits", [
    (8, 1536, 512, 64, 8), (33, 4096, 256, 32, 4),
    # group sizes the small-M kernel does not serve go to the staged MFMA kernel
    (5, 1024, 264, 512, 4), (40, 1536, 256, 96, 4), (130, 1024, 520, 512, 4),
    # five to eight rows, 28 K ranges per tile: their sums are added by the second stage; four rows: in the kernel
    (6, 14336, 512, 128, 4), (7, 14336, 512, 128, 8), (4, 14336, 512, 128, 4)])
def test_gemm_other_layouts(hip, m, k, n, group_size, bits):
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, group_size, bits, seed=8)
    x = synthetic.activations("test8", "x", (m, k))
    got = _run_linear(hip, "mh_gptq_gemm", x, qweight, qzeros, scales, group_size, bits)
    ref = O.matmul_f64(x, qweight, qzeros, scales, None, bits, group_size)
    assert_fp16_close(got, ref, what=f"gemm {m}x{k}x{n} b{bits}")


# More than 64 rows.  K a multiple of 128: blocks of 128 rows with the weights dequantised in registers
# (K walked in rounds of 128, a quarter per wave, the four shares added through LDS), blocks of 256 rows
# (rounds of 64, a half per wave) where they fill the CUs without padding or a split of K.  Other K that are
# multiples of 64, from 192 rows and 192 tiles of 128 x 128: dequantised tiles staged in LDS.
@pytest.mark.parametrize("m,k,n,group_size", [
    (65, 512, 264, 128),       # one ragged row block, ragged last column tile, four rounds
    (128, 4096, 1024, 128),    # 8 tiles: K split over workgroups (partial sums + second stage)
    (200, 1024, 776, 64),      # two row blocks, two groups per round
    (384, 2048, 520, 256),     # groups longer than a round
    (130, 1536, 128, 32),      # four groups per round, one column tile
    (1000, 640, 1032, 128),    # five rounds: the ring of four wraps once
    (384, 320, 8200, 64),      # K % 128 == 64 -- 3 x 65 tiles, ragged last column tile, unsplit, four waves per workgroup
    (500, 576, 6144, 64),      # K % 128 == 64 -- 4 x 48 tiles, ragged last row tile
    (192, 6208, 12288, 64),    # K % 128 == 64 -- 2 x 96 tiles, eight waves per workgroup, K split in two
    (1000, 576, 3080, 192),    # K % 128 == 64 -- 8 x 25 tiles, groups longer than a stage
    (512, 8256, 128, 64),      # K % 128 == 64, too few tiles: the 64-row blocks of the small-M kernel
    (256, 512, 28672, 128),    # blocks of 256 rows (224 tiles, no padding beyond blocks of 128): eight rounds of 64 k
    (500, 384, 14400, 64),     # ... two row blocks, the second ragged, ragged last column tile, two groups per 128 k
    (512, 1024, 14336, 256),   # ... groups longer than a round
    (256, 640, 28800, 32),     # ... two groups per round of 64 k, ten rounds (the ring of four wraps twice), ragged last column tile
    (24, 2048, 5120, 128),     # 17 to 32 rows where the workgroups are many and their walks short: two row tiles, 40 tiles x 4 K ranges
    (31, 2560, 5000, 64),      # ... five K ranges of four rounds, ragged last column tile
    (17, 512, 20488, 32),      # ... 161 tiles, K unsplit, four groups per round
])
def test_gemm_many_rows(hip, m, k, n, group_size):
    """Rows beyond one block of 64: both kernels that dequantise a packed word once for 128 rows."""
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, group_size, 4, seed=9)
    x = synthetic.activations("test9", f"x{m}", (m, k))
    got = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, group_size, 4)
    ref = O.matmul_f64(x, qweight, qzeros, scales, None, 4, group_size)
    assert_fp16_close(got, ref, what=f"many rows {m}x{k}x{n} g{group_size}")
    # one-hot rows pick rows of the dequantized matrix bit for bit (k order inside the LDS tiles)
    rows = np.random.default_rng(m).integers(0, k, m)
    rows[:4] = [0, 63, 64, k - 1]
    onehot = np.zeros((m, k), dtype=np.float16)
    onehot[np.arange(m), rows] = 1.0
    got = _run_linear(hip, "mh_gptq_matmul", onehot, qweight, qzeros, scales, group_size, 4)
    w = O.dequantize_packed(qweight, qzeros, scales, None, 4, group_size)
    np.testing.assert_array_equal(got.view(np.uint16), w[rows].view(np.uint16))


def test_repeated_calls_are_deterministic(hip):
    """Split-K partials are summed in a fixed order: bitwise repeatable, and the
    arrival counters are left zeroed for the next call."""
    from minit_amd import synthetic
    k, n, g = 4096, 1024, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=9)
    for entry, m in (("mh_gptq_gemv", 2), ("mh_gptq_gemm", 24)):
        x = synthetic.activations("test9", f"x{m}", (m, k))
        first = _run_linear(hip, entry, x, qweight, qzeros, scales, g, 4)
        for _ in range(3):
            again = _run_linear(hip, entry, x, qweight, qzeros, scales, g, 4)
            np.testing.assert_array_equal(first.view(np.uint16), again.view(np.uint16))


def test_shared_workspace_across_shapes(hip):
    """One workspace serves calls of different shapes: the partial sums of a call
    with few column tiles must not disturb the arrival counters of a later call
    with many (counters live in a fixed region of the workspace)."""
    from minit_amd import synthetic
    shapes = [(1, 2048, 256), (16, 2048, 512), (1, 1024, 57344), (2, 4096, 1024), (24, 1024, 20480)]
    for m, k, n in shapes:
        qweight, qzeros, scales = _weights(k, n, 128, 4, seed=13)
        x = synthetic.activations("test13", f"x{m}-{k}", (m, k))
        entry = "mh_gptq_gemv" if m <= 4 else "mh_gptq_gemm"
        got = _run_linear(hip, entry, x, qweight, qzeros, scales, 128, 4)
        ref = O.matmul_f64(x, qweight, qzeros, scales, None, 4, 128)
        assert_fp16_close(got, ref, what=f"shared workspace {m}x{k}x{n}")


def test_act_order_through_matmul(hip):
    from minit_amd import synthetic
    m, k, n, g = 3, 512, 128, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=10)
    g_idx = np.random.default_rng(11).permutation(k).astype(np.int32) // g
    x = synthetic.activations("test10", "x", (m, k))
    got = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, g, 4, g_idx=g_idx)
    ref = O.matmul_f64(x, qweight, qzeros, scales, g_idx, 4)
    assert_fp16_close(got, ref, what="act-order")


def _run_with_bias(hip, x, qweight, qzeros, scales, bias, group_size, bits, g_idx=None):
    """(mh_gptq_linear's output, mh_gptq_matmul's, the latter after mh_add_bias)."""
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.lib import DTYPE_CODES
    m, k = x.shape
    n = qweight.shape[1]
    dx, dq, dz, ds, db = (_dev(hip, a) for a in (x, qweight, qzeros, scales, bias))
    dg = None if g_idx is None else _dev(hip, g_idx.astype(np.int32))
    ws = memory.workspace(max(hip.call("mh_gptq_workspace_bytes", m, n, k, group_size, bits), 256))
    outs = []
    for entry in ("mh_gptq_linear", "mh_gptq_matmul"):
        out = HIPTensor.from_numpy(np.full((m, n), np.nan, np.float16))
        args = [None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, None if dg is None else dg.data_ptr]
        if entry == "mh_gptq_linear":
            args.append(db.data_ptr)
        hip.call(entry, *args, out.data_ptr, m, n, k, group_size, bits, ws._pointer, ws._size)
        outs.append(out.numpy())
        if entry == "mh_gptq_matmul":
            hip.call("mh_add_bias", None, out.data_ptr, db.data_ptr, m, n, DTYPE_CODES["float16"])
            outs.append(out.numpy())
    return outs


# one case per place where a product kernel stores results: the column-owner kernel, the small-M
# kernel's direct store, its in-kernel split-K reduction, the split-K second stage, row-blocked
# launches, the LDS-staged kernel with four and with eight waves (direct and split), the 128-row blocks
# (split and direct), the 8-bit kernels;
# then the launches that add the bias in a pass of their own (odd group size, act-order, VALU rows)
@pytest.mark.parametrize("m,k,n,g,bits,act_order", [
    (1, 1024, 256, 128, 4, False), (1, 4096, 8192, 128, 4, False), (1, 8192, 1024, 128, 4, False),
    (4, 512, 28672, 128, 4, False), (8, 4096, 4096, 128, 4, False), (16, 4096, 1024, 128, 4, False),
    (32, 2048, 2048, 64, 4, False), (100, 1088, 1536, 64, 4, False), (130, 4160, 512, 64, 4, False),
    (200, 576, 12288, 64, 4, False), (400, 320, 6144, 64, 4, False), (192, 6208, 12288, 64, 4, False),
    (128, 4096, 1024, 128, 4, False), (300, 1024, 1032, 128, 4, False), (256, 512, 28672, 128, 4, False),
    (1, 2048, 2048, 128, 8, False), (24, 1024, 768, 64, 8, False), (300, 512, 512, 128, 8, False),
    (3, 768, 264, 96, 4, False), (5, 1024, 512, 512, 4, False), (6, 1024, 256, 128, 4, True),
])
def test_linear_with_bias_is_the_product_then_one_fp16_add(hip, m, k, n, g, bits, act_order):
    """mh_gptq_linear == mh_gptq_matmul followed by mh_add_bias == fp16(product + bias) computed
    on the host from the device's fp16 product, all bit for bit (the bias is added to the
    fp16-rounded product in fp16 wherever the kernels store it); the product itself against the
    oracle."""
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, g, bits, seed=60 + m)
    rng = np.random.default_rng(m * 7 + k)
    bias = rng.normal(0, 0.5, size=(n,)).astype(np.float16)
    g_idx = rng.permutation(k).astype(np.int32) // g if act_order else None
    x = synthetic.activations("test60", f"x{m}x{k}", (m, k))
    fused, product, two_pass = _run_with_bias(hip, x, qweight, qzeros, scales, bias, g, bits, g_idx)
    np.testing.assert_array_equal(fused.view(np.uint16), two_pass.view(np.uint16))
    np.testing.assert_array_equal(fused.view(np.uint16), (product + bias[None, :]).astype(np.float16).view(np.uint16))
    assert_fp16_close(product, O.matmul_f64(x, qweight, qzeros, scales, g_idx, bits, g),
                      what=f"product of linear {m}x{k}x{n}")


def test_linear_without_bias_is_the_product(hip):
    from minit_amd import synthetic
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    m, k, n, g = 7, 1024, 512, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=77)
    x = synthetic.activations("test77", "x", (m, k))
    want = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, g, 4)
    dx, dq, dz, ds = (_dev(hip, a) for a in (x, qweight, qzeros, scales))
    out = HIPTensor.allocate((m, n), "float16")
    ws = memory.workspace(max(hip.call("mh_gptq_workspace_bytes", m, n, k, g, 4), 256))
    hip.call("mh_gptq_linear", None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, None, None,
             out.data_ptr, m, n, k, g, 4, ws._pointer, ws._size)
    np.testing.assert_array_equal(out.numpy().view(np.uint16), want.view(np.uint16))


def test_bad_arguments_are_reported(hip):
    from minit_amd.lib import HipError
    with pytest.raises(HipError, match="bits"):
        hip.call("mh_gptq_gemv", None, 256, 256, 256, 256, None, 256, 1, 64, 64, 32, 3, None, 0)
    with pytest.raises(HipError, match="group_size"):
        hip.call("mh_gptq_gemv", None, 256, 256, 256, 256, None, 256, 1, 64, 96, 64, 4, None, 0)
    with pytest.raises(HipError, match="M <="):
        hip.call("mh_gptq_gemv", None, 256, 256, 256, 256, None, 256, 9, 64, 128, 128, 4, None, 0)


def test_operator_api_drop_in(hip):
    """F.matrix_multiply(x, QuantizedTensor) with leading dims folded, and
    QuantizedTensor.dequantize(), as the reference's callers use them."""
    import minit_amd.functional as F
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import quantized_tensor_from_host
    k, n, g = 1024, 512, 128
    qweight, qzeros, scales = _weights(k, n, g, 4, seed=12)
    g_idx = (np.arange(k) // g).astype(np.int32)
    w = quantized_tensor_from_host(qweight, qzeros, scales, g_idx)
    assert w._group is None and w.dtype == "quint4" and tuple(d.item() for d in w.shape) == (k, n)
    x = synthetic.activations("test12", "x", (2, 3, k))
    y = F.matrix_multiply(HIPTensor.from_numpy(x), w)
    assert tuple(d.item() for d in y.shape) == (2, 3, n)
    ref = O.matmul_f64(x.reshape(6, k), qweight, qzeros, scales, None, 4, g).reshape(2, 3, n)
    assert_fp16_close(y.numpy(), ref, what="F.matrix_multiply")
    wd = w.dequantize().numpy()
    np.testing.assert_array_equal(wd.view(np.uint16),
                                  O.dequantize_packed(qweight, qzeros, scales, None, 4, g).view(np.uint16))


@pytest.mark.parametrize("m,k,ffn", [(1, 512, 256), (3, 1024, 384), (8, 256, 128), (16, 512, 256), (32, 768, 512),
                                     (40, 512, 256),     # 33 to 64 rows, K >= 512: one block of 64 rows, SiLU*up in its store
                                     (40, 384, 256), (64, 256, 128),      # ... K < 512: product, then one pass
                                     (130, 1024, 384), (200, 512, 640),   # 128-row blocks, SiLU*up in their store
                                     (128, 4096, 512),   # ... K split over workgroups: product, then one pass
                                     (256, 512, 14336),  # 256-row blocks (224 tiles), SiLU*up in their store
                                     (24, 512, 14336), (32, 1024, 10240)])  # 17 to 32 rows on many short tiles: two row tiles of the 128-row-block kernel
def test_silu_pairs_epilogue(hip, m, k, ffn):
    """gate|up product with SiLU*up applied in the reduction: equals the plain
    product followed by silu(gate) * up on the interleaved column blocks."""
    from minit_amd import synthetic
    from minit_amd.decode import interleave_gate_up
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    g = 128
    qweight, qzeros, scales = interleave_gate_up(*_weights(k, 2 * ffn, g, 4, seed=21))
    x = synthetic.activations("test21", f"x{m}", (m, k))
    dx, dq, dz, ds = _dev(hip, x), _dev(hip, qweight), _dev(hip, qzeros), _dev(hip, scales)
    out = HIPTensor.allocate((m, ffn), "float16")
    ws = memory.workspace(max(hip.call("mh_gptq_silu_pairs_workspace_bytes", m, 2 * ffn, k, g, 4), 256))
    hip.call("mh_gptq_matmul_silu_pairs", None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, out.data_ptr,
             m, 2 * ffn, k, g, 4, ws._pointer, ws._size)
    y = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, g, 4)      # the same device product
    y = y.reshape(m, ffn // 128, 2, 128)
    ref = O.silu_mul_f64(y[:, :, 0], y[:, :, 1]).reshape(m, ffn)
    got = out.numpy()
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    # the plain product may come from another kernel (another summation order): its
    # fp16 values can sit one step away from the ones the epilogue saw
    gate, up = y[:, :, 0].astype(np.float64).reshape(m, ffn), y[:, :, 1].astype(np.float64).reshape(m, ffn)
    dg = np.spacing(np.abs(y[:, :, 0])).astype(np.float64).reshape(m, ffn)
    du = np.spacing(np.abs(y[:, :, 1])).astype(np.float64).reshape(m, ffn)
    silu = gate / (1.0 + np.exp(-gate))
    # sums that nearly cancel differ between two fp32 summation orders by far more than their
    # own fp16 spacing: an absolute term for that (k terms of unit size, fp32 accumulation)
    order = 4.0 * k * 2.0 ** -24
    slack = 1.1 * np.abs(up) * (dg + order) + np.abs(silu) * (du + order)  # |d silu / d gate| <= 1.1
    assert (np.abs(got.astype(np.float64) - ref) <= 1.0 * ulp + slack + 1e-7).all()
    # and the product itself is the oracle's
    assert_fp16_close(y.reshape(m, 2 * ffn), O.matmul_f64(x, qweight, qzeros, scales, None, 4, g), what="gate|up")
    # one-hot activations: the sums are rows of the dequantised matrix whatever the summation order, so the
    # epilogue must return silu(W[k, gate(j)]) * W[k, up(j)] to one fp16 step -- no slack for a wrong pairing
    rows = np.random.default_rng(m).integers(0, k, m)
    onehot = np.zeros((m, k), dtype=np.float16)
    onehot[np.arange(m), rows] = 1.0
    dh = _dev(hip, onehot)
    hip.call("mh_gptq_matmul_silu_pairs", None, dh.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, out.data_ptr,
             m, 2 * ffn, k, g, 4, ws._pointer, ws._size)
    w = O.dequantize_packed(qweight, qzeros, scales, None, 4, g)[rows].reshape(m, ffn // 128, 2, 128)
    ref = O.silu_mul_f64(w[:, :, 0], w[:, :, 1]).reshape(m, ffn)
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    assert (np.abs(out.numpy().astype(np.float64) - ref) <= ulp + 1e-9).all()


def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        bits = int(rng.choice([4, 4, 4, 8]))
        g = int(rng.choice([32, 64, 128, 128, 256]))
        k = g * int(rng.integers(1, 9)) * int(rng.choice([1, 2, 4]))
        n = 8 * int(rng.integers(1, 160))
        m = int(rng.choice([1, 2, 3, 5, 8, 9, 16, 17, 31, 32, 33, 48, 64, 65, 100, 130]))
        cases.append((m, k, n, g, bits))
    return cases


@pytest.mark.parametrize("m,k,n,group_size,bits", _random_cases(28, seed=2024))
def test_random_shapes_match_oracle(hip, m, k, n, group_size, bits):
    """Seeded sweep over row counts, ragged widths, depths, group sizes and bit
    widths: whichever kernel the dispatcher picks must agree with the oracle, and
    one-hot rows must come back as rows of the dequantized matrix bit for bit."""
    from minit_amd import synthetic
    qweight, qzeros, scales = _weights(k, n, group_size, bits, seed=1000 + m + k + n,
                                       zero_range=(0, (1 << bits) - 1))
    x = synthetic.activations("sweep", f"x{m}_{k}_{n}", (m, k))
    got = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, group_size, bits)
    assert_fp16_close(got, O.matmul_f64(x, qweight, qzeros, scales, None, bits, group_size),
                      what=f"sweep {m}x{k}x{n} g{group_size} b{bits}")
    rows = np.random.default_rng(m * k + n).integers(0, k, size=m)
    rows[0] = k - 1
    onehot = np.zeros((m, k), dtype=np.float16)
    onehot[np.arange(m), rows] = 1.0
    got = _run_linear(hip, "mh_gptq_matmul", onehot, qweight, qzeros, scales, group_size, bits)
    w = O.dequantize_packed(qweight, qzeros, scales, None, bits, group_size)
    np.testing.assert_array_equal(got.view(np.uint16), w[rows].view(np.uint16))


def test_two_streams_with_their_own_workspaces(hip):
    """Launchers keep no mutable state of their own: products enqueued on two
    created streams, each with its own workspace, interleaved from one host
    thread, give the bits of the same calls made one after the other on the null
    stream (split-K shapes, so the workspaces are in use)."""
    from minit_amd import synthetic
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    shapes = [(1, 2048, 768, 128, 4), (8, 1024, 1536, 128, 4)]
    jobs = []
    for i, (m, k, n, g, bits) in enumerate(shapes):
        qweight, qzeros, scales = _weights(k, n, g, bits, seed=90 + i)
        x = synthetic.activations("streams", f"x{i}", (m, k))
        dev = [_dev(hip, t) for t in (x, qweight, qzeros, scales)]
        nbytes = max(hip.call("mh_gptq_workspace_bytes", m, n, k, g, bits), 256)
        ws = HIPTensor.allocate((nbytes,), "int8")
        ws._memory.reset()
        jobs.append(dict(m=m, k=k, n=n, g=g, bits=bits, dev=dev, ws=ws, nbytes=nbytes,
                         out=HIPTensor.allocate((m, n), "float16"), stream=memory.create_stream()))
    memory.synchronize()

    def launch(job, stream):
        x, qw, qz, sc = job["dev"]
        hip.call("mh_gptq_matmul", stream, x.data_ptr, qw.data_ptr, qz.data_ptr, sc.data_ptr, None,
                 job["out"].data_ptr, job["m"], job["n"], job["k"], job["g"], job["bits"],
                 job["ws"].data_ptr, job["nbytes"])

    want = []
    for job in jobs:
        launch(job, None)
        memory.synchronize()
        want.append(job["out"].numpy().copy())
        job["out"]._memory.reset()
    memory.synchronize()
    for _ in range(10):
        for job in jobs:
            launch(job, job["stream"])
    for job in jobs:
        memory.synchronize(job["stream"])
    for job, ref in zip(jobs, want):
        np.testing.assert_array_equal(job["out"].numpy().view(np.uint16), ref.view(np.uint16))
        hip.call("mh_stream_destroy", job["stream"])


@pytest.mark.parametrize("bits", [8, 4])
def test_quantized_tensor_from_the_reference_s_unpacked_form(hip, bits):
    """A weight held the way the reference's QuantizedTensor holds it (one uint8
    per sub-word) is packed once and then behaves like the checkpoint tensors:
    same product, same dequantized matrix, bit for bit."""
    import minit_amd.functional as F
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import quantized_tensor_from_host, quantized_tensor_from_unpacked
    k, n, g = 512, 264, 128
    qweight, qzeros, scales = _weights(k, n, g, bits, seed=70 + bits, zero_range=(0, (1 << bits) - 1))
    data, zero = O.unpack(qweight, 0, bits), O.unpack(qzeros, 1, bits)          # uint8 [K, N], [G, N]
    a = quantized_tensor_from_unpacked(HIPTensor.from_numpy(data), HIPTensor.from_numpy(zero), scales, bits=bits)
    b = quantized_tensor_from_host(qweight, qzeros, scales)
    assert (a.bits, a.group_size, a.in_features, a.out_features) == (bits, g, k, n)
    np.testing.assert_array_equal(a._data.numpy(), qweight)
    np.testing.assert_array_equal(a._zero.numpy(), qzeros)
    x = HIPTensor.from_numpy(synthetic.activations("unpacked", "x", (3, k)))
    np.testing.assert_array_equal(F.matrix_multiply(x, a).numpy().view(np.uint16),
                                  F.matrix_multiply(x, b).numpy().view(np.uint16))
    np.testing.assert_array_equal(a.dequantize().numpy().view(np.uint16),
                                  O.dequantize_packed(qweight, qzeros, scales, None, bits, g).view(np.uint16))


@pytest.mark.parametrize("m,k,bits,forced", [(9, 512, 4, False), (17, 768, 4, False), (32, 1024, 4, False), (20, 512, 8, False),
                                             (1, 1024, 4, True), (8, 768, 4, True)])
def test_two_k_shares_inside_a_workgroup(hip, m, k, bits, forced):
    """A wide output (224 column tiles, as many as the 70B gate|up projection has) above 8 rows: workgroups of
    eight waves whose two K shares meet in LDS (K of three stages leaves the second share a dead stage), the
    plain product against the oracle and the SiLU*up epilogue, which then runs inside the launch, against the
    plain product; with MH_GEMM_SMALL_KW=2 also at 1 and 8 rows, where the balanced plan is the default."""
    import os
    from minit_amd import synthetic
    from minit_amd.decode import interleave_gate_up
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    n, g = 57344, 128
    prev = os.environ.get("MH_GEMM_SMALL_KW")
    if forced:
        os.environ["MH_GEMM_SMALL_KW"] = "2"
    try:
        if bits == 8:  # zero points in the middle of the range and finer steps: the same spread as 4 bit
            qweight, qzeros, scales = _weights(k, n, g, bits, seed=61, zero_range=(120, 135))
            scales = (scales.astype(np.float32) / 16).astype(np.float16)
        else:
            qweight, qzeros, scales = _weights(k, n, g, bits, seed=61)
        qweight, qzeros, scales = interleave_gate_up(qweight, qzeros, scales, bits=bits)
        x = synthetic.activations("test61", f"x{m}", (m, k))
        y = _run_linear(hip, "mh_gptq_matmul", x, qweight, qzeros, scales, g, bits)
        assert_fp16_close(y, O.matmul_f64(x, qweight, qzeros, scales, None, bits, g), what=f"two shares M={m} K={k}")
        dx, dq, dz, ds = _dev(hip, x), _dev(hip, qweight), _dev(hip, qzeros), _dev(hip, scales)
        out = HIPTensor.allocate((m, n // 2), "float16")
        ws = memory.workspace(max(hip.call("mh_gptq_silu_pairs_workspace_bytes", m, n, k, g, bits), 256))
        hip.call("mh_gptq_matmul_silu_pairs", None, dx.data_ptr, dq.data_ptr, dz.data_ptr, ds.data_ptr, out.data_ptr,
                 m, n, k, g, bits, ws._pointer, ws._size)
        pairs = y.reshape(m, n // 256, 2, 128)
        ref = O.silu_mul_f64(pairs[:, :, 0], pairs[:, :, 1]).reshape(m, n // 2)
        got = out.numpy().astype(np.float64)
        # same kernel, same sums: the epilogue sees exactly the fp16 values of the plain product
        assert (np.abs(got - ref) <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) + 1e-7).all()
    finally:
        if prev is None:
            os.environ.pop("MH_GEMM_SMALL_KW", None)
        else:
            os.environ["MH_GEMM_SMALL_KW"] = prev
