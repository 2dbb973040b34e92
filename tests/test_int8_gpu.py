"""GPU parity: W8A8 int8 GEMM.  int32 accumulators are bit-exact; the fp16
output of the scale epilogue is bit-exact too, because every step of it
(int32 -> fp32, fp32 product of the scales, fp32 multiply, fp32 -> fp16) is a
single correctly rounded operation in both implementations."""
import numpy as np
import pytest

from oracle import int8 as O

pytestmark = pytest.mark.gpu


def _run(hip, a, w, a_scale, w_scale, want_acc=True, want_out=True):
    from minit_amd.hip.tensor import HIPTensor
    m, k = a.shape
    n = w.shape[0]
    da, dw = HIPTensor.from_numpy(a), HIPTensor.from_numpy(w)
    dsa, dsw = HIPTensor.from_numpy(a_scale), HIPTensor.from_numpy(w_scale)
    out = HIPTensor.allocate((m, n), "float16") if want_out else None
    acc = HIPTensor.allocate((m, n), "int32") if want_acc else None
    hip.call("mh_i8_gemm", None, da.data_ptr, dw.data_ptr, dsa.data_ptr, dsw.data_ptr,
             out.data_ptr if out else None, acc.data_ptr if acc else None, m, n, k)
    return (out.numpy() if out else None), (acc.numpy() if acc else None)


@pytest.mark.parametrize("m,n,k", [
    (128, 256, 64),       # exactly one tile, one k-step
    (1, 8, 64),           # far smaller than a tile
    (130, 260, 192),      # ragged M and N
    (257, 1000, 512),     # 128-k stages, ring of four
    (100, 300, 768),      # 128-k stages, ring of two
    (64, 136, 384),       # 128-k stages, ring of one
    (130, 260, 128),      # a single 128-k stage
    (2048, 4096, 4096),   # config 2
])
def test_i8_gemm_bit_exact(hip, m, n, k):
    from minit_amd import synthetic
    a, w, a_scale, w_scale = synthetic.int8_operands(f"i8-{m}-{n}-{k}", m, n, k)
    out, acc = _run(hip, a, w, a_scale, w_scale)
    ref_out, ref_acc = O.gemm(a, w, a_scale, w_scale)
    np.testing.assert_array_equal(acc, ref_acc)
    np.testing.assert_array_equal(out.view(np.uint16), ref_out.view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(2048, 4096, 4096), (130, 260, 192)])
def test_i8_gemm_fp16_output_only(hip, m, n, k):
    """acc_i32 == NULL, the call the benchmark times: the fp16 output alone, bit for bit."""
    from minit_amd import synthetic
    a, w, a_scale, w_scale = synthetic.int8_operands(f"i8-{m}-{n}-{k}", m, n, k)
    out, acc = _run(hip, a, w, a_scale, w_scale, want_acc=False)
    assert acc is None
    ref_out, _ = O.gemm(a, w, a_scale, w_scale)
    np.testing.assert_array_equal(out.view(np.uint16), ref_out.view(np.uint16))


def _sweep(count, seed):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, 400)), int(rng.integers(1, 700)), 64 * int(rng.integers(1, 13)))
            for _ in range(count)]


@pytest.mark.parametrize("m,n,k", _sweep(16, seed=77))
def test_i8_gemm_random_shapes(hip, m, n, k):
    """Seeded sweep over ragged M and N (any value, not only multiples of the
    tile) and over K in both kernels' ranges (64-k and 128-k stages): int32
    accumulators and the scaled fp16 output bit for bit."""
    from minit_amd import synthetic
    a, w, a_scale, w_scale = synthetic.int8_operands(f"i8-sweep-{m}-{n}-{k}", m, n, k)
    out, acc = _run(hip, a, w, a_scale, w_scale)
    ref_out, ref_acc = O.gemm(a, w, a_scale, w_scale)
    np.testing.assert_array_equal(acc, ref_acc)
    np.testing.assert_array_equal(out.view(np.uint16), ref_out.view(np.uint16))


def test_i8_gemm_extreme_values(hip):
    """All operands at +-127 / -128: the largest accumulators the type allows."""
    m, n, k = 64, 64, 4096
    a = np.full((m, k), -128, dtype=np.int8)
    w = np.full((n, k), -128, dtype=np.int8)
    w[::2] = 127
    ones_m, ones_n = np.ones(m, np.float32), np.ones(n, np.float32)
    _, acc = _run(hip, a, w, ones_m, ones_n, want_out=False)
    np.testing.assert_array_equal(acc, O.gemm_i32(a, w))


def test_i8_gemm_n11008_sample(hip):
    """Config 2's second shape, checked on rows and columns sampled across tiles."""
    from minit_amd import synthetic
    m, n, k = 2048, 11008, 4096
    a, w, a_scale, w_scale = synthetic.int8_operands("i8-cfg2b", m, n, k)
    out, acc = _run(hip, a, w, a_scale, w_scale)
    rows = np.r_[0:3, 127:130, 1000:1003, 2045:2048]
    cols = np.r_[0:5, 255:258, 5000:5005, 10999:11008]
    ref_acc = O.gemm_i32(a[rows], w[cols])
    np.testing.assert_array_equal(acc[np.ix_(rows, cols)], ref_acc)
    ref_out = O.dequant_epilogue(ref_acc, a_scale[rows], w_scale[cols])
    np.testing.assert_array_equal(out[np.ix_(rows, cols)].view(np.uint16), ref_out.view(np.uint16))
    # checksum of checksums over the whole output: sum_n acc[m, n] == a[m] . sum_n w[n]
    colsum = w.astype(np.int64).sum(axis=0)
    np.testing.assert_array_equal(acc.astype(np.int64).sum(axis=1), a.astype(np.int64) @ colsum)


def test_i8_transpose(hip):
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(0)
    w_kn = rng.integers(-128, 128, size=(200, 331), dtype=np.int8)
    out = HIPTensor.allocate((331, 200), "int8")
    src = HIPTensor.from_numpy(w_kn)
    hip.call("mh_i8_transpose", None, src.data_ptr, out.data_ptr, 200, 331)
    np.testing.assert_array_equal(out.numpy(), w_kn.T)


def test_i8_bad_arguments(hip):
    from minit_amd.lib import HipError
    with pytest.raises(HipError, match="multiple of 64"):
        hip.call("mh_i8_gemm", None, 256, 256, 256, 256, 256, None, 4, 4, 100)
    with pytest.raises(HipError, match="no output"):
        hip.call("mh_i8_gemm", None, 256, 256, 256, 256, None, None, 4, 4, 64)
