"""Pins the int8 GEMM oracle: brute-force loops, extreme values, the epilogue."""
import numpy as np

from oracle import int8 as O


def test_gemm_i32_matches_brute_force():
    rng = np.random.default_rng(0)
    a = rng.integers(-128, 128, size=(5, 12), dtype=np.int8)
    w = rng.integers(-128, 128, size=(7, 12), dtype=np.int8)
    np.testing.assert_array_equal(O.gemm_i32(a, w), O.gemm_i32_loops(a, w))
    a2 = rng.integers(-128, 128, size=(33, 1024), dtype=np.int8)
    w2 = rng.integers(-128, 128, size=(65, 1024), dtype=np.int8)
    np.testing.assert_array_equal(O.gemm_i32(a2, w2), O.gemm_i32_int64(a2, w2))
    # orientation: w is [N, K]
    assert O.gemm_i32(a, w).shape == (5, 7)
    assert O.gemm_i32(a, w)[2, 3] == int(a[2].astype(np.int32) @ w[3].astype(np.int32))


def test_gemm_i32_extremes():
    a = np.full((2, 4096), -128, np.int8)
    w = np.full((3, 4096), -128, np.int8)
    assert (O.gemm_i32(a, w) == 128 * 128 * 4096).all()
    w[:] = 127
    assert (O.gemm_i32(a, w) == -128 * 127 * 4096).all()


def test_epilogue_is_fp32_then_fp16():
    acc = np.array([[1, -3], [100000, 7]], np.int32)
    sa = np.array([0.5, 0.25], np.float32)
    sw = np.array([2.0, 0.125], np.float32)
    out = O.dequant_epilogue(acc, sa, sw)
    assert out.dtype == np.float16
    np.testing.assert_array_equal(out, np.array([[1.0, -0.1875], [50000.0, 0.21875]], np.float16))
