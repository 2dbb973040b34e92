"""W8A8 int8 GEMM, restated on the CPU.  Test infrastructure only.

The reference has no int8 x int8 product ("qwen1_5_int8" is weight-only,
examples/qwen1_5_int8.py:156-200), so nothing in the reference pins this; the
integer part is pinned by exact arithmetic.  The operand orientation follows
the reference's dense product, ``C[m, n] = sum_k A[m, k] * B[n, k]`` with the
weight stored ``[N, K]`` (minit/operator/linalg.py:29-35,
minit/cuda/kernel/cublas.py:83), and the epilogue is fixed here as

    out[m, n] = fp16( fp32(acc[m, n]) * (a_scale[m] * w_scale[n]) )

with the scale product formed in fp32.
"""
import numpy as np


def gemm_i32(a_mk: np.ndarray, w_nk: np.ndarray) -> np.ndarray:
    """Exact ``int32`` accumulators; |acc| <= 128^2 * K stays far below 2^31.

    Evaluated with a float64 library matmul: every product and partial sum is an
    integer below 2^53, so float64 arithmetic is exact whatever the summation
    order (numpy's integer matmul is not BLAS-backed and takes minutes at the
    benchmark sizes).  Pinned against int64 and brute-force loops in the tests.
    """
    assert a_mk.dtype == np.int8 and w_nk.dtype == np.int8
    assert 128 * 128 * a_mk.shape[1] < 2 ** 31
    acc = a_mk.astype(np.float64) @ w_nk.astype(np.float64).T
    return acc.astype(np.int64).astype(np.int32)


def gemm_i32_int64(a_mk: np.ndarray, w_nk: np.ndarray) -> np.ndarray:
    """The same product in int64 integer arithmetic (slow; for pinning)."""
    return (a_mk.astype(np.int64) @ w_nk.astype(np.int64).T).astype(np.int32)


def gemm_i32_loops(a_mk: np.ndarray, w_nk: np.ndarray) -> np.ndarray:
    """Brute-force triple loop, for pinning :func:`gemm_i32` on tiny shapes."""
    m, k = a_mk.shape
    n = w_nk.shape[0]
    out = np.zeros((m, n), dtype=np.int32)
    for i in range(m):
        for j in range(n):
            s = 0
            for t in range(k):
                s += int(a_mk[i, t]) * int(w_nk[j, t])
            out[i, j] = s
    return out


def dequant_epilogue(acc: np.ndarray, a_scale: np.ndarray, w_scale: np.ndarray) -> np.ndarray:
    """``fp16(fp32(acc) * (a_scale[m] * w_scale[n]))`` with fp32 products."""
    scale = a_scale.astype(np.float32)[:, None] * w_scale.astype(np.float32)[None, :]
    return (acc.astype(np.float32) * scale).astype(np.float16)


def gemm(a_mk, w_nk, a_scale, w_scale):
    acc = gemm_i32(a_mk, w_nk)
    return dequant_epilogue(acc, a_scale, w_scale), acc
