"""GPU parity of the row-wise and element-wise kernels in the other two storage
types the reference's kernels are generated for (bfloat16 and float32,
minit/cuda/dispatch.py:430-478 with get_cuda_dtype): fp32 arithmetic inside, one
rounding to the storage type at the store.  bfloat16 travels as raw uint16 bits
(numpy has no such type); expected values are the float64 closed forms of the
oracle rounded to bfloat16 here, and one bfloat16 step of slack covers the fp32
internals."""
import numpy as np
import pytest

from oracle import special as O

pytestmark = pytest.mark.gpu


def _to_bf16_bits(x) -> np.ndarray:
    """Round-to-nearest-even float -> bfloat16 bits."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    rounded = u + 0x7FFF + ((u >> 16) & 1)
    return (rounded >> 16).astype(np.uint16)


def _from_bf16_bits(b) -> np.ndarray:
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def _bf16(values):
    """float32 array holding bfloat16-representable values."""
    return _from_bf16_bits(_to_bf16_bits(values))


def _dev(arr32, dtype):
    from minit_amd.hip.tensor import HIPTensor
    if dtype == "float32":
        return HIPTensor.from_numpy(np.ascontiguousarray(arr32, dtype=np.float32))
    t = HIPTensor.allocate(arr32.shape, "bfloat16")
    t.copy_from_numpy(_to_bf16_bits(arr32))
    return t


def _host(t):
    a = t.numpy()
    return _from_bf16_bits(a) if t.dtype == "bfloat16" else a


def _check(got32, ref64, dtype, what, ulps=1.0, atol=1e-6):
    ref64 = np.asarray(ref64, np.float64)
    if dtype == "float32":
        tol = 4e-6 * np.maximum(np.abs(ref64), 1e-3) + atol
    else:
        tol = ulps * np.abs(ref64) * 2.0 ** -7 + atol     # a bfloat16 step is at most 2^-7 of the value
    err = np.abs(got32.astype(np.float64) - ref64)
    finite = np.isfinite(ref64)
    assert (err[finite] <= tol[finite]).all(), f"{what} {dtype}: worst {err[finite].max():.4g}"
    assert (got32[~finite] == ref64[~finite]).all()


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_rowwise_kernels_in_other_storage_types(hip, dtype):
    import minit_amd.functional as F
    rng = np.random.default_rng(3)
    prep = _bf16 if dtype == "bfloat16" else (lambda v: np.asarray(v, np.float32))
    x = prep(rng.normal(0, 1, size=(6, 520)))
    w = prep(rng.normal(1, 0.1, size=520))
    got = _host(F.rms_norm(_dev(x, dtype), _dev(w, dtype), 1, 1e-5))
    _check(got, O.rms_norm(x.astype(np.float64), w.astype(np.float64), 1, 1e-5), dtype, "rms_norm")

    s = prep(rng.normal(0, 3, size=(5, 3, 333)))
    for axis in (2, 1):
        got = _host(F.softmax(_dev(s, dtype), axis))
        _check(got, O.softmax(s.astype(np.float64), axis), dtype, f"softmax axis {axis}", atol=1e-7)
        got = _host(F.sum(_dev(s, dtype), axis))
        _check(got, s.astype(np.float64).sum(axis=axis, keepdims=True), dtype, f"sum axis {axis}", atol=2e-1 if dtype == "bfloat16" else 1e-4)
        got = _host(F.max(_dev(s, dtype), axis))
        assert np.array_equal(got, s.max(axis=axis, keepdims=True))
    ones = np.ones((3, 256), np.float32)
    assert (_host(F.sum(_dev(ones, dtype), 1)) == 256).all() and (_host(F.mean(_dev(ones, dtype), 1)) == 1).all()

    q = prep(rng.normal(0, 1, size=(2, 3, 4, 128)))
    cos, sin = O.rope_tables(128, 3, 1e4)
    from minit_amd.hip.tensor import HIPTensor
    got = _host(F.rope(_dev(q, dtype), HIPTensor.from_numpy(cos), HIPTensor.from_numpy(sin)))
    ref = O.rope(q.astype(np.float64), cos, sin)
    _check(got, ref, dtype, "rope", atol=1e-2 if dtype == "bfloat16" else 1e-5)

    g = prep(rng.normal(0, 3, size=(4, 1031)))
    u = prep(rng.normal(0, 3, size=(4, 1031)))
    _check(_host(F.sigmoid(_dev(g, dtype))), 1.0 / (1.0 + np.exp(-g.astype(np.float64))), dtype, "sigmoid")
    _check(_host(F.multiply(_dev(g, dtype), _dev(u, dtype))), g.astype(np.float64) * u.astype(np.float64), dtype,
           "multiply", ulps=0.51)


def test_bf16_rounding_helpers():
    assert _to_bf16_bits([1.0, -2.0, 0.0])[0] == 0x3F80
    assert _from_bf16_bits(_to_bf16_bits([1.0 + 2.0 ** -8]))[0] == 1.0          # tie to even
    assert _from_bf16_bits(_to_bf16_bits([1.0 + 3 * 2.0 ** -8]))[0] == 1.0 + 2.0 ** -6
