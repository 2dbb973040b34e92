"""Shared checks for the parity tests."""
import numpy as np

# Tolerance of the quantized-linear path: fp16 outputs within max-abs 1e-2 and
# relative L2 1e-3 of dequant(fp16) + matmul(fp32 accumulate).  fp16 cannot
# resolve 1e-2 once |y| >= 16 (its spacing there is >= 1.56e-2), so where the
# spacing of the reference value itself exceeds the bound, one fp16 step is
# allowed instead.
MAX_ABS = 1e-2
REL_L2 = 1e-3


def fp16_spacing(x: np.ndarray) -> np.ndarray:
    return np.spacing(np.abs(x).astype(np.float16)).astype(np.float64)


def assert_fp16_close(got: np.ndarray, ref_f64: np.ndarray, max_abs: float = MAX_ABS,
                      rel_l2: float = REL_L2, what: str = ""):
    assert got.dtype == np.float16, got.dtype
    assert got.shape == ref_f64.shape, (got.shape, ref_f64.shape)
    ref16 = ref_f64.astype(np.float16)
    g = got.astype(np.float64)
    r = ref16.astype(np.float64)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    err = np.abs(g - r)
    tol = np.maximum(max_abs, fp16_spacing(ref16))
    bad = err > tol
    assert not bad.any(), (f"{what}: {bad.sum()} elements beyond tolerance, worst |err|={err.max():.4g} "
                           f"at {np.unravel_index(err.argmax(), err.shape)} (ref {r.flat[err.argmax()]:.4g})")
    denom = np.linalg.norm(r)
    if denom > 0:
        rel = np.linalg.norm(g - r) / denom
        assert rel <= rel_l2, f"{what}: relative L2 error {rel:.3g} > {rel_l2}"
