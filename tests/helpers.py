"""Shared checks for the parity tests."""
import numpy as np

# Tolerance of the quantized-linear path: fp16 outputs within max-abs 1e-2 and
# relative L2 1e-3 of dequant(fp16) + matmul(fp32 accumulate).  fp16 cannot
# resolve 1e-2 once |y| >= 16 (its spacing there is >= 1.56e-2), so where the
# spacing of the reference value itself exceeds the bound, one fp16 step is
# allowed instead -- for a bounded share of the outputs only: an fp32 sum taken
# in another order can land on the other side of a rounding boundary, which
# happens to a few outputs in a hundred, not to most of them.
MAX_ABS = 1e-2
REL_L2 = 1e-3
# share of the outputs with |ref| >= 16 that may differ from the reference by one
# fp16 step (observed: below 2 % at K = 28672; a kernel that is off by a step
# everywhere sits near 100 %)
ONE_STEP_SHARE = 0.06
ONE_STEP_FLOOR = 3          # tiny outputs: a handful of flips says nothing

LAST_REPORT = {}            # what the latest call found, for tests that print or aggregate it


def fp16_spacing(x: np.ndarray) -> np.ndarray:
    return np.spacing(np.abs(x).astype(np.float16)).astype(np.float64)


def fp16_error_report(got: np.ndarray, ref_f64: np.ndarray, max_abs: float = MAX_ABS) -> dict:
    """Counts, for fp16 ``got`` against the float64 reference: elements beyond the
    tolerance, elements that needed the one-step allowance (error above ``max_abs``
    but within one fp16 step of a reference value whose spacing exceeds ``max_abs``),
    and how many elements are that large at all."""
    ref16 = ref_f64.astype(np.float16)
    g = got.astype(np.float64)
    r = ref16.astype(np.float64)
    err = np.abs(g - r)
    spacing = fp16_spacing(ref16)
    tol = np.maximum(max_abs, spacing)
    coarse = spacing > max_abs
    denom = np.linalg.norm(r)
    return {"n": int(err.size), "beyond": int((err > tol).sum()), "needed_one_step": int((err > max_abs).sum()),
            "coarse": int(coarse.sum()), "worst": float(err.max()) if err.size else 0.0,
            "worst_at": np.unravel_index(int(err.argmax()), err.shape) if err.size else (),
            "worst_over_tol": float((err / tol).max()) if err.size else 0.0,
            "rel_l2": float(np.linalg.norm(g - r) / denom) if denom > 0 else 0.0,
            "max_ref": float(np.abs(r).max()) if err.size else 0.0}


def assert_fp16_close(got: np.ndarray, ref_f64: np.ndarray, max_abs: float = MAX_ABS,
                      rel_l2: float = REL_L2, what: str = ""):
    assert got.dtype == np.float16, got.dtype
    assert got.shape == ref_f64.shape, (got.shape, ref_f64.shape)
    assert np.isfinite(got.astype(np.float64)).all(), f"{what}: non-finite output"
    rep = fp16_error_report(got, ref_f64, max_abs)
    LAST_REPORT.clear()
    LAST_REPORT.update(rep, what=what)
    assert rep["beyond"] == 0, (f"{what}: {rep['beyond']} elements beyond tolerance, worst |err|={rep['worst']:.4g} "
                                f"at {rep['worst_at']}")
    # the one-step allowance: none where fp16 resolves the bound, a bounded share where it does not
    allowed = 0 if rep["coarse"] == 0 else max(ONE_STEP_FLOOR, int(ONE_STEP_SHARE * rep["coarse"]))
    assert rep["needed_one_step"] <= allowed, (
        f"{what}: {rep['needed_one_step']} of {rep['coarse']} outputs with |ref| >= 16 are one fp16 step off "
        f"(allowed {allowed}): more than summation order explains")
    if rep["needed_one_step"]:
        print(f"[fp16] {what}: {rep['needed_one_step']} of {rep['n']} outputs ({rep['coarse']} with |ref| >= 16) "
              f"used the one-step allowance, worst |err| {rep['worst']:.4g}")
    assert rep["rel_l2"] <= rel_l2, f"{what}: relative L2 error {rep['rel_l2']:.3g} > {rel_l2}"
    return rep
