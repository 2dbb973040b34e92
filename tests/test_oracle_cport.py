"""The C restatement (CPU baseline) must agree bit for bit with the numpy oracle."""
import numpy as np
import pytest

from oracle import cport
from oracle import gptq as O


def test_half_conversions_exhaustive():
    lib = cport.lib()
    bits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_half_to_float(int(b)) for b in bits[::7]], np.float32)
    finite_or_inf = ~np.isnan(ref[::7])          # NaN payloads are not compared
    np.testing.assert_array_equal(got.view(np.uint32)[finite_or_inf], ref[::7].view(np.uint32)[finite_or_inf])
    assert np.isnan(got[~finite_or_inf]).all()
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.normal(0, 1, 2000), rng.normal(0, 1e-6, 2000), rng.normal(0, 3e4, 2000),
                           [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 6.1e-5, 5.96e-8, 2.98e-8, 2.9802323e-8]])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([lib.oracle_double_to_half(float(v)) for v in vals], np.uint16)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("bits,group_size", [(4, 128), (4, 32), (8, 64)])
def test_c_port_matches_numpy_oracle(bits, group_size):
    from minit_amd import synthetic
    k, n, m = 512, 264, 3
    qweight, qzeros, scales = synthetic.gptq_weights("cport", f"w{bits}", k, n, group_size, bits,
                                                     zero_range=(0, (1 << bits) - 1))
    x = synthetic.activations("cport", "x", (m, k))
    np.testing.assert_array_equal(cport.dequant(qweight, qzeros, scales, None, bits, group_size).view(np.uint16),
                                  O.dequantize_packed(qweight, qzeros, scales, None, bits, group_size).view(np.uint16))
    np.testing.assert_array_equal(cport.matmul(x, qweight, qzeros, scales, None, bits, group_size).view(np.uint16),
                                  O.matmul(x, qweight, qzeros, scales, None, bits, group_size).view(np.uint16))
    g_idx = (np.random.default_rng(1).permutation(k) // group_size).astype(np.int32)
    np.testing.assert_array_equal(cport.matmul(x, qweight, qzeros, scales, g_idx, bits, group_size).view(np.uint16),
                                  O.matmul(x, qweight, qzeros, scales, g_idx, bits, group_size).view(np.uint16))
