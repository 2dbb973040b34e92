"""Pins the GPTQ oracle without a GPU: known-answer words, an independent
restatement of the reference's view algebra, closed-form special cases and a
library matmul.  A wrong bit order, a dropped '+ 1', a transposed operand or a
mis-indexed group each fail at least one of these."""
import numpy as np
import pytest

from oracle import gptq as O


def test_unpack_known_answers():
    # sub-word i sits at bit i * bits (little-endian within the word)
    w = np.array([[0x76543210]], dtype=np.uint32).view(np.int32)
    np.testing.assert_array_equal(O.unpack(w, 0, 4)[:, 0], np.arange(8))
    np.testing.assert_array_equal(O.unpack(w, 1, 4)[0], np.arange(8))
    w8 = np.array([[0x03020100]], dtype=np.uint32).view(np.int32)
    np.testing.assert_array_equal(O.unpack(w8, 0, 8)[:, 0], np.arange(4))
    neg = np.array([[-1]], dtype=np.int32)          # all ones: sign bit must not smear
    assert (O.unpack(neg, 0, 4) == 15).all() and (O.unpack(neg, 1, 8) == 255).all()
    hi = np.array([[np.int32(-2**31)]], dtype=np.int32)
    np.testing.assert_array_equal(O.unpack(hi, 0, 4)[:, 0], [0, 0, 0, 0, 0, 0, 0, 8])


@pytest.mark.parametrize("axis", [0, 1])
def test_unpack_agrees_with_reference_view_algebra(axis):
    """The reference unpacks 8-bit sub-words by reinterpreting int32 as uint8 and
    re-arranging views; the shift/mask form must give the same array."""
    rng = np.random.default_rng(axis)
    packed = rng.integers(-2**31, 2**31, size=(6, 10), dtype=np.int64).astype(np.int32)
    np.testing.assert_array_equal(O.unpack(packed, axis, 8), O.unpack_by_views(packed, axis))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("axis", [0, 1])
def test_pack_round_trip_and_layout(bits, axis):
    rng = np.random.default_rng(bits + axis)
    v = rng.integers(0, 1 << bits, size=(32, 24), dtype=np.uint8)
    packed = O.pack(v, axis, bits)
    per = 32 // bits
    assert packed.shape == ((32 // per, 24) if axis == 0 else (32, 24 // per))
    np.testing.assert_array_equal(O.unpack(packed, axis, bits), v)
    # brute force on one word
    if axis == 0:
        word = sum(int(v[i, 3]) << (bits * i) for i in range(per))
        assert np.uint32(packed.view(np.uint32)[0, 3]) == np.uint32(word)


def test_product_packer_matches_oracle_packer():
    from minit_amd.quantize.gptq import pack_subwords
    rng = np.random.default_rng(7)
    for bits in (4, 8):
        v = rng.integers(0, 1 << bits, size=(64, 48), dtype=np.uint8)
        for axis in (0, 1):
            np.testing.assert_array_equal(pack_subwords(v, axis, bits), O.pack(v, axis, bits))


def _tiny(k=64, n=16, g=32, bits=4, seed=0, zero_hi=None):
    rng = np.random.default_rng(seed)
    hi = (1 << bits) if zero_hi is None else zero_hi
    q = rng.integers(0, 1 << bits, size=(k, n), dtype=np.uint8)
    z = rng.integers(0, hi, size=(k // g, n), dtype=np.uint8)
    s = (np.abs(rng.normal(0, 0.02, size=(k // g, n))) + 1e-3).astype(np.float16)
    return q, z, s, O.pack(q, 0, bits), O.pack(z, 1, bits)


def test_dequantize_closed_form_and_special_cases():
    q, z, s, qweight, qzeros = _tiny()
    k, n = q.shape
    g_idx = np.arange(k) // 32
    w = O.dequantize_packed(qweight, qzeros, s, None, 4, 32)
    # elementwise float64 evaluation, one rounding
    ref = ((q.astype(np.float64) - (z[g_idx].astype(np.float64) + 1.0)) * s[g_idx].astype(np.float64))
    np.testing.assert_array_equal(w.view(np.uint16), ref.astype(np.float16).view(np.uint16))
    # q == z + 1  ->  exactly zero;  zero point 15 does not wrap to 0
    z2 = np.full_like(z, 15)
    q2 = np.full_like(q, 15)
    w2 = O.dequantize(q2, g_idx, z2, s)
    np.testing.assert_array_equal(w2, (-s[g_idx]).astype(np.float16))
    w3 = O.dequantize((z[g_idx] + 1).astype(np.uint8), g_idx, z, s)
    assert (w3 == 0).all()
    # unit scales -> the integers themselves
    ones = np.ones_like(s)
    np.testing.assert_array_equal(O.dequantize(q, g_idx, z, ones).astype(np.int32),
                                  q.astype(np.int32) - z[g_idx].astype(np.int32) - 1)


def test_dequantize_act_order_gathers_rows():
    q, z, s, qweight, qzeros = _tiny(seed=3)
    k = q.shape[0]
    g_idx = np.random.default_rng(4).integers(0, 2, size=k).astype(np.int32)
    w = O.dequantize_packed(qweight, qzeros, s, g_idx, 4)
    for kk in (0, 17, 63):
        g = g_idx[kk]
        np.testing.assert_array_equal(
            w[kk], ((q[kk].astype(np.float16) - (z[g].astype(np.float16) + np.float16(1))) * s[g]))


def test_matmul_against_library_and_invariants():
    torch = pytest.importorskip("torch")
    q, z, s, qweight, qzeros = _tiny(k=256, n=40, g=64, seed=5)
    rng = np.random.default_rng(6)
    x = rng.normal(0, 1, size=(5, 256)).astype(np.float16)
    w = O.dequantize_packed(qweight, qzeros, s, None, 4, 64)
    y = O.matmul(x, qweight, qzeros, s, None, 4, 64)
    assert y.dtype == np.float16 and y.shape == (5, 40)
    # library fp32 matmul of the dequantized matrix, [M,K] @ [K,N] (not transposed)
    lib = (torch.from_numpy(x).float() @ torch.from_numpy(w).float()).numpy()
    np.testing.assert_allclose(y.astype(np.float32), lib, atol=2e-2, rtol=2e-3)
    # one-hot rows pick rows of W exactly
    e = np.zeros((3, 256), np.float16)
    e[[0, 1, 2], [7, 100, 255]] = 1
    np.testing.assert_array_equal(O.matmul(e, qweight, qzeros, s, None, 4, 64), w[[7, 100, 255]])
    # linearity of the accumulator
    x2 = rng.normal(0, 1, size=(5, 256)).astype(np.float16)
    f = lambda v: O.matmul_f64(v, qweight, qzeros, s, None, 4, 64)
    np.testing.assert_allclose(f(x) + f(x2), (x.astype(np.float64) + x2.astype(np.float64)) @ w.astype(np.float64),
                               rtol=1e-12, atol=1e-12)
    # leading dimensions are folded
    y3 = O.matmul(x.reshape(5, 1, 256), qweight, qzeros, s, None, 4, 64)
    np.testing.assert_array_equal(y3.reshape(5, 40), y)


def test_matmul_shape_contract():
    q, z, s, qweight, qzeros = _tiny()
    x = np.zeros((1, 64), np.float16)
    with pytest.raises(ValueError):
        O.matmul(x[:, :56], qweight, qzeros, s)
    with pytest.raises(ValueError):
        O.matmul(x, qweight, qzeros[:, :1], s)
    with pytest.raises(ValueError):
        O.matmul(x, qweight, qzeros, s, g_idx=np.zeros(10, np.int32))


def test_silu_mul_forms_agree():
    rng = np.random.default_rng(8)
    g = rng.normal(0, 3, size=1000).astype(np.float16)
    u = rng.normal(0, 3, size=1000).astype(np.float16)
    a = O.silu_mul(g, u).astype(np.float64)
    b = O.silu_mul_f64(g, u)
    assert np.abs(a - b).max() <= 3 * np.spacing(np.abs(b).astype(np.float16)).astype(np.float64).max()
    assert O.silu_mul(np.zeros(4, np.float16), u[:4]).tolist() == [0, 0, 0, 0]
