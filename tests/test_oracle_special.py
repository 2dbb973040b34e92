"""Pins the RMSNorm / RoPE / softmax / reduction oracle through invariants the
mathematics fixes."""
import numpy as np

from oracle import special as O


def test_rms_norm_invariants():
    rng = np.random.default_rng(0)
    w = rng.normal(1, 0.1, size=64).astype(np.float32)
    x = rng.normal(0, 1, size=(3, 64)).astype(np.float32)
    y = O.rms_norm(x, w, 1, 1e-6)
    # scale invariance (eps negligible) and unit RMS before the weight
    np.testing.assert_allclose(O.rms_norm(4 * x, w, 1, 1e-12), O.rms_norm(x, w, 1, 1e-12), rtol=1e-5)
    np.testing.assert_allclose(np.sqrt(((y / w) ** 2).mean(axis=1)), 1.0, rtol=1e-4)
    # constant row -> sign * w
    c = np.full((1, 64), -2.5, np.float32)
    np.testing.assert_allclose(O.rms_norm(c, w, 1, 1e-12), -w[None], rtol=1e-6)
    # eps matters for tiny rows: x = 0 -> 0
    assert (O.rms_norm(np.zeros((1, 64), np.float32), w, 1, 1e-6) == 0).all()
    # middle axis == moving the axis last
    x3 = rng.normal(0, 1, size=(2, 64, 5)).astype(np.float32)
    a = O.rms_norm(x3, w, 1, 1e-6)
    b = np.moveaxis(O.rms_norm(np.moveaxis(x3, 1, 2).copy(), w, 2, 1e-6), 2, 1)
    np.testing.assert_allclose(a, b, rtol=1e-6)


def test_rope_invariants():
    rng = np.random.default_rng(1)
    hs = 16
    cos, sin = O.rope_tables(hs, 64, 1e4)
    assert cos.dtype == np.float32 and cos.shape == (64, 8)
    np.testing.assert_allclose(cos[0], 1.0)
    np.testing.assert_allclose(sin[0], 0.0)
    # textbook angle: position p, pair i -> p * theta^(-2i/hs)
    np.testing.assert_allclose(cos[5, 3], np.cos(5 * 1e4 ** (-6 / 16)), rtol=1e-6)
    x = rng.normal(0, 1, size=(2, 3, 4, hs)).astype(np.float32)
    # position 0 is the identity
    pos0 = np.zeros((2, 3), np.int32)
    np.testing.assert_allclose(O.rope(x, cos, sin, pos0), x, rtol=1e-6)
    # norm of each pair is preserved; rotations compose additively
    p1 = rng.integers(0, 30, size=(2, 3)).astype(np.int32)
    p2 = rng.integers(0, 30, size=(2, 3)).astype(np.int32)
    y = O.rope(x, cos, sin, p1)
    pair = lambda v: v.reshape(*v.shape[:-1], hs // 2, 2)
    np.testing.assert_allclose((pair(y) ** 2).sum(-1), (pair(x) ** 2).sum(-1), rtol=1e-5)
    np.testing.assert_allclose(O.rope(y, cos, sin, p2), O.rope(x, cos, sin, p1 + p2), rtol=1e-4, atol=1e-5)
    # explicit rotation of one pair, sign convention of the reference kernel
    one = np.zeros((1, 1, 1, hs), np.float32)
    one[..., 2], one[..., 3] = 1.0, 2.0       # pair i = 1
    out = O.rope(one, cos[7:8], sin[7:8])
    c, s = cos[7, 1], sin[7, 1]
    np.testing.assert_allclose(out[0, 0, 0, 2:4], [1 * c - 2 * s, 2 * c + 1 * s], rtol=1e-6)
    # the sequence-index form equals the positions form on a sliced table
    xs = rng.normal(0, 1, size=(2, 3, 4, hs)).astype(np.float32)
    pos = np.broadcast_to(np.arange(10, 13, dtype=np.int32), (2, 3))
    np.testing.assert_array_equal(O.rope(xs, cos[10:13], sin[10:13]), O.rope(xs, cos, sin, pos))


def test_softmax_invariants():
    rng = np.random.default_rng(2)
    x = rng.normal(0, 3, size=(4, 50)).astype(np.float32)
    p = O.softmax(x, 1)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, rtol=1e-6)
    np.testing.assert_allclose(O.softmax(x + 5.0, 1), p, rtol=1e-5)
    np.testing.assert_allclose(O.softmax(np.zeros((1, 8), np.float32), 1), 1 / 8)
    x[:, 10:] = -np.inf
    p = O.softmax(x, 1)
    assert (p[:, 10:] == 0).all()
    np.testing.assert_allclose(p[:, :10].sum(axis=1), 1.0, rtol=1e-6)
    # ratio form
    np.testing.assert_allclose(p[0, 1] / p[0, 0], np.exp(x[0, 1] - x[0, 0]), rtol=1e-5)


def test_causal_mask_matches_the_models_recipe():
    m = O.causal_mask(3, 2, np.float32)        # [3, 5]
    expect = np.array([[0, 0, 0, -np.inf, -np.inf],
                       [0, 0, 0, 0, -np.inf],
                       [0, 0, 0, 0, 0]], np.float32)
    np.testing.assert_array_equal(m, expect)
    # decode step (s = 1): the mask is identically zero
    assert (O.causal_mask(1, 9) == 0).all()
    scores = np.random.default_rng(3).normal(0, 3, size=(1, 2, 3, 5)).astype(np.float32)
    p = O.masked_softmax(scores, 2)
    assert (p[..., 0, 3:] == 0).all() and (p[..., 2, :] > 0).all()
    np.testing.assert_allclose(p.sum(-1), 1.0, rtol=1e-6)


def test_reductions():
    x = np.random.default_rng(4).normal(0, 1, size=(3, 7, 2)).astype(np.float32)
    assert O.reduce_sum(x, 1).shape == (3, 1, 2)
    np.testing.assert_allclose(O.reduce_sum(x, 1)[:, 0], x.sum(axis=1), rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(O.reduce_max(x, 1)[:, 0], x.max(axis=1))
    assert (O.reduce_sum(np.ones((2, 9), np.float16), 1) == 9).all()
    # mean = T(T(sum) / T(n)): constant rows give the constant; the sum is rounded
    # first (2049 ones of fp16 sum to 2048), and so is the length (2049 -> 2048)
    assert (O.reduce_mean(np.full((2, 9), 0.5, np.float16), 1) == 0.5).all()
    assert O.reduce_mean(np.ones((1, 2049), np.float16), 1)[0, 0] == 1.0
    big = np.full((1, 3000), 2.0, np.float16)          # sum 6000 is exact, n = 3000 is exact
    assert O.reduce_mean(big, 1)[0, 0] == 2.0
    m = O.reduce_mean(x, 1)
    assert m.shape == (3, 1, 2)
    np.testing.assert_allclose(m[:, 0], x.mean(axis=1), rtol=2e-3, atol=1e-6)


def test_sigmoid_and_multiply():
    """The element-wise expressions of the models' silu (minit/cuda/dispatch.py:137,143)."""
    x = np.array([0.0, 1.0, -1.0, 20.0, -20.0, 0.5], np.float16)
    s = O.sigmoid(x)
    assert s.dtype == np.float16 and s[0] == 0.5
    assert s[3] == 1.0 and 0 <= s[4] < 1e-7                       # saturation, no NaN
    assert abs(float(s[1]) + float(s[2]) - 1.0) <= 2 ** -11       # sigmoid(-x) = 1 - sigmoid(x)
    assert abs(float(s[1]) - 1 / (1 + np.exp(-1.0))) <= 2 ** -12  # half an fp16 step at 0.73
    # the product is rounded once: 1.001 * 1.001 in fp16
    a = np.array([1.0009765625, 3.0, -0.5], np.float16)
    b = np.array([1.0009765625, 0.333251953125, 0.5], np.float16)
    np.testing.assert_array_equal(O.multiply(a, b), np.array([1.001953125, 1.0, -0.25], np.float16))
    # and it composes to the three-rounding silu(gate) * up of the quantized-path oracle
    from oracle import gptq as OG
    rng = np.random.default_rng(12)
    g = rng.normal(0, 3, 4096).astype(np.float16)
    u = rng.normal(0, 3, 4096).astype(np.float16)
    np.testing.assert_array_equal(O.multiply(O.multiply(g, O.sigmoid(g)), u).view(np.uint16),
                                  OG.silu_mul(g, u).view(np.uint16))
