"""GPU parity: RMSNorm, RoPE, softmax (+ causal), sum / max, SiLU*up, and the
dense fp16 product, against the float64 closed forms of the oracle.

Tolerances (fp16 storage, fp32 arithmetic on the device, float64 in the oracle):
the result may differ from the correctly rounded value by one fp16 step when the
fp32 intermediate lands next to a rounding boundary, so outputs are compared to
within 1 fp16 ulp of the reference plus a small absolute term."""
import numpy as np
import pytest

from helpers import assert_fp16_close, fp16_spacing
from oracle import gptq as OG
from oracle import special as O

pytestmark = pytest.mark.gpu


def _t(arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


def _assert_ulp(got, ref, ulps=1.0, atol=1e-6, what=""):
    g, r = got.astype(np.float64), ref.astype(np.float64)
    tol = ulps * fp16_spacing(ref) + atol
    err = np.abs(g - r)
    assert (err <= tol).all(), f"{what}: worst {err.max():.4g} (tol {tol.flat[err.argmax()]:.4g})"


@pytest.mark.parametrize("shape,axis", [
    ((16, 4096), 1),        # config 3
    ((4, 8192), 1),         # 70B hidden size
    ((3, 5, 264), 2),
    ((2, 100, 6), 1),       # normalise a middle axis (strided path)
    ((7, 33), 1),           # not a multiple of the vector width
    ((37, 128), 1),         # 16 threads per row, 16 rows per workgroup, the last workgroup part empty
    ((2, 19, 64), 2),       # ... half of the 16 threads of a row without a piece
    ((21, 520), 1),         # 64 threads per row, two pieces per lane, the second part empty
    ((9, 2048), 1),         # ... four pieces per lane
    ((6, 2056), 1),         # ... five of up to eight pieces per lane, the fifth for one lane only
    ((5, 16384), 1),        # longer than the registers of a workgroup: two walks over the row
    ((3, 28680), 1),        # ... a length that is no multiple of the workgroup's stride
])
def test_rms_norm(hip, shape, axis):
    import minit_amd.functional as F
    rng = np.random.default_rng(1)
    x = rng.normal(0, 1, size=shape).astype(np.float16)
    w = rng.normal(1, 0.1, size=shape[axis]).astype(np.float16)
    got = F.rms_norm(_t(x), _t(w), axis, 1e-6).numpy()
    _assert_ulp(got, O.rms_norm(x, w, axis, 1e-6), what=f"rms_norm {shape}")


def test_rms_norm_constant_row(hip):
    """A constant row c normalises to sign(c) * w (eps negligible)."""
    import minit_amd.functional as F
    x = np.full((2, 4096), -3.0, dtype=np.float16)
    w = np.random.default_rng(2).normal(1, 0.1, size=4096).astype(np.float16)
    got = F.rms_norm(_t(x), _t(w), 1, 1e-6).numpy()
    _assert_ulp(got, np.broadcast_to(-w, x.shape), what="constant row")


@pytest.mark.parametrize("use_positions", [False, True])
def test_rope(hip, use_positions):
    import minit_amd.functional as F
    from minit_amd import synthetic
    rng = np.random.default_rng(3)
    bs, seq, nh, hs = (16, 1, 32, 128) if use_positions else (2, 5, 4, 128)
    x = rng.normal(0, 1, size=(bs, seq, nh, hs)).astype(np.float16)
    cos, sin = synthetic.rope_tables(hs, 4096, 1e6)
    if use_positions:
        pos = rng.integers(0, 4096, size=(bs, seq)).astype(np.int32)   # config 3
        got = F.rope(_t(x), _t(cos), _t(sin), positions=_t(pos)).numpy()
        ref = O.rope(x, cos, sin, pos)
    else:
        offset = 37
        got = F.rope(_t(x), _t(cos[offset:offset + seq]), _t(sin[offset:offset + seq])).numpy()
        ref = O.rope(x, cos[offset:offset + seq], sin[offset:offset + seq])
        # the positions form reduces to the reference form
        pos = np.broadcast_to(np.arange(offset, offset + seq, dtype=np.int32), (bs, seq)).copy()
        got2 = F.rope(_t(x), _t(cos), _t(sin), positions=_t(pos)).numpy()
        np.testing.assert_array_equal(got.view(np.uint16), got2.view(np.uint16))
    _assert_ulp(got, ref, what="rope")


def test_rope_scalar_path(hip):
    """Head size whose half is not a multiple of four takes the per-pair kernel."""
    import minit_amd.functional as F
    rng = np.random.default_rng(4)
    x = rng.normal(0, 1, size=(2, 3, 2, 12)).astype(np.float16)
    cos, sin = O.rope_tables(12, 3, 1e4)
    got = F.rope(_t(x), _t(cos), _t(sin)).numpy()
    _assert_ulp(got, O.rope(x, cos, sin), what="rope scalar")


@pytest.mark.parametrize("shape,axis", [
    ((16, 32, 1, 1024), 3),   # config 3
    ((16, 32, 1, 4096), 3),
    ((2, 3, 40), 2),
    ((4, 50, 3), 1),          # strided
    ((2, 16384), 1),          # longer than the register-resident path
    ((3, 128264), 1),         # ... a vocabulary-sized row, no multiple of the workgroup's stride
    ((37, 128), 1),           # 16 threads per row
    ((2, 19, 72), 2),         # ... nine of them with a piece
    ((21, 520), 1),           # 64 threads per row, two pieces per lane
    ((9, 2048), 1),           # ... four pieces per lane
    ((6, 3080), 1),           # ... seven of up to eight pieces per lane
])
def test_softmax(hip, shape, axis):
    import minit_amd.functional as F
    x = np.random.default_rng(5).normal(0, 3, size=shape).astype(np.float16)
    got = F.softmax(_t(x), axis).numpy()
    ref = O.softmax(x, axis)
    _assert_ulp(got, ref, what=f"softmax {shape}")
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=axis), 1.0, atol=2e-3)


def test_softmax_with_minus_inf(hip):
    """-inf entries (the models' additive mask) come out as exact zeros."""
    import minit_amd.functional as F
    x = np.random.default_rng(6).normal(0, 3, size=(4, 256)).astype(np.float16)
    x[:, 100:] = -np.inf
    got = F.softmax(_t(x), 1).numpy()
    assert (got[:, 100:] == 0).all()
    _assert_ulp(got, O.softmax(x, 1), what="softmax -inf")


@pytest.mark.parametrize("b,n,s,offset", [(2, 3, 8, 24), (16, 32, 1, 1023), (1, 2, 16, 0),
                                          (2, 3, 40, 88),       # rows of 128: 16 threads per row
                                          (1, 2, 100, 412),     # rows of 512: 64 threads per row
                                          (1, 1, 5, 9003)])     # rows of 9008: three walks over the row
def test_softmax_causal(hip, b, n, s, offset):
    from minit_amd.hip.tensor import HIPTensor
    t = offset + s
    x = np.random.default_rng(7).normal(0, 3, size=(b, n, s, t)).astype(np.float16)
    out = HIPTensor.allocate(x.shape, "float16")
    dx = _t(x)
    hip.call("mh_softmax_causal", None, dx.data_ptr, out.data_ptr, b * n, s, t, offset, 1.0, 0)
    ref = O.masked_softmax(x, offset)
    got = out.numpy()
    _assert_ulp(got, ref, what="causal softmax")
    assert (got[ref == 0] == 0).all()
    # with the 1/sqrt(d) scale fused: same as scaling (rounded to fp16) first
    scale = np.float32(O.attention_scale(128))
    hip.call("mh_softmax_causal", None, dx.data_ptr, out.data_ptr, b * n, s, t, offset, float(scale), 0)
    xs = (x.astype(np.float32) * scale).astype(np.float16)
    _assert_ulp(out.numpy(), O.masked_softmax(xs, offset), what="causal softmax scaled")


@pytest.mark.parametrize("shape,axis", [((512, 4096), 1), ((512, 1024), 1), ((3, 77, 5), 1), ((9, 13), 1),
                                        ((37, 128), 1), ((35, 100), 1), ((21, 520), 1), ((5, 16392), 1),
                                        ((3, 40011), 1)])   # a workgroup of 1024 threads per row, scalar tail
def test_sum_max(hip, shape, axis):
    import minit_amd.functional as F
    x = np.random.default_rng(8).normal(0, 3, size=shape).astype(np.float16)
    s = F.sum(_t(x), axis).numpy()
    assert s.shape == O.reduce_sum(x, axis).shape
    _assert_ulp(s, O.reduce_sum(x, axis), atol=1e-3, what="sum")
    np.testing.assert_array_equal(F.max(_t(x), axis).numpy(), O.reduce_max(x, axis))
    ones = np.ones(shape, np.float16)
    assert (F.sum(_t(ones), axis).numpy() == shape[axis]).all()
    # mean: the rounded sum divided by the rounded length, rounded again
    s16 = s.astype(np.float64)
    n16 = np.float64(np.asarray(shape[axis]).astype(np.float16))
    np.testing.assert_array_equal(F.mean(_t(x), axis).numpy(), (s16 / n16).astype(np.float16))
    assert (F.mean(_t(ones), axis).numpy() == 1).all()


def test_silu_mul(hip):
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(9)
    g = rng.normal(0, 3, size=(8, 28672)).astype(np.float16)
    u = rng.normal(0, 3, size=(8, 28672)).astype(np.float16)
    out = HIPTensor.allocate(g.shape, "float16")
    dg, du = _t(g), _t(u)
    hip.call("mh_silu_mul", None, dg.data_ptr, du.data_ptr, out.data_ptr, g.size, 1, 0)
    # three-rounding form of the models: equal up to expf vs exp in the sigmoid
    _assert_ulp(out.numpy(), OG.silu_mul(g, u), ulps=1.0, what="silu_mul exact")
    mism = (out.numpy().view(np.uint16) != OG.silu_mul(g, u).view(np.uint16)).mean()
    assert mism < 1e-3, f"{mism:.2%} of elements differ from the three-rounding form"
    hip.call("mh_silu_mul", None, dg.data_ptr, du.data_ptr, out.data_ptr, g.size, 0, 0)
    _assert_ulp(out.numpy(), OG.silu_mul_f64(g, u).astype(np.float16), what="silu_mul fused")


def test_sigmoid_multiply_compose_to_silu(hip):
    """``x * F.sigmoid(x)`` and ``silu(gate) * up`` through the operator API, as
    the models spell them (examples/llama3_70b.py:44-45,126-130): the product is
    bit-exact, sigmoid is the oracle's up to expf against exp, and the composition
    equals the fused kernel's three-rounding mode bit for bit."""
    import minit_amd.functional as F
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(13)
    g = rng.normal(0, 3, size=(5, 1031)).astype(np.float16)      # odd width: vector body and scalar tail
    u = rng.normal(0, 3, size=(5, 1031)).astype(np.float16)
    dg, du = _t(g), _t(u)
    np.testing.assert_array_equal(F.multiply(dg, du).numpy().view(np.uint16), O.multiply(g, u).view(np.uint16))
    sig = F.sigmoid(dg).numpy()
    _assert_ulp(sig, O.sigmoid(g), ulps=1.0, what="sigmoid")
    assert (sig.view(np.uint16) != O.sigmoid(g).view(np.uint16)).mean() < 1e-3
    h = ((dg * F.sigmoid(dg)) * du).numpy()
    fused = HIPTensor.allocate(g.shape, "float16")
    hip.call("mh_silu_mul", None, dg.data_ptr, du.data_ptr, fused.data_ptr, g.size, 1, 0)
    np.testing.assert_array_equal(h.view(np.uint16), fused.numpy().view(np.uint16))
    _assert_ulp(h, OG.silu_mul(g, u), ulps=1.0, what="silu through operators")
    with pytest.raises(AssertionError):
        F.multiply(dg, _t(u[:2]))
    # the residual add: one fp16 rounding, equal to numpy's half add bit for bit
    np.testing.assert_array_equal((dg + du).numpy().view(np.uint16), (g + u).view(np.uint16))
    np.testing.assert_array_equal(F.add(dg, du).numpy().view(np.uint16), O.add(g, u).view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(1, 1000, 512), (8, 128256, 256), (40, 72, 4096), (3, 50, 37),
                                   # one to four rows and a tall weight: the dot-product kernel (row groups of
                                   # four, ragged last group, waves with one group more than others)
                                   (1, 128256, 1024), (2, 8193, 2048), (3, 9001, 1024), (4, 8192, 8192), (8, 8200, 8192), (5, 16390, 1024),
                                   (1, 8190, 4096),
                                   # more than eight rows and a tall weight: the weight streamed through LDS (ragged
                                   # last tile, seven rounds for six stages; exactly six rounds, four row tiles; two
                                   # blocks of 64 rows, the second ragged)
                                   (9, 16390, 448), (33, 16384, 384), (64, 20000, 1024), (70, 16400, 512), (32, 32768, 2048),
                                   # 17 rows (two row tiles, the second ragged) on a ragged last tile of columns; 48 rows (four row tiles, one empty)
                                   (17, 16390, 640), (48, 16384, 512),
                                   # more than eight rows and a weight of few rows: the four waves of a workgroup split K
                                   # (one, two and four row tiles, ragged columns, two row blocks, nine steps of 128 k per wave set)
                                   (16, 200, 1024), (20, 1000, 2048), (100, 520, 1152), (32, 8192, 8192)])
def test_dense_matmul_nk(hip, m, n, k):
    import minit_amd.functional as F
    rng = np.random.default_rng(10)
    a = rng.normal(0, 1, size=(m, k)).astype(np.float16)
    b = rng.normal(0, 0.05, size=(n, k)).astype(np.float16)
    got = F.matrix_multiply(_t(a), _t(b)).numpy()
    assert_fp16_close(got, a.astype(np.float64) @ b.astype(np.float64).T, what="dense nk")


def test_batch_matrix_multiply(hip):
    """BatchMatrixMultiply (minit/cuda/dispatch.py:82-101): c[i] = a[i] @ b[i]^T, leading axes folded
    (minit/functional/linalg.py:23-33) -- the two products either side of the models' softmax."""
    import minit_amd.functional as F
    rng = np.random.default_rng(12)
    a = rng.normal(0, 1, size=(2, 3, 5, 128)).astype(np.float16)       # [b, heads, s, d]
    b = rng.normal(0, 0.2, size=(2, 3, 40, 128)).astype(np.float16)    # [b, heads, t, d]
    got = F.batch_matrix_multiply(_t(a), _t(b)).numpy()
    assert got.shape == (2, 3, 5, 40)
    ref = np.einsum("bhsd,bhtd->bhst", a.astype(np.float64), b.astype(np.float64))
    assert_fp16_close(got.reshape(-1, 40), ref.reshape(-1, 40), what="batched nk")


@pytest.mark.parametrize("batch,m,n,k", [(6, 5, 40, 128),      # q.k^T of a short prefill, one 16-row tile
                                         (64, 70, 70, 128),    # 64 heads, four row tiles, ragged
                                         (3, 33, 129, 64),     # two row tiles, ragged columns
                                         (4, 7, 9, 20),        # K not a multiple of 32: the generic kernel
                                         (1, 12, 300, 96),     # a batch of one
                                         (3, 24, 100, 1024),   # 17 rows and more, K of 384 and more: the weight through LDS
                                         (2, 70, 130, 512),    # the same with two blocks of rows and two tiles of columns, both ragged
                                         (3, 12, 100, 1024)])  # up to 16 rows: the waves of a workgroup split K
def test_batched_dense_product_is_one_launch_per_batch(hip, batch, m, n, k):
    """mh_f16_matmul_nk_batched against the oracle's dense product matrix by matrix, and bit for bit
    against the same matrices through mh_f16_matmul_nk one by one."""
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(batch * 1000 + m)
    a = rng.normal(0, 1, size=(batch, m, k)).astype(np.float16)
    b = rng.normal(0, 0.2, size=(batch, n, k)).astype(np.float16)
    da, db = _t(a), _t(b)
    out = HIPTensor.allocate((batch, m, n), "float16")
    hip.call("mh_f16_matmul_nk_batched", None, da.data_ptr, db.data_ptr, out.data_ptr, batch, m, n, k)
    got = out.numpy()
    one = HIPTensor.allocate((m, n), "float16")
    for i in range(batch):
        ref = OG.dense_matmul(a[i], np.ascontiguousarray(b[i].T))
        assert_fp16_close(got[i], ref.astype(np.float64), what=f"batched nk, matrix {i}")
        if k % 32 == 0:   # same kernel, same tiling: same bits
            hip.call("mh_f16_matmul_nk", None, da.data_ptr + i * m * k * 2, db.data_ptr + i * n * k * 2,
                     one.data_ptr, m, n, k)
            np.testing.assert_array_equal(one.numpy().view(np.uint16), got[i].view(np.uint16))
