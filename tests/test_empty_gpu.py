"""GPU: empty inputs through the operator API and the C ABI.  A product with no
rows, a row-wise operator over no rows and a reduction over an empty axis return
without touching memory beyond their (possibly empty) outputs; the reduction of
an empty axis yields the reference's initial values (0 for sum, -inf for max,
minit/cuda/kernel/cuda/reduce.py:76-92)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _t(arr):
    from minit_amd.hip.tensor import HIPTensor
    return HIPTensor.from_numpy(np.ascontiguousarray(arr))


def test_products_with_no_rows(hip):
    import minit_amd.functional as F
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import quantized_tensor_from_host
    qweight, qzeros, scales, *_ = synthetic.gptq_weights("empty", "w", 256, 64, 128, 4)
    weight = quantized_tensor_from_host(qweight, qzeros, scales)
    x = HIPTensor.allocate((0, 256), "float16")
    y = F.matrix_multiply(x, weight)
    assert y._shape == (0, 64) and y.numpy().shape == (0, 64)
    dense = _t(np.ones((8, 256), np.float16))
    assert F.matrix_multiply(x, dense).numpy().shape == (0, 8)

    # C ABI: M = 0 is accepted with null activation / output pointers and leaves a guard untouched
    guard = _t(np.full((4, 64), 7, np.float16))
    ws = HIPTensor.allocate((1024,), "int8")
    for entry in ("mh_gptq_matmul", "mh_gptq_gemm", "mh_gptq_gemv"):
        hip.call(entry, None, None, weight._data.data_ptr, weight._zero.data_ptr, weight._scale.data_ptr, None,
                 None, 0, 64, 256, 128, 4, ws.data_ptr, 1024)
    a = HIPTensor.allocate((0, 128), "int8")
    w = _t(np.ones((64, 128), np.int8))
    sa, sw = HIPTensor.allocate((0,), "float32"), _t(np.ones(64, np.float32))
    hip.call("mh_i8_gemm", None, a.data_ptr, w.data_ptr, sa.data_ptr, sw.data_ptr, guard.data_ptr, None, 0, 64, 128)
    assert (guard.numpy() == 7).all()


def test_rowwise_operators_over_nothing(hip):
    import minit_amd.functional as F
    from minit_amd.hip.tensor import HIPTensor
    x = HIPTensor.allocate((0, 128), "float16")
    w = _t(np.ones(128, np.float16))
    assert F.rms_norm(x, w, 1, 1e-6).numpy().shape == (0, 128)
    assert F.softmax(x, 1).numpy().shape == (0, 128)
    assert F.sum(x, 1).numpy().shape == (0, 1)
    # an empty reduced axis leaves the initial values
    e = HIPTensor.allocate((3, 0, 2), "float16")
    s, m = F.sum(e, 1).numpy(), F.max(e, 1).numpy()
    assert s.shape == m.shape == (3, 1, 2)
    assert (s == 0).all() and np.isneginf(m).all()
    cos, sin = _t(np.ones((4, 64), np.float32)), _t(np.zeros((4, 64), np.float32))
    q = HIPTensor.allocate((0, 4, 2, 128), "float16")
    assert F.rope(q, cos, sin).numpy().shape == (0, 4, 2, 128)
