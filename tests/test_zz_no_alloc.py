"""mh_gptq_matmul_static -- the quantized product for callers that cannot
allocate -- against mh_gptq_matmul with a caller-owned workspace: same kernels,
same plan, so the fp16 outputs must agree bit for bit, on calls in a row that
share the library's one scratch buffer (the later ones smaller than the first),
and against the oracle within the tolerance of the product."""
import numpy as np
import pytest

from helpers import assert_fp16_close
from oracle import cport

pytestmark = pytest.mark.gpu

GROUP, BITS = 128, 4


def _run_both(hip, m, k, n, seed):
    from minit_amd import synthetic
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    qw, qz, sc = synthetic.gptq_weights("noalloc", f"w{seed}", k, n, GROUP, BITS)
    x = synthetic.activations("noalloc", f"x{seed}", (m, k))
    dx, dqw, dqz, dsc = (HIPTensor.from_numpy(t) for t in (x, qw, qz, sc))
    need = hip.call("mh_gptq_workspace_bytes", m, n, k, GROUP, BITS)
    print(f"[no-alloc] M={m} K={k} N={n}: split-K scratch {need} bytes", flush=True)
    assert need <= hip.call("mh_gptq_static_scratch_bytes")
    want = HIPTensor.allocate((m, n), "float16")
    ws = memory.HIPMemory(max(need, 256))
    ws.reset()
    hip.call("mh_gptq_matmul", None, dx.data_ptr, dqw.data_ptr, dqz.data_ptr, dsc.data_ptr, None, want.data_ptr,
             m, n, k, GROUP, BITS, ws._pointer, ws._size)
    got = HIPTensor.allocate((m, n), "float16")
    got._memory.reset()
    hip.call("mh_gptq_matmul_static", None, dx.data_ptr, dqw.data_ptr, dqz.data_ptr, dsc.data_ptr, None,
             got.data_ptr, m, n, k, GROUP, BITS)
    return got.numpy(), want.numpy(), (x, qw, qz, sc)


def test_static_scratch_matches_caller_workspace_on_calls_in_a_row(hip):
    # a cut plan with partial sums across workgroups, then smaller and differently planned products, then
    # the first shape again: every call finds what the one before left in the buffer
    for seed, (m, k, n) in enumerate([(8, 8192, 10240), (1, 4096, 4096), (32, 2048, 3072), (3, 1024, 512),
                                      (8, 8192, 10240)]):
        got, want, (x, qw, qz, sc) = _run_both(hip, m, k, n, seed)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), f"M={m} K={k} N={n}: outputs differ"
        if k * n <= 4096 * 4096:
            ref = cport.matmul(x, qw, qz, sc, None, BITS, GROUP)
            assert_fp16_close(got, ref.astype(np.float64), what=f"static M={m} K={k} N={n}")


def test_static_scratch_rejects_what_does_not_fit(hip):
    from minit_amd.hip.tensor import HIPTensor
    limit = hip.call("mh_gptq_static_scratch_bytes")
    assert limit == 24 << 20
    # a product whose split-K partial sums exceed the built-in buffer (the plan depends on the CU count and
    # on the kernel: 8-bit weights at 64 rows run as one block of 64 rows with K split over workgroups)
    shapes = [(64, 8192, 57344, 8), (48, 16384, 57344, 8), (64, 8192, 57344, 4), (32, 8192, 57344, 4)]
    needs = [hip.call("mh_gptq_workspace_bytes", m, n, k, GROUP, bits) for m, k, n, bits in shapes]
    assert max(needs) > limit, f"no shape exceeds the built-in buffer: {needs}"
    (m, k, n, bits), need = max(zip(shapes, needs), key=lambda t: t[1])
    dummy = HIPTensor.allocate((16,), "float16")     # never dereferenced: the size check comes first
    with pytest.raises(hip.HipError, match="scratch"):
        hip.call("mh_gptq_matmul_static", None, dummy.data_ptr, dummy.data_ptr, dummy.data_ptr, dummy.data_ptr, None,
                 dummy.data_ptr, m, n, k, GROUP, bits)
