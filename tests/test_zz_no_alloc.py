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
    # Up to 32 rows the workspace always holds the arrival counters and at least one fp32 copy of the
    # output (epilogues go through it even when K is not split), whatever plan the CU count gives: 32 rows
    # of 262144 columns are 32 MiB of partial sums.  The rows are searched downwards so that the test
    # follows the limit if it is ever raised.
    k, n, bits = 128, 262144, 4
    m = next(r for r in (32, 24, 16, 8) if hip.call("mh_gptq_workspace_bytes", r, n, k, GROUP, bits) > limit)
    need = hip.call("mh_gptq_workspace_bytes", m, n, k, GROUP, bits)
    assert need >= m * n * 4 > limit
    dummy = HIPTensor.allocate((16,), "float16")     # never dereferenced: the size check comes first
    with pytest.raises(hip.HipError, match="scratch"):
        hip.call("mh_gptq_matmul_static", None, dummy.data_ptr, dummy.data_ptr, dummy.data_ptr, dummy.data_ptr, None,
                 dummy.data_ptr, m, n, k, GROUP, bits)


def test_static_entry_recorded_into_a_graph_replays_like_the_eager_call(hip):
    """One mh_gptq_matmul_static call captured into a HIP graph (after an eager first call, which
    looks up the built-in buffer) and replayed three times with other eager calls on the same buffer
    in between: every replay returns the eager call's bits.  The recorded launches carry no memset
    node: the counters are cleared by a kernel."""
    import ctypes
    from minit_amd import synthetic
    from minit_amd.hip import memory
    from minit_amd.hip.tensor import HIPTensor
    rt = ctypes.CDLL("libamdhip64.so")
    m, k, n = 8, 8192, 10240
    qw, qz, sc = synthetic.gptq_weights("noalloc", "wg", k, n, GROUP, BITS)
    x = synthetic.activations("noalloc", "xg", (m, k))
    dx, dqw, dqz, dsc = (HIPTensor.from_numpy(t) for t in (x, qw, qz, sc))
    out = HIPTensor.allocate((m, n), "float16")

    def call(stream):
        hip.call("mh_gptq_matmul_static", stream, dx.data_ptr, dqw.data_ptr, dqz.data_ptr, dsc.data_ptr, None,
                 out.data_ptr, m, n, k, GROUP, BITS)

    call(None)
    memory.synchronize()
    want = out.numpy().copy()
    stream = ctypes.c_void_p()
    hip.call("mh_stream_create", ctypes.byref(stream))
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.hipStreamBeginCapture(stream, 0) == 0
    call(stream)
    assert rt.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert rt.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    try:
        for replay in range(3):
            out._memory.reset()
            memory.synchronize()
            assert rt.hipGraphLaunch(graph_exec, stream) == 0
            hip.call("mh_stream_synchronize", stream)
            assert np.array_equal(out.numpy().view(np.uint16), want.view(np.uint16)), f"replay {replay} differs"
            # eager work of another shape on the same built-in buffer between the replays
            got, ref, _ = _run_both(hip, 3 + replay, 1024, 512, 40 + replay)
            assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    finally:
        rt.hipGraphExecDestroy(graph_exec)
        rt.hipGraphDestroy(graph)
        hip.call("mh_stream_destroy", stream)
