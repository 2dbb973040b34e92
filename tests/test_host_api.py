"""Host-side logic that needs no GPU: the multimethod table, the C ABI surface
and the loader."""
import ctypes
import os
import re
from typing import Union

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from minit_amd import lib
    header = open(os.path.join(ROOT, "include", "minit_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(mh_[a-z0-9_]+)\s*\(", header))
    assert len(declared) > 30
    cdll = lib.cdll()                      # loads without a GPU
    for name in sorted(declared):
        assert hasattr(cdll, name), f"{name} is declared in minit_hip.h but not exported"
        assert name in lib.PROTOTYPES, f"{name} has no ctypes prototype"
    assert set(lib.PROTOTYPES) <= declared, set(lib.PROTOTYPES) - declared
    assert cdll.mh_abi_version() == 1


def test_loader_raises_without_the_library(monkeypatch, tmp_path):
    from minit_amd import lib
    monkeypatch.setattr(lib, "_cdll", None)
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(lib.HipError, match="no CPU fallback"):
        lib.cdll()


def test_status_codes_raise_with_message():
    from minit_amd import lib
    with pytest.raises(lib.HipError, match="bits must be 4 or 8"):
        lib.call("mh_gptq_unpack", None, 256, 256, 4, 4, 0, 5)
    with pytest.raises(lib.HipError, match="t=7 must equal"):
        lib.call("mh_softmax_causal", None, 256, 256, 1, 2, 7, 3, 1.0, 0)
    assert lib.call("mh_gptq_workspace_bytes", 1, 4096, 4096, 128, 4) > 0
    assert lib.call("mh_gptq_workspace_bytes", 1, 4096, 4100, 128, 4) == 0   # contract violated


def test_oversized_matrices_are_kept_off_the_mfma_kernels():
    """The MFMA kernels address a matrix's packed weights with 32-bit offsets: 2 GiB and more go to
    the per-element kernel through mh_gptq_matmul, and mh_gptq_gemm says so instead of launching
    (argument checks only: nothing is dereferenced or launched here)."""
    from minit_amd import lib
    k = n = 65536                          # 4-bit: k * n / 2 = 2 GiB exactly
    fake = 4096                            # a non-null pointer value; the size check comes before any use
    with pytest.raises(lib.HipError, match="2 GiB"):
        lib.call("mh_gptq_gemm", None, fake, fake, fake, fake, None, fake, 16, n, k, 128, 4, None, 0)
    # the same matrix just below the limit is accepted by the planner
    assert lib.call("mh_gptq_workspace_bytes", 16, n - 8, k, 128, 4) > 0
    # a plain product of more than 32 rows that is not split along K needs no workspace
    assert lib.call("mh_gptq_workspace_bytes", 2048, 57344, 8192, 128, 4) == 0
    # ... and the split one still does
    assert lib.call("mh_gptq_workspace_bytes", 64, 4096, 14336, 128, 4) > 0


def test_dispatch_rules():
    from minit_amd.core.dispatch import DISPATCH_CACHE, DISPATCH_TABLE, dispatch, register_dispatch
    from minit_amd.core.operator import Operator
    from minit_amd.core.tensor import Tensor

    class Op(Operator):
        pass

    class A(Tensor):
        pass

    class B(A):
        pass

    class C(Tensor):
        pass

    saved = list(DISPATCH_TABLE)
    try:
        @register_dispatch()
        def generic(op: Op, x: Tensor):
            return ("generic",)

        @register_dispatch(priority=1)
        def for_a(op: Op, x: A):
            return ("a",)

        @register_dispatch()
        def union(op: Op, x: Union[A, C], y: Union[A, C]):
            return ("union",)

        @register_dispatch()
        def variadic(op: Op, x: C, y: C, *rest: C):
            return ("variadic", len(rest))

        assert dispatch(Op(), C()) == ("generic",)
        assert dispatch(Op(), A()) == ("a",)          # higher priority wins
        assert dispatch(Op(), B()) == ("a",)          # subclasses match
        assert dispatch(Op(), A(), C()) == ("union",)
        assert dispatch(Op(), C(), C(), C(), C()) == ("variadic", 2)
        with pytest.raises(AssertionError, match="more than one"):
            dispatch(Op(), C(), C())                   # union and variadic tie
        with pytest.raises(AssertionError, match="no matching"):
            dispatch(Op(), A(), A(), A())

        @register_dispatch(predicate=lambda *tys: False, priority=5)
        def never(op: Op, x: Tensor):
            return ("never",)

        assert dispatch(Op(), C()) == ("generic",)
    finally:
        DISPATCH_TABLE[:] = saved
        DISPATCH_CACHE.clear()


def test_quantized_rule_outranks_the_generic_one():
    """(MatrixMultiply, HIPTensor, QuantizedTensor) must resolve to the fused
    rule, registered above priority 0."""
    import minit_amd  # noqa: F401
    from minit_amd.core.dispatch import lookup_implementation_from_types
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.operator import MatrixMultiply, RMSNorm, RoPE, Softmax, Sum
    from minit_amd.quantize.tensor import QuantizedTensor
    fn = lookup_implementation_from_types((MatrixMultiply, HIPTensor, QuantizedTensor))
    assert fn.__name__ == "dispatch_quantized_matmul"
    assert lookup_implementation_from_types((MatrixMultiply, HIPTensor, HIPTensor)).__name__ == "dispatch_matmul"
    for tys in [(RMSNorm, HIPTensor, HIPTensor), (RoPE, HIPTensor, HIPTensor, HIPTensor),
                (RoPE, HIPTensor, HIPTensor, HIPTensor, HIPTensor), (Softmax, HIPTensor), (Sum, HIPTensor)]:
        assert lookup_implementation_from_types(tys) is not None


def test_functional_argument_checks():
    import minit_amd.functional as F
    with pytest.raises(AssertionError):
        F.rms_norm(None, None, 0, 1)         # eps must be a float, as in the reference
    with pytest.raises(AssertionError):
        F.rms_norm(None, None, 0, 0.75)


def test_interleave_gate_up_moves_whole_columns():
    """The load-time column order of the fused gate|up projection: blocks of 128
    gate columns followed by their 128 up columns; dequantizing after the
    permutation equals permuting the dequantized matrix."""
    import numpy as np
    from minit_amd import synthetic
    from minit_amd.decode import interleave_gate_up
    from oracle import gptq as O
    k, ffn, g = 256, 384, 128
    qweight, qzeros, scales = synthetic.gptq_weights("host", "gu", k, 2 * ffn, g, 4, (0, 15))
    w = O.dequantize_packed(qweight, qzeros, scales, None, 4, g)
    wi = O.dequantize_packed(*interleave_gate_up(qweight, qzeros, scales), None, 4, g)
    for t in range(ffn // 128):
        np.testing.assert_array_equal(wi[:, t * 256:t * 256 + 128], w[:, t * 128:(t + 1) * 128])
        np.testing.assert_array_equal(wi[:, t * 256 + 128:(t + 1) * 256], w[:, ffn + t * 128:ffn + (t + 1) * 128])


def test_v_cache_tiling_follows_the_kernels_offset_rule():
    """tile_v_cache puts value d of position p at ((p // 64) * D + d) * 64 + p % 64 of its row and
    KV head (vt_offset in csrc/gptq_common.h), and untile_v_cache is its inverse."""
    import numpy as np
    from minit_amd.decode import tile_v_cache, untile_v_cache
    b, h, t, d = 2, 3, 192, 128
    v = np.arange(b * h * t * d, dtype=np.int64).reshape(b, h, t, d).astype(np.float32)
    tiled = tile_v_cache(v)
    assert tiled.shape == (b, h, t // 64, d, 64) and tiled.flags["C_CONTIGUOUS"]
    flat = tiled.reshape(b, h, -1)
    for p, dim in ((0, 0), (1, 0), (63, 127), (64, 5), (130, 77), (191, 127)):
        np.testing.assert_array_equal(flat[:, :, ((p // 64) * d + dim) * 64 + p % 64], v[:, :, p, dim])
    np.testing.assert_array_equal(untile_v_cache(tiled), v)
    import pytest
    with pytest.raises(AssertionError):
        tile_v_cache(v[:, :, :100])


def test_prototypes_match_header_argument_counts():
    """ctypes converts surplus arguments by default rules (a pointer becomes a
    truncated int), so a prototype that is one entry short corrupts a call
    silently: every prototype must list exactly the header's parameters."""
    import os
    import re
    from minit_amd import lib
    header = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include",
                               "minit_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    decls = dict(re.findall(r"\b(mh_\w+)\s*\(([^;{]*?)\)\s*;", header))
    assert decls, "no declarations parsed"
    for name, (_, argtypes) in lib.PROTOTYPES.items():
        assert name in decls, f"{name} is not declared in the header"
        params = decls[name].strip()
        n = 0 if params in ("", "void") else len([p for p in params.split(",") if p.strip()])
        assert n == len(argtypes), f"{name}: header has {n} parameters, prototype lists {len(argtypes)}"
    for name in decls:
        assert name in lib.PROTOTYPES, f"{name} has no ctypes prototype"


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N above 1 exits with a message that says so."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                          text=True, timeout=120)
    assert proc.returncode != 0 and "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_shared_workspace_refuses_a_second_thread(monkeypatch):
    """memory.workspace() is one buffer for every split-K launch of the null stream: a second host
    thread would race on its arrival counters and partial sums, so it is refused."""
    import threading
    from minit_amd import lib
    from minit_amd.hip import memory
    monkeypatch.setattr(memory, "_OWNER_THREAD", threading.get_ident())
    memory._single_thread("here")                      # the owner passes
    seen = []

    def other():
        try:
            memory._single_thread("there")
        except lib.HipError as exc:
            seen.append(str(exc))
    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen and "single-threaded" in seen[0]
