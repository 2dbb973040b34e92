"""ctypes binding of ``libminit_hip.so`` (the C ABI declared in include/minit_hip.h).

The reference binds each generated launcher with ``import_symbol``, which reads
ctypes argument types from a stub's annotations (minit/compiler/cxx.py:39-59).
Here the prototypes are listed once, every function returns an ``int`` status,
and a non-zero status raises :class:`HipError` carrying ``mh_last_error()``.
There is no fallback: if the library is missing, loading raises.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MINIT_HIP_LIB") or os.path.join(_HERE, "libminit_hip.so")


class HipError(RuntimeError):
    pass


_P = c_void_p
PROTOTYPES = {
    # name: (restype, argtypes)
    "mh_abi_version": (c_int, []),
    "mh_last_error": (c_char_p, []),
    "mh_device_count": (c_int, [POINTER(c_int)]),
    "mh_device_info": (c_int, [POINTER(c_int), POINTER(c_int), POINTER(c_size_t), POINTER(c_size_t),
                               POINTER(c_int), c_char_p, c_size_t]),
    "mh_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "mh_free": (c_int, [_P]),
    "mh_host_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "mh_host_free": (c_int, [_P]),
    "mh_memcpy": (c_int, [_P, _P, c_size_t, _P]),
    "mh_memset": (c_int, [_P, c_int, c_size_t, _P]),
    "mh_stream_create": (c_int, [POINTER(c_void_p)]),
    "mh_stream_destroy": (c_int, [_P]),
    "mh_stream_synchronize": (c_int, [_P]),
    "mh_device_synchronize": (c_int, []),
    "mh_event_create": (c_int, [POINTER(c_void_p)]),
    "mh_event_destroy": (c_int, [_P]),
    "mh_event_record": (c_int, [_P, _P]),
    "mh_event_synchronize": (c_int, [_P]),
    "mh_event_elapsed_ms": (c_int, [POINTER(c_float), _P, _P]),
    "mh_copy_kernel": (c_int, [_P, _P, _P, c_size_t]),
    "mh_gptq_unpack": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_int, c_int]),
    "mh_gptq_dequant": (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int]),
    "mh_gptq_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "mh_gptq_gemv": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_gptq_gemm": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_gptq_matmul": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_gptq_linear": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_gptq_static_scratch_bytes": (c_size_t, []),
    "mh_gptq_matmul_static": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int]),
    "mh_gptq_silu_pairs_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "mh_gptq_matmul_silu_pairs": (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_f16_matmul_nk": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int]),
    "mh_f16_matmul_nk_batched": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_int]),
    "mh_i8_gemm": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int]),
    "mh_i8_transpose": (c_int, [_P, _P, _P, c_int, c_int]),
    "mh_gptq_permute_rows": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int]),
    "mh_rms_norm": (c_int, [_P, _P, _P, _P, c_size_t, c_size_t, c_size_t, c_double, c_int]),
    "mh_rope": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_size_t, c_size_t, c_size_t, c_int]),
    "mh_softmax": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_size_t, c_int]),
    "mh_softmax_causal": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_size_t, c_size_t, c_float, c_int]),
    "mh_sum": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_size_t, c_int]),
    "mh_max": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_size_t, c_int]),
    "mh_mean": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_size_t, c_int]),
    "mh_sigmoid": (c_int, [_P, _P, _P, c_size_t, c_int]),
    "mh_gather_columns": (c_int, [_P, _P, _P, _P, c_size_t, c_size_t, c_int]),
    "mh_multiply": (c_int, [_P, _P, _P, _P, c_size_t, c_int]),
    "mh_add": (c_int, [_P, _P, _P, _P, c_size_t, c_int]),
    "mh_silu_mul": (c_int, [_P, _P, _P, _P, c_size_t, c_int, c_int]),
    "mh_add_bias": (c_int, [_P, _P, _P, c_size_t, c_size_t, c_int]),
    "mh_add_rms_norm": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, c_float]),
    "mh_argmax": (c_int, [_P, _P, _P, c_int, c_int]),
    "mh_attn_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "mh_attn_decode": (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, c_size_t]),
    "mh_rope_kv_append": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int]),
    "mh_llama_create": (c_int, [POINTER(c_void_p), _P]),
    "mh_llama_destroy": (c_int, [_P]),
    "mh_llama_set_layer": (c_int, [_P, c_int, _P]),
    "mh_llama_set_globals": (c_int, [_P, _P, _P, _P, _P, _P]),
    "mh_llama_scratch_bytes": (c_size_t, [_P, c_int]),
    "mh_llama_norm_clamped": (c_int, [_P, _P, c_int, _P, POINTER(c_int)]),
    "mh_llama_decode": (c_int, [_P, _P, c_int, _P, _P, c_int, _P, _P, _P, c_size_t]),
    "mh_llama_decode_graph": (c_int, [_P, _P, c_int, _P, _P, c_int, _P, _P, _P, c_size_t]),
    "mh_synth_u32": (c_int, [_P, _P, c_size_t, c_uint64]),
    "mh_synth_subwords": (c_int, [_P, _P, c_size_t, c_int, c_uint32, c_uint32, c_uint64]),
    "mh_synth_normal": (c_int, [_P, _P, c_size_t, c_float, c_float, c_int, c_float, c_uint64, c_int]),
    "mh_synth_i8": (c_int, [_P, _P, c_size_t, c_int, c_int, c_uint64]),
}

# functions whose return value is not a status code
_NOT_STATUS = {"mh_abi_version", "mh_last_error", "mh_gptq_workspace_bytes", "mh_gptq_static_scratch_bytes", "mh_gptq_silu_pairs_workspace_bytes", "mh_llama_scratch_bytes",
               "mh_attn_decode_workspace_bytes"}

DTYPE_CODES = {"float16": 0, "bfloat16": 1, "float32": 2}

_cdll = None


def cdll() -> ctypes.CDLL:
    """Loads the shared library (once).  Raises if it has not been built."""
    global _cdll
    if _cdll is None:
        if not os.path.exists(LIB_PATH):
            raise HipError(
                f"{LIB_PATH} is missing: build it with `python -m minit_amd.build` "
                "(there is no CPU fallback for this path)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _cdll = lib
    return _cdll


def last_error() -> str:
    return cdll().mh_last_error().decode(errors="replace")


def call(name: str, *args):
    """Calls ``name`` and raises :class:`HipError` on a non-zero status."""
    fn = getattr(cdll(), name)
    rc = fn(*args)
    if name in _NOT_STATUS:
        return rc
    if rc != 0:
        raise HipError(f"{name} failed ({rc}): {last_error()}")
    return rc


def device_count() -> int:
    n = c_int(0)
    try:
        call("mh_device_count", ctypes.byref(n))
    except HipError:
        return 0
    return n.value


def device_info() -> dict:
    cus, wave, clock = c_int(0), c_int(0), c_int(0)
    mem, lds = c_size_t(0), c_size_t(0)
    name = ctypes.create_string_buffer(256)
    call("mh_device_info", ctypes.byref(cus), ctypes.byref(wave), ctypes.byref(mem), ctypes.byref(lds),
         ctypes.byref(clock), name, 256)
    return {"name": name.value.decode(), "compute_units": cus.value, "wavefront": wave.value,
            "total_mem": mem.value, "lds_per_block": lds.value, "clock_khz": clock.value}
