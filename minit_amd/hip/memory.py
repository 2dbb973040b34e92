"""Device memory, streams and events over the C ABI.

``HIPMemory`` mirrors the reference's ``CUDAMemory`` (minit/cuda/allocator.py:
85-117: pointer + size, freed in ``__del__``, ``copy_from`` / ``copy`` /
``reset``).  The reference draws from ``cudaMallocAsync``'s pool; here freed
blocks go to a small size-keyed free list so a steady-state loop does not call
``hipMalloc`` / ``hipFree`` (which synchronises the device) per tensor.
"""
import ctypes
import threading
from typing import Dict, List

from .. import lib

_POOL: Dict[int, List[int]] = {}
_POOL_BYTES = 0
_POOL_LIMIT = 4 << 30


def _round(size: int) -> int:
    return max(256, (size + 255) // 256 * 256)


def allocate(size: int) -> int:
    global _POOL_BYTES
    size = _round(size)
    bucket = _POOL.get(size)
    if bucket:
        _POOL_BYTES -= size
        return bucket.pop()
    ptr = ctypes.c_void_p()
    try:
        lib.call("mh_malloc", ctypes.byref(ptr), size)
    except lib.HipError:
        empty_cache()
        lib.call("mh_malloc", ctypes.byref(ptr), size)
    return ptr.value


def release(ptr: int, size: int) -> None:
    global _POOL_BYTES
    size = _round(size)
    if _POOL_BYTES + size <= _POOL_LIMIT:
        _POOL.setdefault(size, []).append(ptr)
        _POOL_BYTES += size
    else:
        lib.call("mh_free", ptr)


def empty_cache() -> None:
    global _POOL_BYTES
    for bucket in _POOL.values():
        for ptr in bucket:
            lib.call("mh_free", ptr)
    _POOL.clear()
    _POOL_BYTES = 0


def synchronize(stream=None) -> None:
    """``sync_cuda`` of the reference (allocator.py:44-46)."""
    if stream is None:
        lib.call("mh_device_synchronize")
    else:
        lib.call("mh_stream_synchronize", stream)


def copy(dst: int, src: int, size: int, stream=None) -> None:
    lib.call("mh_memcpy", dst, src, size, stream)


class HIPMemory:
    __slots__ = ["_pointer", "_size", "_owner"]

    def __init__(self, size: int, pointer: int = None, owner=None) -> None:
        """Allocates ``size`` bytes, or wraps ``pointer`` kept alive by ``owner``."""
        self._size = size
        self._owner = owner
        self._pointer = allocate(size) if pointer is None else pointer

    def __del__(self):
        try:
            if self._owner is None and self._pointer is not None:
                release(self._pointer, self._size)
        except Exception:
            pass
        self._pointer = None

    def copy_from(self, src: "HIPMemory"):
        assert self._size == src._size
        copy(self._pointer, src._pointer, self._size)

    def copy(self) -> "HIPMemory":
        new = HIPMemory(self._size)
        copy(new._pointer, self._pointer, self._size)
        return new

    def reset(self):
        lib.call("mh_memset", self._pointer, 0, self._size, None)


class Event:
    """HIP event for timing work on a given stream."""

    def __init__(self):
        h = ctypes.c_void_p()
        lib.call("mh_event_create", ctypes.byref(h))
        self.handle = h.value

    def record(self, stream=None):
        lib.call("mh_event_record", self.handle, stream)

    def synchronize(self):
        lib.call("mh_event_synchronize", self.handle)

    def elapsed_ms(self, stop: "Event") -> float:
        ms = ctypes.c_float(0)
        lib.call("mh_event_elapsed_ms", ctypes.byref(ms), self.handle, stop.handle)
        return ms.value

    def __del__(self):
        try:
            lib.call("mh_event_destroy", self.handle)
        except Exception:
            pass


def create_stream() -> int:
    h = ctypes.c_void_p()
    lib.call("mh_stream_create", ctypes.byref(h))
    return h.value


_WORKSPACE = None
_OWNER_THREAD = None


def _single_thread(what: str) -> None:
    """The operator API is the reference's: one host thread, every launch on the null stream
    (minit/cuda/dispatch.py passes ``None`` for the stream throughout).  The free list above
    recycles a block as soon as its tensor dies and the workspace below is shared by every
    split-K launch; both are only safe while launches are ordered on one stream by one thread,
    so a second thread is refused instead of silently racing on partial sums."""
    global _OWNER_THREAD
    me = threading.get_ident()
    if _OWNER_THREAD is None:
        _OWNER_THREAD = me
    elif _OWNER_THREAD != me:
        raise lib.HipError(f"{what}: the operator API is single-threaded (null stream); callers with their own "
                           "threads or streams pass their own workspace to the C ABI")


def workspace(nbytes: int) -> HIPMemory:
    """Zero-initialised scratch shared by the split-K kernels of the null stream.

    The kernels leave the part that must be zero (their arrival counters) zeroed,
    so the buffer is cleared only when it is (re)allocated.
    """
    global _WORKSPACE
    _single_thread("memory.workspace")
    if _WORKSPACE is None or _WORKSPACE._size < nbytes:
        size = max(_round(nbytes), 64 << 20)
        synchronize()
        _WORKSPACE = HIPMemory(size)
        _WORKSPACE.reset()
        synchronize()
    return _WORKSPACE
