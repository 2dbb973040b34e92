"""Device tensor with the surface of the reference's ``CUDATensor``
(minit/cuda/tensor.py:15-131): contiguous row-major, ``_shape`` / ``_dtype`` /
``_memory``, ``allocate`` / ``wrap`` / ``from_numpy`` / ``from_item`` /
``copy_from_numpy`` / ``numpy`` / ``item`` / ``data_ptr``; ``shape`` is a tuple
of scalar tensors and ``type()`` is the class itself.
"""
from numbers import Number
from typing import Optional, Tuple

import numpy

from ..core.dtype import dtype_info
from ..core.scalar import ScalarTensor
from ..core.tensor import Tensor
from . import memory
from .memory import HIPMemory

_NUMPY_DTYPES = {
    "float64": numpy.float64, "float32": numpy.float32, "float16": numpy.float16,
    "bfloat16": numpy.uint16,  # raw bits; numpy has no bfloat16
    "int64": numpy.int64, "int32": numpy.int32, "int16": numpy.int16, "int8": numpy.int8,
    "uint64": numpy.uint64, "uint32": numpy.uint32, "uint16": numpy.uint16, "uint8": numpy.uint8,
}


def _nbytes(shape: Tuple[int, ...], dtype: str) -> int:
    size = dtype_info(dtype).size_in_bytes
    for dim in shape:
        assert isinstance(dim, int), f"shape entries must be int, got {type(dim)}"
        size *= dim
    return size


class HIPTensor(Tensor):
    __slots__ = ["_memory", "_shape", "_item", "_dtype"]

    def __init__(self, shape: Tuple[int, ...], dtype: str) -> None:
        self._memory: Optional[HIPMemory] = None
        self._item: Optional[Number] = None
        self._shape = tuple(shape)
        self._dtype = dtype

    @property
    def shape(self) -> Tuple[Tensor, ...]:
        return tuple(ScalarTensor(dim, (), "int32") for dim in self._shape)

    @property
    def dtype(self) -> str:
        return self._dtype

    @property
    def device(self) -> str:
        return "hip"

    @property
    def memory(self) -> HIPMemory:
        if self._memory is None and self._item is not None:
            self._memory = HIPMemory(dtype_info(self.dtype).size_in_bytes)
            self.copy_from_numpy(numpy.full((), self._item, _NUMPY_DTYPES[self.dtype]))
        return self._memory

    @property
    def data_ptr(self) -> int:
        return self.memory._pointer

    @staticmethod
    def allocate(shape: Tuple[int, ...], dtype: str) -> "HIPTensor":
        result = HIPTensor(tuple(shape), dtype)
        result._memory = HIPMemory(_nbytes(tuple(shape), dtype))
        return result

    @staticmethod
    def wrap(shape: Tuple[int, ...], dtype: str, memory: HIPMemory) -> "HIPTensor":
        assert memory._size == _nbytes(tuple(shape), dtype), "wrap: size mismatch"
        result = HIPTensor(tuple(shape), dtype)
        result._memory = memory
        return result

    @staticmethod
    def from_pointer(shape: Tuple[int, ...], dtype: str, pointer: int, owner) -> "HIPTensor":
        """Zero-copy view of device memory owned by ``owner`` (e.g. a torch tensor)."""
        result = HIPTensor(tuple(shape), dtype)
        result._memory = HIPMemory(_nbytes(tuple(shape), dtype), pointer=pointer, owner=owner)
        return result

    @staticmethod
    def from_torch(tensor) -> "HIPTensor":
        """Wraps a contiguous torch tensor on the GPU without copying."""
        assert tensor.is_cuda and tensor.is_contiguous()
        dtype = str(tensor.dtype).split(".")[-1]
        return HIPTensor.from_pointer(tuple(tensor.shape), dtype, tensor.data_ptr(), tensor)

    @staticmethod
    def from_numpy(array) -> "HIPTensor":
        dtype = str(array.dtype).split(".")[-1]
        device_array = HIPTensor.allocate(tuple(array.shape), dtype)
        device_array.copy_from_numpy(array)
        return device_array

    @staticmethod
    def from_item(item: Number, dtype: str) -> "HIPTensor":
        result = HIPTensor((), dtype)
        result._item = item
        return result

    def copy_from_numpy(self, array) -> None:
        assert tuple(array.shape) == self._shape, f"{tuple(array.shape)} vs {self._shape}"
        if type(array).__module__.startswith("torch"):
            if not array.is_cpu:
                array = array.cpu()
            array = array.contiguous()
            pointer = array.data_ptr()
        else:
            array = numpy.ascontiguousarray(array)
            pointer = array.__array_interface__["data"][0]
        dtype = str(array.dtype).split(".")[-1]
        if self.dtype == "bfloat16" and dtype == "uint16":
            dtype = "bfloat16"
        assert dtype == self.dtype, f"{dtype} vs {self.dtype}"
        size = _nbytes(self._shape, self.dtype)
        memory.synchronize()
        memory.copy(self.data_ptr, pointer, size)
        memory.synchronize()  # the host buffer may be a temporary

    def numpy(self) -> numpy.ndarray:
        host = numpy.zeros(self._shape, _NUMPY_DTYPES[self.dtype])
        size = _nbytes(self._shape, self.dtype)
        if size:
            memory.copy(host.__array_interface__["data"][0], self.data_ptr, size)
        memory.synchronize()
        return host

    def item(self):
        if self._item is not None:
            return dtype_info(self.dtype).python_type(self._item)
        return self.numpy().item()

    def reshape(self, shape: Tuple[int, ...]) -> "HIPTensor":
        """A re-``wrap`` of the same memory (the reference's fold / expand)."""
        return HIPTensor.wrap(tuple(shape), self.dtype, self.memory)

    def type(self):
        return HIPTensor
