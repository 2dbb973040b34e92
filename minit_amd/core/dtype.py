"""dtype registry; names and sizes as in the reference (minit/core/dtype.py:36-49)."""
from typing import Dict, Optional


class DataTypeInfo:
    __slots__ = ["name", "python_type", "size_in_bytes"]

    def __init__(self, name: str, python_type: Optional[type], size_in_bytes: int) -> None:
        self.name = name
        self.python_type = python_type
        self.size_in_bytes = size_in_bytes


DATA_TYPES: Dict[str, DataTypeInfo] = {}


def register_dtype(name: str, python_type: Optional[type], size_in_bytes: int):
    assert name not in DATA_TYPES
    DATA_TYPES[name] = DataTypeInfo(name, python_type, size_in_bytes)


def dtype_info(name: str) -> DataTypeInfo:
    return DATA_TYPES[name]


for _name, _py, _size in [
    ("float64", float, 8), ("float32", float, 4), ("float16", float, 2), ("bfloat16", float, 2),
    ("int64", int, 8), ("int32", int, 4), ("int16", int, 2), ("int8", int, 1),
    ("uint64", int, 8), ("uint32", int, 4), ("uint16", int, 2), ("uint8", int, 1),
]:
    register_dtype(_name, _py, _size)
