"""dtype registry: the reference's names with their python type and size
(minit/core/dtype.py:36-49)."""
from typing import Dict, NamedTuple, Optional


class DataTypeInfo(NamedTuple):
    name: str
    python_type: Optional[type]
    size_in_bytes: int


DATA_TYPES: Dict[str, DataTypeInfo] = {}


def register_dtype(name: str, python_type: Optional[type], size_in_bytes: int) -> None:
    if name in DATA_TYPES:
        raise AssertionError(f"dtype {name} is registered already")
    DATA_TYPES[name] = DataTypeInfo(name, python_type, size_in_bytes)


def dtype_info(name: str) -> DataTypeInfo:
    return DATA_TYPES[name]


def _register_builtin() -> None:
    # floating types by bit width (bfloat16 shares float16's size), then the integers of 8 to 64 bits
    for bits in (64, 32, 16):
        register_dtype(f"float{bits}", float, bits // 8)
    register_dtype("bfloat16", float, 2)
    for prefix in ("int", "uint"):
        for bits in (64, 32, 16, 8):
            register_dtype(f"{prefix}{bits}", int, bits // 8)


_register_builtin()
