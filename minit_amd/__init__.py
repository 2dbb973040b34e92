"""MI355X-native quantized-linear hot path behind MiniT's operator API.

``import minit_amd`` registers the HIP implementations; it needs the built
``libminit_hip.so`` only when an operator actually runs.
"""
from . import functional  # noqa: F401
from .core import Tensor, dispatch, register_dispatch  # noqa: F401
from .hip import HIPTensor  # noqa: F401
from .quantize import QuantizedTensor, dequantize  # noqa: F401
