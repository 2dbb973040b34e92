from .memory import Event, HIPMemory, synchronize
from .tensor import HIPTensor
from . import dispatch  # registers the HIP implementations
