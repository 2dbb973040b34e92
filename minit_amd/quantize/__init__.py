from .functional import dequantize
from .operator import Dequantize
from .tensor import QuantizedTensor
