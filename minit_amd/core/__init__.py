from .dispatch import dispatch, register_dispatch
from .dtype import dtype_info
from .operator import Operator
from .scalar import ScalarTensor, to_immediate_shape
from .tensor import Tensor
