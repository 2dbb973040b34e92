from .linalg import matrix_multiply
from .reduce import max, mean, sum
from .arith import multiply
from .special import rms_norm, rope, sigmoid, softmax
