from .linalg import matrix_multiply
from .reduce import max, mean, sum
from .arith import add, multiply
from .special import rms_norm, rope, sigmoid, softmax
