from .linalg import batch_matrix_multiply, matrix_multiply
from .reduce import max, mean, sum
from .arith import add, multiply
from .special import rms_norm, rope, sigmoid, softmax
