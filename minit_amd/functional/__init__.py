from .linalg import matrix_multiply
from .reduce import max, mean, sum
from .special import rms_norm, rope, softmax
