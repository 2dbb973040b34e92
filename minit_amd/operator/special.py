from . import RMSNorm, RoPE, Sigmoid, Softmax  # noqa: F401
