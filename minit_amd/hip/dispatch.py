"""HIPTensor implementations of the hot-path operators, registered into the
multimethod table.  Each rule does what the reference's CUDATensor rule does --
collapse the shape to ``[a, b, c]``, allocate the output, call one ``extern "C"``
launcher on the null stream (minit/cuda/dispatch.py:59-78,152-173,430-478) --
against the HIP library.
"""
from ..core.dispatch import register_dispatch
from ..core.tensor import Tensor
from ..lib import DTYPE_CODES, call
from ..operator import Add, BatchMatrixMultiply, MatrixMultiply, Max, Mean, Multiply, RMSNorm, RoPE, Sigmoid, Softmax, Sum
from ..quantize.operator import Dequantize
from ..quantize.tensor import QuantizedTensor, _NoGroup
from . import memory
from .tensor import HIPTensor


def _abc(shape, axis):
    a = b = c = 1
    for dim in shape[:axis]:
        a *= dim
    b = shape[axis]
    for dim in shape[axis + 1:]:
        c *= dim
    return a, b, c


def _count(shape) -> int:
    n = 1
    for dim in shape:
        n *= dim
    return n


def _code(dtype: str) -> int:
    assert dtype in DTYPE_CODES, f"unsupported dtype {dtype}"
    return DTYPE_CODES[dtype]


# The generic (MatrixMultiply, Tensor, QuantizedTensor) rule of the reference
# sits at priority 0 (minit/quantize/dispatch.py:8-11); the fused rule outranks it.
@register_dispatch(priority=1)
def dispatch_quantized_matmul(op: MatrixMultiply, a: HIPTensor, b: QuantizedTensor):
    m, k = a._shape
    assert k == b.in_features, f"x has K={k}, weight has K={b.in_features}"
    assert a.dtype == "float16" and b._scale.dtype == a.dtype
    n = b.out_features
    out = HIPTensor.allocate((m, n), a.dtype)
    if m == 0:
        return (out,)
    nbytes = call("mh_gptq_workspace_bytes", m, n, k, b.group_size, b.bits)
    ws = memory.workspace(max(nbytes, 256))
    g_idx = None if b._group is None else b._group.data_ptr
    call("mh_gptq_matmul", None, a.data_ptr, b._data.data_ptr, b._zero.data_ptr, b._scale.data_ptr, g_idx,
         out.data_ptr, m, n, k, b.group_size, b.bits, ws._pointer, ws._size)
    return (out,)


@register_dispatch()
def dispatch_dequantize(op: Dequantize, data: HIPTensor, group: Tensor, zero: HIPTensor, scale: HIPTensor):
    assert op.axis == 0, "GPTQ weights are grouped along K (axis 0)"
    rows, n = data._shape
    groups, packed_n = zero._shape
    per_word = n // packed_n
    bits = 32 // per_word
    k = rows * per_word
    out = HIPTensor.allocate((k, n), scale.dtype)
    g_idx = None if isinstance(group, _NoGroup) else group.data_ptr
    call("mh_gptq_dequant", None, data.data_ptr, zero.data_ptr, scale.data_ptr, g_idx, out.data_ptr,
         n, k, k // groups, bits)
    return (out,)


@register_dispatch()
def dispatch_matmul(op: MatrixMultiply, a: HIPTensor, b: HIPTensor):
    # dense product with the reference's orientation: b is [N, K]
    m, k0 = a._shape
    n, k1 = b._shape
    assert k0 == k1
    assert a.dtype == b.dtype == "float16"
    c = HIPTensor.allocate((m, n), a.dtype)
    call("mh_f16_matmul_nk", None, a.data_ptr, b.data_ptr, c.data_ptr, m, n, k0)
    return (c,)


@register_dispatch()
def dispatch_batch_matmul(op: BatchMatrixMultiply, a: HIPTensor, b: HIPTensor):
    # minit/cuda/dispatch.py:82-101: c[i] = a[i] @ b[i]^T for i < batch, b stored [batch, N, K];
    # one strided launch for the whole batch, like the reference's library call
    b0, m, k0 = a._shape
    b1, n, k1 = b._shape
    assert b0 == b1
    assert k0 == k1
    assert a.dtype == b.dtype == "float16"
    c = HIPTensor.allocate((b0, m, n), a.dtype)
    for i0 in range(0, b0, 65535):   # the launch takes at most 65535 matrices
        nb = min(65535, b0 - i0)
        call("mh_f16_matmul_nk_batched", None, a.data_ptr + i0 * m * k0 * 2, b.data_ptr + i0 * n * k0 * 2,
             c.data_ptr + i0 * m * n * 2, nb, m, n, k0)
    return (c,)


@register_dispatch()
def register_rms_norm_operator(op: RMSNorm, x: HIPTensor, weight: HIPTensor):
    z = HIPTensor.allocate(x._shape, x.dtype)
    a, b, c = _abc(x._shape, op.axis)
    assert len(weight._shape) == 1
    assert weight._shape[0] == b
    assert weight.dtype == x.dtype
    call("mh_rms_norm", None, x.data_ptr, weight.data_ptr, z.data_ptr, a, b, c, op.eps, _code(x.dtype))
    return (z,)


@register_dispatch()
def register_rope_operator(op: RoPE, x: HIPTensor, freqs_cos: HIPTensor, freqs_sin: HIPTensor,
                           *positions: HIPTensor):
    bs, seqlen, nh, hs = x._shape
    assert freqs_cos.dtype == "float32"
    assert freqs_sin.dtype == "float32"
    assert freqs_cos._shape == freqs_sin._shape and freqs_cos._shape[1] == hs // 2
    pos_ptr = None
    if positions:
        (pos,) = positions
        assert pos.dtype == "int32" and pos._shape == (bs, seqlen)
        pos_ptr = pos.data_ptr
    else:
        assert freqs_cos._shape[0] == seqlen, "tables must be sliced to the sequence"
    z = HIPTensor.allocate(x._shape, x.dtype)
    call("mh_rope", None, x.data_ptr, freqs_cos.data_ptr, freqs_sin.data_ptr, pos_ptr, z.data_ptr,
         bs, seqlen, nh, hs, _code(x.dtype))
    return (z,)


@register_dispatch()
def register_softmax_operator(op: Softmax, x: HIPTensor):
    z = HIPTensor.allocate(x._shape, x.dtype)
    a, b, c = _abc(x._shape, op.axis)
    call("mh_softmax", None, x.data_ptr, z.data_ptr, a, b, c, _code(x.dtype))
    return (z,)


# The two element-wise rules the models' ``silu`` needs (minit/cuda/dispatch.py:104-117
# with the expressions of :137 and :143); operands of one shape and dtype.
@register_dispatch()
def dispatch_sigmoid(op: Sigmoid, x: HIPTensor):
    z = HIPTensor.allocate(x._shape, x.dtype)
    call("mh_sigmoid", None, x.data_ptr, z.data_ptr, _count(x._shape), _code(x.dtype))
    return (z,)


@register_dispatch()
def dispatch_multiply(op: Multiply, x: HIPTensor, y: HIPTensor):
    assert x._shape == y._shape, f"multiply: shapes {x._shape} and {y._shape} differ"
    assert x.dtype == y.dtype
    z = HIPTensor.allocate(x._shape, x.dtype)
    call("mh_multiply", None, x.data_ptr, y.data_ptr, z.data_ptr, _count(x._shape), _code(x.dtype))
    return (z,)


@register_dispatch()
def dispatch_add(op: Add, x: HIPTensor, y: HIPTensor):
    assert x._shape == y._shape, f"add: shapes {x._shape} and {y._shape} differ"
    assert x.dtype == y.dtype
    z = HIPTensor.allocate(x._shape, x.dtype)
    call("mh_add", None, x.data_ptr, y.data_ptr, z.data_ptr, _count(x._shape), _code(x.dtype))
    return (z,)


def _register_reduce(op_type, symbol):
    @register_dispatch()
    def _reduce(op: op_type, x: HIPTensor):  # type: ignore
        z = HIPTensor.allocate(x._shape[:op.axis] + (1,) + x._shape[op.axis + 1:], x.dtype)
        a, b, c = _abc(x._shape, op.axis)
        call(symbol, None, x.data_ptr, z.data_ptr, a, b, c, _code(x.dtype))
        return (z,)


_register_reduce(Sum, "mh_sum")
_register_reduce(Max, "mh_max")
_register_reduce(Mean, "mh_mean")
