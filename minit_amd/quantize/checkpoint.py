"""GPTQ checkpoint ingestion: safetensors files to quantized linears on the device.

The reference keeps the four GPTQ buffers of a linear under
``<prefix>.qweight / .qzeros / .scales / .g_idx`` (plus ``.bias``), declares
their shapes from the layer sizes (examples/qwen1_5_int8.py:276-305) and fills
them from safetensors files, one file or an index of several
(minit/module/checkpoint.py:23-44), asserting that every stored shape equals the
declared one.  Here nothing is declared up front: the geometry (bit width,
group size, K, N) is inferred from the stored shapes, which is all a GPTQ
checkpoint fixes, and checked against the shape contract of the reference's
fused product (examples/qwen1_5_int8.py:247-254).  Everything in this module
is host code (numpy); ``quantized_linear`` does the one upload.

Files are read with ``safetensors``, which executes nothing from the file.
"""
import json
import os
from typing import Dict, Iterable, List, Mapping, NamedTuple, Optional

import numpy

GPTQ_SUFFIXES = ("qweight", "qzeros", "scales", "g_idx", "bias")


class GPTQGeometry(NamedTuple):
    bits: int
    group_size: int
    in_features: int
    out_features: int


class GPTQLinearWeights(NamedTuple):
    """Host arrays of one quantized linear; ``g_idx`` is None when groups are sequential."""
    qweight: numpy.ndarray
    qzeros: numpy.ndarray
    scales: numpy.ndarray
    g_idx: Optional[numpy.ndarray]
    bias: Optional[numpy.ndarray]
    geometry: GPTQGeometry


def infer_geometry(qweight_shape, qzeros_shape, scales_shape, g_idx_len: Optional[int] = None) -> GPTQGeometry:
    """Bit width, group size, K and N from the stored shapes.

    ``scales [G, N]`` gives N and G; ``qzeros [G, N * bits / 32]`` gives the bit
    width; ``qweight [K * bits / 32, N]`` then gives K and ``K / G`` the group
    size.  Raises ``ValueError`` where the reference's shape asserts would fail.
    """
    if len(qweight_shape) != 2 or len(qzeros_shape) != 2 or len(scales_shape) != 2:
        raise ValueError("qweight, qzeros and scales must be 2-D")
    groups, n = (int(v) for v in scales_shape)
    zg, zcols = (int(v) for v in qzeros_shape)
    rows, wn = (int(v) for v in qweight_shape)
    if zg != groups:
        raise ValueError(f"qzeros has {zg} groups, scales has {groups}")
    if wn != n:
        raise ValueError(f"qweight has N={wn}, scales has N={n}")
    if zcols == 0 or n % zcols != 0:
        raise ValueError(f"qzeros has {zcols} words per group for N={n}")
    per_word = n // zcols
    if per_word not in (4, 8):
        raise ValueError(f"{per_word} sub-words per 32-bit word: only 4- and 8-bit checkpoints are supported")
    bits = 32 // per_word
    k = rows * per_word
    if groups == 0 or k % groups != 0:
        raise ValueError(f"K={k} is not a whole number of the {groups} groups")
    if g_idx_len is not None and g_idx_len != k:
        raise ValueError(f"g_idx has {g_idx_len} entries for K={k}")
    return GPTQGeometry(bits, k // groups, k, n)


def is_sequential_g_idx(g_idx: numpy.ndarray, group_size: int) -> bool:
    """True when ``g_idx[k] == k // group_size`` (act_order off): the kernels then
    compute the group themselves and the tensor need not travel."""
    g = numpy.asarray(g_idx)
    return bool(numpy.array_equal(g, numpy.arange(g.shape[0], dtype=g.dtype) // group_size))


def linear_prefixes(tensors: Mapping[str, numpy.ndarray]) -> List[str]:
    """Prefixes of all quantized linears of a checkpoint, in name order."""
    return sorted(name[: -len(".qweight")] for name in tensors if name.endswith(".qweight"))


def read_linear(tensors: Mapping[str, numpy.ndarray], prefix: str) -> GPTQLinearWeights:
    """Collects and validates the buffers of ``prefix`` from a name -> array mapping."""
    def get(suffix):
        return tensors.get(f"{prefix}.{suffix}")
    qweight, qzeros, scales = get("qweight"), get("qzeros"), get("scales")
    missing = [s for s, v in (("qweight", qweight), ("qzeros", qzeros), ("scales", scales)) if v is None]
    if missing:
        raise KeyError(f"{prefix}: missing {', '.join(missing)}")
    g_idx, bias = get("g_idx"), get("bias")
    geo = infer_geometry(qweight.shape, qzeros.shape, scales.shape, None if g_idx is None else int(g_idx.shape[0]))
    if qweight.dtype != numpy.int32 or qzeros.dtype != numpy.int32:
        raise ValueError(f"{prefix}: packed tensors must be int32, got {qweight.dtype} / {qzeros.dtype}")
    if bias is not None and tuple(bias.shape) != (geo.out_features,):
        raise ValueError(f"{prefix}: bias has shape {tuple(bias.shape)} for N={geo.out_features}")
    if g_idx is not None:
        g_idx = numpy.ascontiguousarray(g_idx, dtype=numpy.int32)
        if g_idx.min(initial=0) < 0 or g_idx.max(initial=0) >= geo.in_features // geo.group_size:
            raise ValueError(f"{prefix}: g_idx names a group outside [0, {geo.in_features // geo.group_size})")
        if is_sequential_g_idx(g_idx, geo.group_size):
            g_idx = None
    return GPTQLinearWeights(numpy.ascontiguousarray(qweight), numpy.ascontiguousarray(qzeros),
                             numpy.ascontiguousarray(scales, dtype=numpy.float16), g_idx,
                             None if bias is None else numpy.ascontiguousarray(bias, dtype=numpy.float16), geo)


def load_safetensors(paths: Iterable[str]) -> Dict[str, numpy.ndarray]:
    """All tensors of the given files as numpy arrays (later files win on a clash,
    as in the reference's loop over parts, minit/module/checkpoint.py:23-37)."""
    from safetensors.numpy import load_file
    out: Dict[str, numpy.ndarray] = {}
    for path in paths:
        out.update(load_file(path))
    return out


def load_safetensors_index(index_path: str) -> Dict[str, numpy.ndarray]:
    """``model.safetensors.index.json`` -> tensors of the parts its ``weight_map``
    names, each part read once (minit/module/checkpoint.py:40-44)."""
    with open(index_path) as f:
        index = json.load(f)
    parts = list(dict.fromkeys(index["weight_map"].values()))
    return load_safetensors(os.path.join(os.path.dirname(index_path), part) for part in parts)


def quantized_linear(tensors: Mapping[str, numpy.ndarray], prefix: str):
    """``QLinear`` on the device for the buffers under ``prefix``."""
    from .linear import QLinear
    return QLinear.from_host(read_linear(tensors, prefix))
