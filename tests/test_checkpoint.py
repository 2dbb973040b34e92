"""GPTQ checkpoint ingestion (examples/qwen1_5_int8.py:276-317,
minit/module/checkpoint.py:23-44): geometry from stored shapes, sequential
g_idx detection, safetensors files and indexes; on the GPU, a linear loaded from
a file -- with bias, and with an act-order g_idx -- against the oracle."""
import json
import os

import numpy as np
import pytest

from minit_amd.quantize import checkpoint as ck
from minit_amd.quantize.gptq import pack_subwords
from oracle import gptq as O
from tests.helpers import assert_fp16_close


def _linear(rng, k, n, g, bits, act_order=False, bias=True):
    q = rng.integers(0, 1 << bits, size=(k, n))
    z = rng.integers(0, 1 << bits, size=(k // g, n))
    tensors = {
        "qweight": pack_subwords(q, 0, bits),
        "qzeros": pack_subwords(z, 1, bits),
        "scales": (np.abs(rng.normal(0, 0.02, size=(k // g, n))) + 1e-3).astype(np.float16),
        "g_idx": (rng.permutation(k) // g if act_order else np.arange(k) // g).astype(np.int32),
    }
    if bias:
        tensors["bias"] = rng.normal(0, 0.5, size=(n,)).astype(np.float16)
    return tensors


def _named(prefix, tensors):
    return {f"{prefix}.{k}": v for k, v in tensors.items()}


@pytest.mark.parametrize("k,n,g,bits", [(4096, 4096, 128, 4), (512, 264, 64, 8), (256, 8, 256, 4), (96, 16, 32, 8)])
def test_geometry_from_shapes(k, n, g, bits):
    per_word = 32 // bits
    geo = ck.infer_geometry((k // per_word, n), (k // g, n // per_word), (k // g, n), k)
    assert geo == ck.GPTQGeometry(bits, g, k, n)


@pytest.mark.parametrize("shapes", [
    ((512, 4096), (32, 512), (31, 4096), None),    # group counts differ
    ((512, 4096), (32, 512), (32, 4088), None),    # N differs
    ((512, 4096), (32, 256), (32, 4096), None),    # 16 sub-words per word: 2-bit, unsupported
    ((513, 4096), (32, 512), (32, 4096), None),    # K not a whole number of groups
    ((512, 4096), (32, 512), (32, 4096), 4095),    # g_idx length (qwen1_5_int8.py:247-254)
    ((512,), (32, 512), (32, 4096), None),
])
def test_geometry_rejects_inconsistent_shapes(shapes):
    with pytest.raises(ValueError):
        ck.infer_geometry(*shapes)


def test_sequential_g_idx_is_dropped_and_act_order_kept():
    rng = np.random.default_rng(1)
    w = ck.read_linear(_named("m.q_proj", _linear(rng, 512, 64, 128, 4)), "m.q_proj")
    assert w.g_idx is None and w.geometry == ck.GPTQGeometry(4, 128, 512, 64) and w.bias.shape == (64,)
    w = ck.read_linear(_named("m.q_proj", _linear(rng, 512, 64, 128, 4, act_order=True, bias=False)), "m.q_proj")
    assert w.g_idx is not None and w.g_idx.dtype == np.int32 and w.bias is None
    one_swap = np.arange(512) // 128
    one_swap[[0, 511]] = one_swap[[511, 0]]
    assert not ck.is_sequential_g_idx(one_swap, 128) and ck.is_sequential_g_idx(np.arange(512) // 128, 128)


def test_read_linear_reports_what_is_wrong():
    rng = np.random.default_rng(2)
    t = _named("l", _linear(rng, 256, 32, 128, 4))
    with pytest.raises(KeyError, match="qzeros"):
        ck.read_linear({k: v for k, v in t.items() if not k.endswith("qzeros")}, "l")
    bad = dict(t)
    bad["l.bias"] = np.zeros(31, np.float16)
    with pytest.raises(ValueError, match="bias"):
        ck.read_linear(bad, "l")
    bad = dict(t)
    bad["l.g_idx"] = np.full(256, 2, np.int32)  # only groups 0 and 1 exist
    with pytest.raises(ValueError, match="g_idx"):
        ck.read_linear(bad, "l")
    bad = dict(t)
    bad["l.qweight"] = t["l.qweight"].astype(np.int64)
    with pytest.raises(ValueError, match="int32"):
        ck.read_linear(bad, "l")


def test_safetensors_files_and_index(tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(3)
    a = _named("model.layers.0.self_attn.q_proj", _linear(rng, 256, 64, 128, 4))
    b = _named("model.layers.0.mlp.down_proj", _linear(rng, 512, 32, 128, 8, bias=False))
    extra = {"model.norm.weight": np.ones(64, np.float16)}
    save_file(a, os.path.join(tmp_path, "part-1.safetensors"))
    save_file({**b, **extra}, os.path.join(tmp_path, "part-2.safetensors"))
    weight_map = {**{k: "part-1.safetensors" for k in a}, **{k: "part-2.safetensors" for k in {**b, **extra}}}
    index = os.path.join(tmp_path, "model.safetensors.index.json")
    with open(index, "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f)
    tensors = ck.load_safetensors_index(index)
    assert set(tensors) == set(a) | set(b) | set(extra)
    assert ck.linear_prefixes(tensors) == ["model.layers.0.mlp.down_proj", "model.layers.0.self_attn.q_proj"]
    w = ck.read_linear(tensors, "model.layers.0.mlp.down_proj")
    assert w.geometry == ck.GPTQGeometry(8, 128, 512, 32)
    np.testing.assert_array_equal(w.qweight, b["model.layers.0.mlp.down_proj.qweight"])
    same = ck.load_safetensors([os.path.join(tmp_path, "part-1.safetensors")])
    np.testing.assert_array_equal(same["model.layers.0.self_attn.q_proj.scales"],
                                  a["model.layers.0.self_attn.q_proj.scales"])


@pytest.mark.gpu
@pytest.mark.parametrize("k,n,g,bits,act_order", [(1024, 512, 128, 4, False), (512, 264, 64, 8, False),
                                                  (1024, 256, 128, 4, True)])
def test_linear_from_checkpoint_matches_oracle(hip, tmp_path, k, n, g, bits, act_order):
    """File -> QLinear -> forward, bias included, leading axes folded; the act-order
    checkpoint is repacked once (rows sorted by group) and runs on the MFMA kernels
    with gathered activations."""
    from safetensors.numpy import save_file
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    rng = np.random.default_rng(10 + bits + int(act_order))
    t = _linear(rng, k, n, g, bits, act_order=act_order)
    path = os.path.join(tmp_path, "w.safetensors")
    save_file(_named("layer.proj", t), path)
    lin = ck.quantized_linear(ck.load_safetensors([path]), "layer.proj")
    assert lin.weight._group is None and (lin.input_order is not None) == act_order
    assert lin.weight.bits == bits and lin.weight.group_size == g
    x = synthetic.activations("ckpt", f"x{k}", (2, 3, k))
    y = lin(HIPTensor.from_numpy(x)).numpy()
    assert y.shape == (2, 3, n)
    g_idx = t["g_idx"] if act_order else None
    prod = O.matmul_f64(x.reshape(6, k), t["qweight"], t["qzeros"], t["scales"], g_idx, bits, g)
    # the reference adds the bias to the fp16 product, in fp16
    ref = (prod.astype(np.float16).astype(np.float64) + t["bias"].astype(np.float64)).reshape(2, 3, n)
    assert_fp16_close(y, ref, what="checkpoint linear")


def test_sort_rows_by_group_is_a_row_permutation_with_sequential_groups():
    """W_sorted[j] = W[perm[j]] bit for bit (the oracle's act-order dequantization
    against its sequential one on the repacked words), groups become sequential,
    and a weight whose groups are of uneven size is left alone."""
    from minit_amd.quantize.gptq import sort_rows_by_group, unpack_subwords
    rng = np.random.default_rng(5)
    for k, n, g, bits in ((512, 24, 128, 4), (256, 16, 64, 8)):
        t = _linear(rng, k, n, g, bits, act_order=True)
        qsorted, perm = sort_rows_by_group(t["qweight"], t["g_idx"], bits, g)
        assert sorted(perm.tolist()) == list(range(k))
        assert (t["g_idx"][perm] == np.arange(k) // g).all()
        np.testing.assert_array_equal(unpack_subwords(qsorted, 0, bits), O.unpack(t["qweight"], 0, bits)[perm])
        w_act = O.dequantize_packed(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], bits, g)
        w_seq = O.dequantize_packed(qsorted, t["qzeros"], t["scales"], None, bits, g)
        np.testing.assert_array_equal(w_seq.view(np.uint16), w_act[perm].view(np.uint16))
    uneven = t["g_idx"].copy()
    uneven[np.flatnonzero(uneven == 0)[0]] = 1
    assert sort_rows_by_group(t["qweight"], uneven, bits, g) is None


@pytest.mark.gpu
@pytest.mark.parametrize("k,n,g,bits", [(512, 24, 128, 4), (256, 16, 64, 8), (4096, 1000, 128, 4), (1024, 12, 32, 8)])
def test_device_repack_equals_the_host_repack(hip, k, n, g, bits):
    """mh_gptq_permute_rows against the numpy repack, word for word; a random permutation
    (not only a sort by group) as well, and the identity returns the input."""
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.gptq import (group_order, sort_rows_by_group, sort_rows_by_group_on_device,
                                         unpack_subwords)
    rng = np.random.default_rng(k + n)
    t = _linear(rng, k, n, g, bits, act_order=True)
    qsorted, perm = sort_rows_by_group(t["qweight"], t["g_idx"], bits, g)
    np.testing.assert_array_equal(perm, group_order(t["g_idx"], g))
    words = HIPTensor.from_numpy(t["qweight"])
    got = sort_rows_by_group_on_device(words, HIPTensor.from_numpy(perm), bits).numpy()
    np.testing.assert_array_equal(got, qsorted)
    shuffle = rng.permutation(k).astype(np.int32)
    got = sort_rows_by_group_on_device(words, HIPTensor.from_numpy(shuffle), bits).numpy()
    np.testing.assert_array_equal(got, pack_subwords(unpack_subwords(t["qweight"], 0, bits)[shuffle], 0, bits))
    same = sort_rows_by_group_on_device(words, HIPTensor.from_numpy(np.arange(k, dtype=np.int32)), bits).numpy()
    np.testing.assert_array_equal(same, t["qweight"])


@pytest.mark.gpu
def test_act_order_repacked_and_per_element_paths_agree(hip):
    """The same act-order checkpoint with and without the one-time repack, against
    the oracle; one-hot activations return rows of the dequantized matrix bit for
    bit on both paths."""
    from minit_amd import synthetic
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.quantize.linear import QLinear
    k, n, g, bits = 2048, 1024, 128, 4
    t = _linear(np.random.default_rng(21), k, n, g, bits, act_order=True, bias=False)
    w = ck.read_linear(_named("p", t), "p")
    fast, slow = QLinear.from_host(w), QLinear.from_host(w, reorder=False)
    assert fast.input_order is not None and slow.input_order is None and slow.weight._group is not None
    x = synthetic.activations("ckpt", "act", (5, k))
    ref = O.matmul_f64(x, t["qweight"], t["qzeros"], t["scales"], t["g_idx"], bits, g)
    dx = HIPTensor.from_numpy(x)
    assert_fp16_close(fast(dx).numpy(), ref, what="repacked act-order")
    assert_fp16_close(slow(dx).numpy(), ref, what="per-element act-order")
    dense = O.dequantize_packed(t["qweight"], t["qzeros"], t["scales"], t["g_idx"], bits, g)
    rows = [0, 1, k // 2 + 3, k - 2, k - 1]
    onehot = np.zeros((5, k), np.float16)
    onehot[np.arange(5), rows] = 1.0
    dh = HIPTensor.from_numpy(onehot)
    np.testing.assert_array_equal(fast(dh).numpy().view(np.uint16), dense[rows].view(np.uint16))
    np.testing.assert_array_equal(slow(dh).numpy().view(np.uint16), dense[rows].view(np.uint16))


@pytest.mark.gpu
def test_add_bias_is_one_fp16_add(hip):
    from minit_amd.hip.tensor import HIPTensor
    from minit_amd.lib import DTYPE_CODES
    rng = np.random.default_rng(5)
    x = rng.normal(0, 4, size=(37, 264)).astype(np.float16)
    b = rng.normal(0, 1, size=(264,)).astype(np.float16)
    dx, db = HIPTensor.from_numpy(x), HIPTensor.from_numpy(b)
    hip.call("mh_add_bias", None, dx.data_ptr, db.data_ptr, 37, 264, DTYPE_CODES["float16"])
    np.testing.assert_array_equal(dx.numpy().view(np.uint16), (x + b[None, :]).astype(np.float16).view(np.uint16))
