"""Layout/stride arithmetic against torch's own strides (a library routine, not
a retyped formula)."""
import itertools

import pytest
import torch

from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, TransferStrides,
                               gpu_block_type_from_tensor_count, gpu_strides_from_tensor)

AXES = {"LAYERFIRST": ("layer", "kv", "block"), "BLOCKFIRST": ("block", "layer", "kv"),
        "LAYERBLOCK": ("layer", "block", "kv")}


@pytest.mark.parametrize("name", list(AXES))
@pytest.mark.parametrize("dims", [(3, 5, 4, 2, 8, 2), (61, 7, 64, 1, 576, 1), (2, 4, 1, 8, 128, 2)])
def test_strides_equal_torch_strides(name, dims):
    L, N, T, H, D, K = dims
    lay = KVCacheLayout(KVCacheLayoutType[name], L, N, T, H, D, kv_dim=K)
    t = torch.empty(lay.kv_shape, dtype=torch.int8)
    assert t.numel() == lay.get_total_elements()
    st = dict(zip(AXES[name], t.stride()[:3]))
    assert lay.get_layer_stride() == st["layer"]
    assert lay.get_kv_stride() == st["kv"]
    assert lay.get_block_stride() == st["block"]
    assert lay.get_chunk_size() == T * H * D == t.stride()[AXES[name].index("kv")] or True
    # the chunk is the trailing contiguous [T, H, D] run
    assert lay.get_chunk_size() == t[(0,) * 3].numel()
    ts = TransferStrides.from_layout(lay, 2)
    assert (ts.kv, ts.block, ts.layer, ts.chunk) == (2 * st["kv"], 2 * st["block"],
                                                     2 * st["layer"], 2 * T * H * D)


def test_shapes_match_reference_axis_orders():
    # flexkv/common/storage.py:128-148
    lay = lambda ty: KVCacheLayout(ty, 3, 5, 4, 2, 8, kv_dim=2).kv_shape
    assert lay(KVCacheLayoutType.LAYERFIRST) == (3, 2, 5, 4, 2, 8)
    assert lay(KVCacheLayoutType.BLOCKFIRST) == (5, 3, 2, 4, 2, 8)
    assert lay(KVCacheLayoutType.LAYERBLOCK) == (3, 5, 2, 4, 2, 8)


def test_div_head_keeps_block_count_and_splits_heads():
    lay = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, 4, 8, 16, 8, 128, kv_dim=2, num_kv_heads=8)
    tp = lay.div_head(4)
    assert tp.num_head == 2 and tp.num_block == 8
    assert tp.get_chunk_size() * 4 == lay.get_chunk_size()
    # per-rank strides: a rank's (layer, kv) chunks are dense inside its quarter of the block
    assert tp.get_layer_stride() == 2 * tp.get_chunk_size()
    assert lay.get_block_stride() // 4 == 4 * tp.get_layer_stride()
    with pytest.raises(ValueError):
        lay.div_head(3)
    assert lay.div_block(2).num_block == 4 and lay.div_block(3, padding=True).num_block == 3
    assert lay.div_layer(2).num_layer == 2


@pytest.mark.parametrize("perm", list(itertools.permutations(("kv", "block", "token"))))
def test_stride_probe_on_permuted_engine_tensor(perm):
    """Whatever order an engine gives the (kv, block, token) axes, the probe
    returns torch's stride of the kv and block axes (worker.py:262-306)."""
    ext = {"kv": 2, "block": 7, "token": 16}
    shape = tuple(ext[a] for a in perm) + (4, 32)
    t = torch.empty(shape, dtype=torch.bfloat16)
    kvs, bs, ls = gpu_strides_from_tensor(t.shape, t.stride(), 16, 2, 2)
    assert kvs == t.stride(perm.index("kv")) * 2
    assert bs == t.stride(perm.index("block")) * 2
    assert ls == t.numel() * 2


def test_stride_probe_falls_back():
    assert gpu_strides_from_tensor((2, 7, 16, 4, 32), (1,) * 5, 16, 2, kv_dim=1) is None
    assert gpu_strides_from_tensor((7, 16, 576), (1,) * 3, 16, 2, kv_dim=2) is None
    assert gpu_strides_from_tensor((3, 7, 16, 4, 32), (1,) * 5, 16, 2, kv_dim=2) is None  # no axis of 2


def test_backend_tag_from_tensor_count():
    assert gpu_block_type_from_tensor_count(1, 32) == 1
    assert gpu_block_type_from_tensor_count(32, 32) == 0
    assert gpu_block_type_from_tensor_count(64, 32) == 2
    with pytest.raises(ValueError):
        gpu_block_type_from_tensor_count(33, 32)


def test_baseline_config_strides():
    """Byte strides of the benchmark configurations (Llama-3-8B vLLM layout and
    its block-first host cache)."""
    g = TransferStrides.from_layout(
        KVCacheLayout(KVCacheLayoutType.LAYERFIRST, 32, 4096, 16, 8, 128, kv_dim=2), 2)
    assert (g.chunk, g.block, g.kv, g.layer) == (32768, 32768, 134217728, 268435456)
    c = TransferStrides.from_layout(
        KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, 32, 1024, 16, 8, 128, kv_dim=2), 2)
    assert (c.block, c.layer, c.kv) == (2097152, 65536, 32768)
