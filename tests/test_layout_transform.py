"""Engine KV blocks <-> a dense device buffer (the re-layout step of the
reference's direct-storage path, csrc/gds/layout_transform.cu): the oracle
against numpy indexing of shaped arrays, the HIP path against the oracle."""
import numpy as np
import pytest
import torch

from kvsetup import KVSetup, SGLANG, TRTLLM, VLLM
from oracle import fkv_oracle as O

BACKENDS = [pytest.param(VLLM, "LAYERFIRST", id="vllm"),
            pytest.param(VLLM, "LAYERBLOCK", id="vllm-layerblock"),
            pytest.param(TRTLLM, "LAYERFIRST", id="trtllm"),
            pytest.param(SGLANG, "LAYERFIRST", id="sglang")]


def shaped_engine_view(s: KVSetup, arrays=None):
    """chunk(l, kv, block) as numpy views of the engine's byte buffers, by the
    documented tensor shapes (not by the stride arithmetic under test)."""
    L, K, N, C = s.num_layers, s.kv_dim, s.num_gpu_blocks, s.chunk
    arrays = s.gpu_ref if arrays is None else arrays
    if s.backend == VLLM and s.gpu_layout == "LAYERFIRST":
        t = [a.reshape(K, N, C) for a in arrays]
        return lambda l, kv, b: t[l][kv, b]
    if s.backend == VLLM:
        t = [a.reshape(N, K, C) for a in arrays]
        return lambda l, kv, b: t[l][b, kv]
    if s.backend == TRTLLM:
        t = arrays[0].reshape(N, L, K, C)
        return lambda l, kv, b: t[b, l, kv]
    t = [a.reshape(N, C) for a in arrays]
    return lambda l, kv, b: t[kv * L + l][b]


def buffer_strides(L, K, C, order, pad):
    """Dense [block, layer, kv, chunk] as the reference's staging slot is laid out
    (buffer_block_stride = slot size), or [block, kv, layer, chunk]; `pad` extra
    bytes after every chunk."""
    c = C + pad
    if order == "layer_kv":
        return dict(layer=K * c, kv=c, block=L * K * c)
    return dict(kv=L * c, layer=c, block=L * K * c)


def oracle_run(s, buf, st, ids, to_target, start_layer=0, num_layers=None):
    nl = s.num_layers - start_layer if num_layers is None else num_layers
    O.layout_transform(buf.ctypes.data, st["layer"], st["kv"], st["block"], s.chunk, s.backend,
                       s.ref_ptrs(), s.num_layers_total, s.gpu_kv_stride, s.gpu_block_stride,
                       s.gpu_layer_stride, ids, nl, s.kv_dim, to_target, start_layer)


@pytest.mark.parametrize("backend,gpu_layout", BACKENDS)
@pytest.mark.parametrize("order,pad", [("layer_kv", 0), ("kv_layer", 0), ("layer_kv", 48)])
def test_oracle_equals_shaped_indexing(backend, gpu_layout, order, pad):
    L, K, N, C = 3, 2, 11, 96
    s = KVSetup(backend, L, K, N, 4, C, gpu_layout=gpu_layout, seed=4)
    chunk_of = shaped_engine_view(s)
    st = buffer_strides(L, K, C, order, pad)
    ids = [7, 0, 10, 3, 3]
    buf = np.full(len(ids) * st["block"], 0xEE, dtype=np.uint8)
    oracle_run(s, buf, st, ids, False)
    c = C + pad
    shaped = buf.reshape(len(ids), L, K, c) if order == "layer_kv" else \
        buf.reshape(len(ids), K, L, c).transpose(0, 2, 1, 3)
    for i, b in enumerate(ids):
        for l in range(L):
            for kv in range(K):
                assert np.array_equal(shaped[i, l, kv, :C], chunk_of(l, kv, b)), (i, l, kv)
    assert (shaped[..., C:] == 0xEE).all()                      # padding untouched
    # the other direction: new bytes in the buffer land in the engine's tensors, and only there
    rng = np.random.default_rng(9)
    before = [a.copy() for a in s.gpu_ref]
    buf[:] = rng.integers(0, 256, buf.size, dtype=np.uint8)
    ids = [7, 0, 10, 3, 5]
    oracle_run(s, buf, st, ids, True)
    was = shaped_engine_view(s, before)
    for l in range(L):
        for kv in range(K):
            for i, b in enumerate(ids):
                assert np.array_equal(chunk_of(l, kv, b), shaped[i, l, kv, :C]), (i, l, kv)
            for b in set(range(N)) - set(ids):                   # blocks not named keep their bytes
                assert np.array_equal(chunk_of(l, kv, b), was(l, kv, b)), (l, kv, b)


def test_oracle_layer_window():
    L, K, N, C = 5, 2, 6, 64
    s = KVSetup(VLLM, L, K, N, 4, C, seed=2)
    chunk_of = shaped_engine_view(s)
    st = buffer_strides(2, K, C, "layer_kv", 0)
    buf = np.zeros(3 * st["block"], dtype=np.uint8)
    oracle_run(s, buf, st, [5, 1, 2], False, start_layer=3, num_layers=2)
    shaped = buf.reshape(3, 2, K, C)
    for i, b in enumerate([5, 1, 2]):
        for l in range(2):
            for kv in range(K):
                assert np.array_equal(shaped[i, l, kv], chunk_of(3 + l, kv, b))


# ---- the HIP path ----------------------------------------------------------------------------------

def device_run(d, buf_t, st, ids, to_target, start_layer=0, num_layers=None, **kw):
    from flexkv_amd.c_ext import layout_transform
    s = d.s
    nl = s.num_layers - start_layer if num_layers is None else num_layers
    layout_transform(buf_t, st["layer"], st["kv"], st["block"], s.chunk, d.ptrs, s.gpu_kv_stride,
                     s.gpu_block_stride, s.gpu_layer_stride,
                     torch.as_tensor(np.asarray(ids, dtype=np.int64)), nl, s.kv_dim, to_target,
                     gpu_block_type=s.backend, start_layer_id=start_layer, **kw)
    torch.cuda.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("backend,gpu_layout", BACKENDS)
@pytest.mark.parametrize("chunk,pad,nblk", [(4096, 0, 37), (1536, 16, 5), (264, 8, 1200),
                                             (100, 4, 9), (131072, 0, 12)])
def test_device_matches_the_oracle(gpu_device, backend, gpu_layout, chunk, pad, nblk):
    L, K, N = 4, 2, max(16, nblk + 3)
    s = KVSetup(backend, L, K, N, 4, chunk, gpu_layout=gpu_layout, seed=chunk % 97)
    d = s.to_device(gpu_device)
    rng = np.random.default_rng(nblk)
    ids = rng.permutation(N)[:nblk]
    for order in ("layer_kv", "kv_layer"):
        st = buffer_strides(L, K, chunk, order, pad)
        ref = rng.integers(0, 256, nblk * st["block"], dtype=np.uint8)
        buf = torch.from_numpy(ref.copy()).to(gpu_device)
        device_run(d, buf, st, ids, False)
        oracle_run(s, ref, st, ids, False)
        assert np.array_equal(buf.cpu().numpy(), ref), order
        # scatter fresh bytes back into other blocks
        ids2 = rng.permutation(N)[:nblk]
        ref[:] = rng.integers(0, 256, ref.size, dtype=np.uint8)
        buf.copy_(torch.from_numpy(ref))
        device_run(d, buf, st, ids2, True)
        oracle_run(s, ref, st, ids2, True)
        for got, want in zip(d.gpu_bytes(), s.gpu_ref):
            assert np.array_equal(got, want), order


@pytest.mark.gpu
def test_device_layer_window_many_pairs_and_errors(gpu_device):
    from flexkv_amd.c_ext import layout_transform
    # more (layer, kv) pairs than one launch's table holds: 600 layers x 2
    L, K, N, C = 600, 2, 6, 64
    s = KVSetup(TRTLLM, L, K, N, 2, C, seed=1)
    d = s.to_device(gpu_device)
    st = buffer_strides(L, K, C, "layer_kv", 0)
    ref = np.zeros(4 * st["block"], dtype=np.uint8)
    buf = torch.zeros(ref.size, dtype=torch.uint8, device=gpu_device)
    device_run(d, buf, st, [5, 0, 2, 3], False)
    oracle_run(s, ref, st, [5, 0, 2, 3], False)
    assert np.array_equal(buf.cpu().numpy(), ref)
    # a window of layers
    s = KVSetup(VLLM, 6, 2, 8, 2, 512, seed=3)
    d = s.to_device(gpu_device)
    st = buffer_strides(2, 2, 512, "layer_kv", 0)
    ref = np.zeros(3 * st["block"], dtype=np.uint8)
    buf = torch.zeros(ref.size, dtype=torch.uint8, device=gpu_device)
    device_run(d, buf, st, [7, 1, 4], False, start_layer=4, num_layers=2)
    oracle_run(s, ref, st, [7, 1, 4], False, start_layer=4, num_layers=2)
    assert np.array_equal(buf.cpu().numpy(), ref)
    device_run(d, buf, st, [], False)                               # nothing to do
    with pytest.raises(ValueError, match="shorter than"):
        device_run(d, buf[:100], st, [7, 1, 4], False, start_layer=4, num_layers=2)
    with pytest.raises(ValueError, match="negative block id"):
        device_run(d, buf, st, [7, -1, 4], False, start_layer=4, num_layers=2)
    with pytest.raises(ValueError, match="tensor pointers"):
        device_run(d, buf, st, [1], False, start_layer=5, num_layers=2)
    with pytest.raises(RuntimeError, match="Unsupported gpu_block_type: 7"):
        layout_transform(buf, 1024, 512, 2048, 512, d.ptrs, 0, 0, 0,
                         torch.tensor([1]), 2, 2, False, gpu_block_type=7)
    with pytest.raises(ValueError, match="device memory"):
        layout_transform(torch.zeros(10, dtype=torch.uint8), 1024, 512, 2048, 512, d.ptrs, 0, 0,
                         0, torch.tensor([1]), 2, 2, False)
