"""Pins the CPU oracle (oracle/fkv_oracle.c) before anything is compared to it.

None of these checks retypes the oracle's formula: addresses are checked
against torch/numpy indexing of real tensors with the engines' shapes, the
transfer against fancy-index assignment on shaped tensors, the reference
tests' deterministic fill as a known answer, and invariants (round trip,
untouched bytes, layer split == single call).
"""
import ctypes

import numpy as np
import pytest
import torch

from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, gpu_strides_from_tensor)
from kvsetup import KVSetup, VLLM, TRTLLM, SGLANG, block_ids
from oracle import fkv_oracle as O


def _byte_at(addr: int) -> int:
    return ctypes.c_uint8.from_address(addr).value


def _first_bytes(t: torch.Tensor, n: int = 4) -> bytes:
    return bytes(t.contiguous().view(torch.uint8).flatten()[:n].tolist())


def _bytes_at(addr: int, n: int = 4) -> bytes:
    return bytes(_byte_at(addr + i) for i in range(n))


# ---- address arithmetic vs real engine tensors ------------------------------

def test_chunk_addr_vllm_both_axis_orders():
    """vLLM per-layer tensors: [2, N, T, H, D] (flash-attn) and [N, 2, T, H, D]
    (triton/flashinfer), reference tests/common_utils.py:261-265 and
    flexkv/transfer/worker.py:262-306."""
    L, N, T, H, D = 3, 7, 4, 2, 8
    for order in ("kv_first", "block_first"):
        shape = (2, N, T, H, D) if order == "kv_first" else (N, 2, T, H, D)
        layers = [torch.arange(l * 10000, l * 10000 + 2 * N * T * H * D, dtype=torch.int32)
                  .reshape(shape) for l in range(L)]
        kvs, bs, ls = gpu_strides_from_tensor(shape, layers[0].stride(), T, 4, 2)
        ptrs = [x.data_ptr() for x in layers]
        for l in range(L):
            for kv in range(2):
                for b in (0, 3, N - 1):
                    addr = O.chunk_addr(VLLM, ptrs, L, kvs, bs, ls, l, kv, b)
                    want = layers[l][kv, b] if order == "kv_first" else layers[l][b, kv]
                    assert _bytes_at(addr) == _first_bytes(want), (order, l, kv, b)
                    # the chunk is the contiguous run of T*H*D elements
                    last = addr + (T * H * D - 1) * 4
                    assert _bytes_at(last) == _first_bytes(want.flatten()[-1:]), (order, l, kv, b)


def test_chunk_addr_trtllm_single_tensor():
    """TRT-LLM: one tensor [N, L, kv, T, H, D] (tests/common_utils.py:266-270)."""
    N, L, T, H, D = 5, 4, 2, 3, 8
    x = torch.arange(N * L * 2 * T * H * D, dtype=torch.int32).reshape(N, L, 2, T, H, D)
    lay = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, N, T, H, D, kv_dim=2)
    kvs, bs, ls = (lay.get_kv_stride() * 4, lay.get_block_stride() * 4, lay.get_layer_stride() * 4)
    for b in range(N):
        for l in range(L):
            for kv in range(2):
                addr = O.chunk_addr(TRTLLM, [x.data_ptr()], L, kvs, bs, ls, l, kv, b)
                assert _bytes_at(addr) == _first_bytes(x[b, l, kv])


def test_chunk_addr_sglang_k_then_v_tensors():
    """SGLang: K_0..K_{L-1}, V_0..V_{L-1}, each [tokens, H, D]; a block is a page
    of `page` tokens (flexkv/integration/sglang/connector.py:1976-1987)."""
    L, tokens, H, D, page = 3, 40, 2, 8, 8
    ts = [torch.arange(i * 100000, i * 100000 + tokens * H * D, dtype=torch.int32)
          .reshape(tokens, H, D) for i in range(2 * L)]
    bs = page * H * D * 4
    ptrs = [t.data_ptr() for t in ts]
    for l in range(L):
        for kv in range(2):
            for b in range(tokens // page):
                addr = O.chunk_addr(SGLANG, ptrs, L, 0, bs, 0, l, kv, b)
                want = ts[kv * L + l].view(tokens // page, page, H, D)[b]
                assert _bytes_at(addr) == _first_bytes(want)


# ---- whole transfer vs fancy-index assignment on shaped tensors -------------

@pytest.mark.parametrize("cpu_type", [KVCacheLayoutType.BLOCKFIRST, KVCacheLayoutType.LAYERFIRST,
                                      KVCacheLayoutType.LAYERBLOCK])
@pytest.mark.parametrize("kv_dim", [1, 2])
def test_d2h_equals_torch_index_assignment(cpu_type, kv_dim):
    """host[shape-indexed] = layer[kv, gpu_ids] with torch fancy indexing."""
    L, N, NH, T, H, D = 3, 9, 6, 4, 2, 8
    g = torch.Generator().manual_seed(0)
    layers = [torch.randint(-30000, 30000, (kv_dim, N, T, H, D), dtype=torch.int16, generator=g)
              for _ in range(L)]
    gl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, N, T, H, D, kv_dim=kv_dim)
    cl = KVCacheLayout(cpu_type, L, NH, T, H, D, kv_dim=kv_dim)
    host = torch.zeros(cl.kv_shape, dtype=torch.int16)
    want = host.clone()
    gids = torch.tensor([7, 0, 3, 8], dtype=torch.int64)
    cids = torch.tensor([2, 5, 0, 1], dtype=torch.int64)
    for l in range(L):
        for kv in range(kv_dim):
            rows = layers[l][kv, gids]                      # [n, T, H, D]
            if cpu_type == KVCacheLayoutType.BLOCKFIRST:    # [NH, L, kv, ...]
                want[cids, l, kv] = rows
            elif cpu_type == KVCacheLayoutType.LAYERFIRST:  # [L, kv, NH, ...]
                want[l, kv, cids] = rows
            else:                                           # [L, NH, kv, ...]
                want[l, cids, kv] = rows
    O.transfer_c(VLLM, [x.data_ptr() for x in layers], L,
                 gl.get_kv_stride() * 2, gl.get_block_stride() * 2, gl.get_layer_stride() * 2, 0,
                 host.data_ptr(), cl.get_kv_stride() * 2, cl.get_layer_stride() * 2,
                 cl.get_block_stride() * 2, 0, gl.get_chunk_size() * 2, 0, L, kv_dim,
                 gids.numpy(), cids.numpy(), False)
    assert torch.equal(host, want)
    # and back: H2D into other blocks reproduces torch index assignment
    gids2 = torch.tensor([1, 2, 4, 6], dtype=torch.int64)
    want_layers = [x.clone() for x in layers]
    for l in range(L):
        for kv in range(kv_dim):
            if cpu_type == KVCacheLayoutType.BLOCKFIRST:
                want_layers[l][kv, gids2] = host[cids, l, kv]
            elif cpu_type == KVCacheLayoutType.LAYERFIRST:
                want_layers[l][kv, gids2] = host[l, kv, cids]
            else:
                want_layers[l][kv, gids2] = host[l, cids, kv]
    O.transfer_c(VLLM, [x.data_ptr() for x in layers], L,
                 gl.get_kv_stride() * 2, gl.get_block_stride() * 2, gl.get_layer_stride() * 2, 0,
                 host.data_ptr(), cl.get_kv_stride() * 2, cl.get_layer_stride() * 2,
                 cl.get_block_stride() * 2, 0, gl.get_chunk_size() * 2, 0, L, kv_dim,
                 gids2.numpy(), cids.numpy(), True)
    for a, b in zip(layers, want_layers):
        assert torch.equal(a, b)


def test_reference_cpu_path_gather_equals_oracle():
    """The torch index-gather the benchmark times as CPU baseline produces the
    same host cache as the byte-address oracle."""
    L, N, NH, T, H, D = 4, 16, 8, 4, 2, 8
    g = torch.Generator().manual_seed(3)
    layers = [torch.randn(2, N, T, H, D, generator=g).to(torch.bfloat16) for _ in range(L)]
    host_a = torch.zeros(NH, L, 2, T, H, D, dtype=torch.bfloat16)
    host_b = torch.zeros_like(host_a)
    gids = torch.randperm(N, generator=g)[:5]
    cids = torch.randperm(NH, generator=g)[:5]
    O.torch_index_gather(layers, host_a, gids, cids)
    chunk = T * H * D * 2
    O.transfer_c(VLLM, [x.data_ptr() for x in layers], L, N * chunk, chunk, 2 * N * chunk, 0,
                 host_b.data_ptr(), chunk, 2 * chunk, L * 2 * chunk, 0, chunk, 0, L, 2,
                 gids.numpy(), cids.numpy(), False)
    assert torch.equal(host_a.view(torch.int16), host_b.view(torch.int16))
    # scatter back into zeroed tensors restores exactly the selected blocks
    restored = [torch.zeros_like(x) for x in layers]
    O.torch_index_scatter(restored, host_a, gids, cids)
    for r, x in zip(restored, layers):
        assert torch.equal(r[:, gids].view(torch.int16), x[:, gids].view(torch.int16))
        mask = torch.ones(N, dtype=torch.bool)
        mask[gids] = False
        assert not r[:, mask].view(torch.int16).any()


@pytest.mark.parametrize("kv_dim", [1, 2])
def test_reference_cpu_path_on_planes_equals_oracle(kv_dim):
    """The per-(layer, K-or-V) form of the CPU baseline (SGLang pages, MLA blocks):
    same host cache as the byte-address oracle with SGLang addressing, and the
    scatter puts the selected blocks back."""
    L, N, NH, T, H, D = 3, 12, 9, 4, 2, 8
    g = torch.Generator().manual_seed(4)
    planes = [[torch.randn(N, T, H, D, generator=g).to(torch.bfloat16) for _ in range(kv_dim)]
              for _ in range(L)]
    host_a = torch.zeros(NH, L, kv_dim, T, H, D, dtype=torch.bfloat16)
    host_b = torch.zeros_like(host_a)
    gids = torch.randperm(N, generator=g)[:6]
    cids = torch.randperm(NH, generator=g)[:6]
    O.torch_index_gather_planes(planes, host_a, gids, cids)
    chunk = T * H * D * 2
    ptrs = [planes[l][kv].data_ptr() for kv in range(kv_dim) for l in range(L)]  # K_0.., V_0..
    O.transfer_c(O.BACKEND_SGLANG, ptrs, L, 0, chunk, N * chunk, 0, host_b.data_ptr(), chunk,
                 kv_dim * chunk, L * kv_dim * chunk, 0, chunk, 0, L, kv_dim, gids.numpy(),
                 cids.numpy(), False)
    assert torch.equal(host_a.view(torch.int16), host_b.view(torch.int16))
    restored = [[torch.zeros_like(x) for x in kvs] for kvs in planes]
    O.torch_index_scatter_planes(restored, host_a, gids, cids)
    for l in range(L):
        for kv in range(kv_dim):
            want = torch.zeros_like(planes[l][kv])
            want[gids] = planes[l][kv][gids]
            assert torch.equal(restored[l][kv].view(torch.int16), want.view(torch.int16))


# ---- the reference tests' deterministic fill as a known answer --------------

def _reference_fill(gpu_id, L, N, T, H, D, kv_dim):
    """fill_gpu of tests/test_kv_transfer_correctness.py:262-272: value depends on
    (gpu, kv, layer, block, token, last-axis index), identical across heads."""
    out = []
    for layer in range(L):
        kv = torch.arange(kv_dim).view(kv_dim, 1, 1, 1, 1)
        blk = torch.arange(N).view(1, N, 1, 1, 1)
        tok = torch.arange(T).view(1, 1, T, 1, 1)
        h = torch.arange(D).view(1, 1, 1, 1, D)
        vals = (gpu_id * 100000 + kv * 500000 + layer * 10000 + blk * 1000 + tok * 10 + h) % 997
        out.append((vals / 997.0).to(torch.float16).expand(kv_dim, N, T, H, D).contiguous())
    return out


def _reference_expected(gpu_id, layer, block, token, d, kv):
    """expected_val of tests/test_kv_transfer_correctness.py:275-278."""
    return float(((gpu_id * 100000 + kv * 500000 + layer * 10000 + block * 1000 +
                   token * 10 + d) % 997) / 997.0)


@pytest.mark.parametrize("cpu_name", ["LAYERFIRST", "BLOCKFIRST"])
@pytest.mark.parametrize("cfg", [(4, 8, 16, 1, 512, 1), (4, 8, 16, 8, 128, 2)],
                         ids=["mla_packed", "mha_plain"])  # TP1_CONFIGS :715-721
def test_known_answer_from_reference_fill(cpu_name, cfg):
    L, N, T, H, D, kv_dim = cfg
    layers = _reference_fill(0, L, N, T, H, D, kv_dim)
    gl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, N, T, H, D, kv_dim=kv_dim)
    cl = KVCacheLayout(KVCacheLayoutType[cpu_name], L, N, T, H, D, kv_dim=kv_dim)
    host = torch.zeros(cl.kv_shape, dtype=torch.float16)
    ids = np.arange(N, dtype=np.int64)
    O.transfer_c(VLLM, [x.data_ptr() for x in layers], L, gl.get_kv_stride() * 2,
                 gl.get_block_stride() * 2, gl.get_layer_stride() * 2, 0, host.data_ptr(),
                 cl.get_kv_stride() * 2, cl.get_layer_stride() * 2, cl.get_block_stride() * 2, 0,
                 gl.get_chunk_size() * 2, 0, L, kv_dim, ids, ids, False)
    for layer in (0, L - 1):
        for block in (0, N - 1):
            for kv in range(kv_dim):
                for d in (0, D - 1):
                    exp = _reference_expected(0, layer, block, 0, d, kv)
                    got = (host[block, layer, kv, 0, 0, d] if cpu_name == "BLOCKFIRST"
                           else host[layer, kv, block, 0, 0, d]).item()
                    assert abs(got - exp) < 1e-3  # tolerance of the reference's spot check :498-510
    # round trip through zeroed GPU tensors (the reference's test shape :760-795)
    zeroed = [torch.zeros_like(x) for x in layers]
    O.transfer_c(VLLM, [x.data_ptr() for x in zeroed], L, gl.get_kv_stride() * 2,
                 gl.get_block_stride() * 2, gl.get_layer_stride() * 2, 0, host.data_ptr(),
                 cl.get_kv_stride() * 2, cl.get_layer_stride() * 2, cl.get_block_stride() * 2, 0,
                 gl.get_chunk_size() * 2, 0, L, kv_dim, ids, ids, True)
    for a, b in zip(zeroed, layers):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


# ---- C byte loop == independent numpy index formulation ---------------------

CASES = [
    (VLLM, 3, 2, 12, 9, 256, "BLOCKFIRST", "LAYERFIRST", 0),
    (VLLM, 3, 2, 12, 9, 256, "LAYERFIRST", "LAYERBLOCK", 64),
    (VLLM, 2, 1, 10, 10, 1152, "BLOCKFIRST", "LAYERFIRST", 0),
    (TRTLLM, 4, 2, 8, 8, 512, "BLOCKFIRST", "LAYERFIRST", 0),
    (TRTLLM, 4, 1, 8, 6, 96, "LAYERFIRST", "LAYERFIRST", 32),
    (SGLANG, 3, 2, 16, 8, 1024, "BLOCKFIRST", "LAYERFIRST", 0),
    (SGLANG, 3, 2, 16, 8, 40, "LAYERFIRST", "LAYERFIRST", 8),
]


@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout,pad", CASES)
@pytest.mark.parametrize("is_h2d", [False, True])
def test_c_loop_equals_index_form(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, pad, is_h2d):
    a = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=9, gpu_block_pad=pad)
    b = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=9, gpu_block_pad=pad)
    rng = np.random.default_rng(1)
    n = min(N, NH) - 2
    gids, cids = block_ids(rng, N, n), block_ids(rng, NH, n)
    a.oracle_transfer(gids, cids, is_h2d, start_layer=1, num_layers=L - 1)
    b.oracle_transfer(gids, cids, is_h2d, start_layer=1, num_layers=L - 1, use_index_form=True)
    np.testing.assert_array_equal(a.host_ref, b.host_ref)
    for x, y in zip(a.gpu_ref, b.gpu_ref):
        np.testing.assert_array_equal(x, y)


# ---- invariants --------------------------------------------------------------

@pytest.mark.parametrize("backend", [VLLM, TRTLLM, SGLANG])
def test_untouched_bytes_and_round_trip(backend):
    s = KVSetup(backend, 3, 2, 10, 10, 128, "BLOCKFIRST", seed=4, gpu_block_pad=16)
    gpu0 = [x.copy() for x in s.gpu_ref]
    host0 = s.host_ref.copy()
    gids = np.array([4, 1, 7], dtype=np.int64)
    cids = np.array([0, 9, 5], dtype=np.int64)
    s.oracle_transfer(gids, cids, False)
    for x, y in zip(s.gpu_ref, gpu0):           # a gather never writes the source
        np.testing.assert_array_equal(x, y)
    touched = np.zeros(s.host_bytes, dtype=bool)
    for c in cids:
        touched[c * s.cpu_block_stride:(c + 1) * s.cpu_block_stride] = True
    np.testing.assert_array_equal(s.host_ref[~touched], host0[~touched])
    assert (s.host_ref[touched] != host0[touched]).any()
    # erase the blocks on the "GPU", scatter back: identity on the data, padding untouched
    for x in s.gpu_ref:
        x[:] = 0
    s.oracle_transfer(gids, cids, True)
    bs, C = s.gpu_block_stride, s.chunk
    for t, (x, y) in enumerate(zip(s.gpu_ref, gpu0)):
        for l in range(s.num_layers):
            for kv in range(2):
                for b in range(10):
                    if backend == VLLM:
                        if t != l:
                            continue
                        off = kv * s.gpu_kv_stride + b * bs
                    elif backend == TRTLLM:
                        off = b * bs + l * s.gpu_layer_stride + kv * s.gpu_kv_stride
                    else:
                        if t != kv * s.num_layers + l:
                            continue
                        off = b * bs
                    if b in gids:
                        np.testing.assert_array_equal(x[off:off + C], y[off:off + C])
                    else:
                        assert not x[off:off + C].any()
                    assert not x[off + C:off + C + 16].any()  # inter-block padding never written


def test_layer_split_equals_single_call():
    a = KVSetup(VLLM, 6, 2, 8, 8, 64, "BLOCKFIRST", seed=2)
    b = KVSetup(VLLM, 6, 2, 8, 8, 64, "BLOCKFIRST", seed=2)
    ids = np.array([3, 5, 0], dtype=np.int64)
    a.oracle_transfer(ids, ids[::-1].copy(), False)
    for l0 in range(0, 6, 2):
        b.oracle_transfer(ids, ids[::-1].copy(), False, start_layer=l0, num_layers=2)
    np.testing.assert_array_equal(a.host_ref, b.host_ref)


def test_in_chunk_offsets_select_a_byte_range():
    """gpu/cpu start offsets + a shorter chunk move exactly that byte range of
    every chunk (the sharded MLA D2H case, tp_transfer_thread_group.cpp:295-300)."""
    s = KVSetup(VLLM, 2, 1, 6, 6, 96, "BLOCKFIRST", seed=8)
    host0 = s.host_ref.copy()
    ids = np.array([2, 4], dtype=np.int64)
    s.oracle_transfer(ids, ids, False, gpu_off=32, cpu_off=32, chunk=32)
    for l in range(2):
        for b in ids:
            g = s.gpu_ref[l][b * 96:(b + 1) * 96]
            c0 = b * s.cpu_block_stride + l * s.cpu_layer_stride
            np.testing.assert_array_equal(s.host_ref[c0 + 32:c0 + 64], g[32:64])
            np.testing.assert_array_equal(s.host_ref[c0:c0 + 32], host0[c0:c0 + 32])
            np.testing.assert_array_equal(s.host_ref[c0 + 64:c0 + 96], host0[c0 + 64:c0 + 96])


def test_units_precondition():
    L = O.lib()
    assert L.fkv_oracle_units_ok(32768, 0, 0, 64, 32768, 128, 32768, 65536, 2097152) == 16
    assert L.fkv_oracle_units_ok(37440, 4680, 4680, 0, 37440, 0, 37440, 37440, 37440) == 8
    assert L.fkv_oracle_units_ok(100, 0, 0, 0, 100, 0, 100, 100, 100) == 0


# ---- host staging rows, full-block test, eventfd table ----------------------

@pytest.mark.parametrize("cpu_layout", ["BLOCKFIRST", "LAYERFIRST"])
@pytest.mark.parametrize("kv_dim", [1, 2])
def test_host_scatter_equals_numpy_indexing_of_a_shaped_pool(cpu_layout, kv_dim):
    """scatter_to_cpu / gather_from_cpu (csrc/ce_transfer.cu:523-641) move the rows of
    one (layer, kv) between a dense staging array [n, chunk] and the host cache.  On a
    shaped pool that is pool[ids, l, kv] = staging (block-first) or pool[l, kv, ids] =
    staging (layer-first), and the reverse; nothing else may change."""
    L, N, n, chunk = 3, 11, 6, 40
    rng = np.random.default_rng(kv_dim + (7 if cpu_layout == "BLOCKFIRST" else 0))
    shape = (N, L, kv_dim, chunk) if cpu_layout == "BLOCKFIRST" else (L, kv_dim, N, chunk)
    pool = rng.integers(0, 256, shape, dtype=np.uint8)
    s = pool.strides
    cbs, cls, cks = (s[0], s[1], s[2]) if cpu_layout == "BLOCKFIRST" else (s[2], s[0], s[1])
    ids = rng.permutation(N)[:n]
    for l in range(L):
        for kv in range(kv_dim):
            staging = rng.integers(0, 256, (n, chunk), dtype=np.uint8)
            want = pool.copy()
            if cpu_layout == "BLOCKFIRST":
                want[ids, l, kv] = staging
            else:
                want[l, kv, ids] = staging
            O.host_scatter(staging, pool.reshape(-1), ids, cbs, 0, chunk, l, kv, cks, cls, True)
            assert np.array_equal(pool, want), (l, kv)
            back = np.zeros_like(staging)
            O.host_scatter(back, pool.reshape(-1), ids, cbs, 0, chunk, l, kv, cks, cls, False)
            assert np.array_equal(back, staging), (l, kv)
    # an in-chunk offset with a shorter row moves that byte range of every chunk only
    staging = rng.integers(0, 256, (n, 8), dtype=np.uint8)
    want = pool.copy()
    if cpu_layout == "BLOCKFIRST":
        want[ids, 1, 0, 16:24] = staging
    else:
        want[1, 0, ids, 16:24] = staging
    O.host_scatter(staging, pool.reshape(-1), ids, cbs, 16, 8, 1, 0, cks, cls, True)
    assert np.array_equal(pool, want)


def test_is_full_block_on_the_shapes_the_reference_names():
    """csrc/transfer.cu:219-220: a call is a full block when the layers, K/V planes and
    chunk bytes it moves fill one block-first host block.  The reference's comment and
    its test predictor (tests/test_kv_transfer_correctness.py:1292-1300) name the
    shapes: rank0_only / all_write move all layers of the whole chunk -> full;
    layer_parallel moves a slice of the layers and a sharded put a slice of every
    chunk -> not full.  The per-rank shapes come from the rank plan (pinned by its own
    partition properties), the host block from the layout's closed form."""
    L, N, T, H, D, es = 6, 16, 8, 1, 64, 2
    for kv_dim in (1, 2):
        lay = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, N, T, H, D, kv_dim=kv_dim)
        chunk, cbs = lay.get_chunk_size() * es, lay.get_block_stride() * es
        assert cbs == torch.empty(lay.kv_shape, dtype=torch.int16).stride()[0] * es
        for n in (1, 2, 4):
            for mode, want_full in (("rank0_only", True), ("all_write", True),
                                    ("layer_parallel", n == 1), ("sharded", n == 1)):
                for rank in range(n):
                    p = O.tp_rank_plan(rank, n, 1, False, mode, 0, 0, 0, L, 4, chunk, cbs, cbs // n)
                    if not p.active:
                        continue
                    got = O.is_full_block(p.num_layers, kv_dim, p.chunk_size, cbs)
                    assert got == want_full, (kv_dim, n, mode, rank)
        # a host block with padding behind the layers is never full
        assert not O.is_full_block(L, kv_dim, chunk, cbs + 64)
        assert not O.is_full_block(L - 1, kv_dim, chunk, cbs)


def test_eventfd_index_enumerates_the_table():
    """csrc/layerwise.cpp:15-34, 537-544: the eventfd of (counter, tp_rank, layer) in the
    flat table the engine hands over as [num_counters, tp_size, num_layers]
    (flexkv/integration/sglang/comm.py:771 builds it with three counters)."""
    for tp, L in ((1, 5), (2, 6), (8, 61)):
        table = np.arange(3 * tp * L).reshape(3, tp, L)
        seen = set()
        for c in range(3):
            for r in range(tp):
                for l in range(L):
                    i = O.eventfd_index(c, r, l, tp, L)
                    assert table[c, r, l] == i
                    seen.add(i)
        assert seen == set(range(3 * tp * L))
