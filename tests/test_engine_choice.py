"""Per-transfer choice between the gather/scatter kernel and the copy engine
(use_ce_transfer == 2): a pure cost model, checked here on the benchmark
configurations' shapes without a GPU."""
import ctypes

import numpy as np

from flexkv_amd import _lib

L = _lib.load()


def choose(backend, n_layers, kv_dim, chunk, gpu_strides, cpu_strides, gids, cids, h2d,
           blockfirst=True, heads=8, memcpy2d=False, num_ptrs=None):
    g = np.ascontiguousarray(gids, dtype=np.int64)
    c = np.ascontiguousarray(cids, dtype=np.int64)
    ptrs = np.full(num_ptrs or max(1, 2 * n_layers), 1 << 40, dtype=np.uint64)
    d = _lib.TransferDesc()
    d.backend, d.num_layers_total = backend, n_layers
    d.gpu_tensor_ptrs, d.num_gpu_tensor_ptrs, d.device = ptrs.ctypes.data, ptrs.size, -1
    d.gpu_kv_stride, d.gpu_block_stride, d.gpu_layer_stride = gpu_strides
    d.cpu_ptr = 1 << 41
    d.cpu_kv_stride, d.cpu_layer_stride, d.cpu_block_stride = cpu_strides
    d.chunk_size, d.start_layer_id, d.num_layers, d.kv_dim = chunk, 0, n_layers, kv_dim
    d.num_blocks, d.gpu_block_ids, d.cpu_block_ids = g.size, g.ctypes.data, c.ctypes.data
    d.is_host_to_device, d.use_ce_transfer = int(h2d), 2
    d.ce = _lib.default_ce_config()
    d.ce.is_blockfirst, d.ce.num_kv_heads, d.ce.enable_memcpy2d = int(blockfirst), heads, int(memcpy2d)
    use_ce, tk, tc = ctypes.c_int32(-1), ctypes.c_double(), ctypes.c_double()
    _lib.check(L.fkv_choose_engine(ctypes.byref(d), ctypes.byref(use_ce), ctypes.byref(tk),
                                   ctypes.byref(tc)))
    return bool(use_ce.value), tk.value, tc.value


def test_llama_vllm_random_blocks_take_the_kernel():
    """256 scattered 2 MiB host blocks: 256 DMAs + a compaction pass lose ~6 % to
    the kernel (measured 50-54 vs 56.7-57.2 GB/s)."""
    rng = np.random.default_rng(1)
    ch = 32768
    for h2d in (False, True):
        ce, tk, tc = choose(0, 32, 2, ch, (4096 * ch, ch, 2 * 4096 * ch), (ch, 2 * ch, 64 * ch),
                            rng.permutation(4096)[:256], rng.permutation(1024)[:256], h2d)
        assert not ce and tc > 1.03 * tk
        assert 9.0 < tk < 10.0            # 512 MiB at the link rate is 9.4 ms


def test_block_major_engine_tensor_takes_the_copy_engine():
    """TRT-LLM layout: a block is one 5 MiB run on both sides -> 2048 plain DMAs."""
    rng = np.random.default_rng(2)
    ch, L_ = 32768, 80
    blk = L_ * 2 * ch
    ce, tk, tc = choose(1, L_, 2, ch, (ch, blk, 2 * ch), (ch, 2 * ch, blk),
                        rng.permutation(4096)[:2048], np.arange(2048), False, num_ptrs=1)
    assert ce and tc <= 1.03 * tk


def test_pages_into_adjacent_host_blocks_take_the_copy_engine():
    """SGLang pages (c1): 1024 scattered pages of 128 KiB x 64 (layer, kv) into host blocks
    0..1023.  GATHER_DIRECT stages them in two alternating buffers, so only the first
    group's compaction is exposed and the copies are sixteen of 512 MiB: within 3 % of the
    kernel (measured 56.6 against 57.0 / 57.6 GB/s), which leaves the compute units free."""
    rng = np.random.default_rng(4)
    ch, n = 131072, 4096
    for h2d in (False, True):
        ce, tk, tc = choose(2, 32, 2, ch, (0, ch, n * ch), (ch, 2 * ch, 64 * ch),
                            rng.permutation(n)[:1024], np.arange(1024), h2d, num_ptrs=64)
        assert ce and tc <= 1.03 * tk
        assert tc - 8 * 2**30 / 57.2e6 < 1.0       # ms beyond the bytes: one group's compaction, not eight
    # the same pages into scattered host blocks: 1024 copies of 8 MiB and every group's
    # compaction on the critical path
    ce, tk, tc = choose(2, 32, 2, ch, (0, ch, n * ch), (ch, 2 * ch, 64 * ch),
                        rng.permutation(n)[:1024], rng.permutation(4096)[:1024] * 2, False, num_ptrs=64)
    assert tc - 8 * 2**30 / 57.2e6 > 3.0


def test_one_contiguous_run_takes_the_copy_engine():
    ch = 73728
    # layer-first host, packed KV: 61 linear copies of 512 adjacent blocks
    ce, tk, tc = choose(0, 61, 1, ch, (16384 * ch, ch, 16384 * ch), (512 * ch, 512 * ch, ch),
                        np.arange(100, 612), np.arange(512), True, blockfirst=False, heads=1)
    assert ce


def test_per_block_copies_of_small_chunks_never_win():
    rng = np.random.default_rng(3)
    ch = 32768
    d_kw = dict(backend=0, n_layers=32, kv_dim=2, chunk=ch,
                gpu_strides=(4096 * ch, ch, 2 * 4096 * ch), cpu_strides=(1024 * ch, 2 * 1024 * ch, ch),
                gids=rng.permutation(4096)[:256], cids=rng.permutation(1024)[:256], h2d=True,
                blockfirst=False)
    ce, tk, tc = choose(**d_kw)
    assert not ce and tc > 2 * tk      # layer-first host + scattered ids: staging through the host


def test_empty_transfer_and_bad_descriptor():
    none = np.empty(0, dtype=np.int64)
    ce, tk, tc = choose(0, 4, 2, 64, (64, 64, 128), (64, 128, 512), none, none, True)
    assert (ce, tk, tc) == (False, 0.0, 0.0)
    d = _lib.TransferDesc()
    d.backend = 9
    out = ctypes.c_int32()
    assert L.fkv_choose_engine(ctypes.byref(d), ctypes.byref(out), None, None) == _lib.FKV_ERR_RUNTIME


# ---- the model's link figures follow the device --------------------------------

def table_of_device_0():
    p = _lib.LaunchPolicy()
    _lib.check(L.fkv_launch_policy_get(0, ctypes.byref(p)))   # no GPU: the table of a device of unknown shape
    return p


def seeded(p, d2h, h2d, overhead_us):
    out = _lib.LaunchPolicy()
    _lib.check(L.fkv_launch_policy_seeded(ctypes.byref(p), d2h, h2d, overhead_us, ctypes.byref(out)))
    return out


def test_link_figures_are_rebased_on_a_measurement():
    p = table_of_device_0()
    assert (p.model_link_mbps, p.model_kernel_d2h_mbps, p.model_kernel_h2d_mbps) == (57200, 57000, 57200)
    assert (p.link_gbps_estimate, p.staged_copy_overhead_us, p.model_seed, p.model_seeded) == (45, 10, 1, 0)
    q = seeded(p, 28.0, 29.0, 14.2)             # a Gen4 slot, slower copy commands
    assert (q.model_link_mbps, q.model_kernel_d2h_mbps, q.model_kernel_h2d_mbps) == (28500, 28000, 29000)
    assert q.link_gbps_estimate == 22           # the same 79 % of the link other processes are told
    assert (q.staged_copy_overhead_us, q.model_seeded) == (14, 1)
    # everything that does not depend on the link is untouched
    for f in ("model_dma_ns", "model_compaction_gbps", "model_host_pass_mbps", "model_launch_ns",
              "model_gather_thread_mbps", "staged_overhead_pct", "gather_threads", "h2d_wg_per_cta"):
        assert getattr(q, f) == getattr(p, f), f
    # a figure the caller (or the environment) has set stays
    p.model_link_mbps, p.staged_copy_overhead_us = 50000, 3
    q = seeded(p, 28.0, 29.0, 14.2)
    assert (q.model_link_mbps, q.staged_copy_overhead_us, q.model_kernel_h2d_mbps) == (50000, 3, 29000)
    # a measurement that cannot be right changes nothing
    p = table_of_device_0()
    q = seeded(p, 0.0, 29.0, 14.2)
    assert (q.model_link_mbps, q.model_kernel_h2d_mbps, q.model_seeded) == (57200, 57200, 0)
    q = seeded(p, 28.0, 29.0, 0.0)              # rates without a copy-command figure
    assert (q.model_link_mbps, q.staged_copy_overhead_us, q.model_seeded) == (28500, 10, 1)


def test_the_engine_choice_moves_with_the_link_figure():
    """Fixed costs (copy commands, the compaction pass) weigh half as much on a link half
    as fast: a transfer the kernel wins by 5 % at 57 GB/s goes to the copy engine at
    28.5 GB/s, and what the copy engine costs beyond the bytes stays the same."""
    rng = np.random.default_rng(11)
    ch = 65536                                   # 4 MiB host blocks: 256 copy commands of 4 MiB
    args = (0, 32, 2, ch, (4096 * ch, ch, 2 * 4096 * ch), (ch, 2 * ch, 64 * ch),
            rng.permutation(4096)[:256], rng.permutation(1024)[:256], True)
    nbytes = 256 * 64 * ch
    p = table_of_device_0()
    try:
        ce, tk, tc = choose(*args)
        assert not ce and 1.03 * tk < tc < 1.08 * tk
        extra = tc - nbytes / 57.2e6
        half = seeded(p, 28.5, 28.6, 10.0)
        _lib.check(L.fkv_launch_policy_set(0, ctypes.byref(half)))
        ce2, tk2, tc2 = choose(*args)
        assert ce2 and tc2 <= 1.03 * tk2
        assert abs(tk2 - 2 * tk) < 0.02 * tk2
        assert abs((tc2 - nbytes / 28.55e6) - extra) < 0.05 * extra
    finally:
        _lib.check(L.fkv_launch_policy_reset(0))
