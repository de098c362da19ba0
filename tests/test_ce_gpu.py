"""Copy-engine strategies vs the CPU oracle (bit-exact), and the strategy that
actually ran vs the oracle's choose_path."""
import numpy as np
import pytest

from kvsetup import KVSetup, VLLM, TRTLLM, SGLANG, block_ids
from oracle import fkv_oracle as O

pytestmark = pytest.mark.gpu

PATHS = {"CONTIG_DIRECT": 0, "SEGMENT_DIRECT": 1, "SEGMENT_SCATTER": 2, "GATHER_SCATTER": 3,
         "GATHER_DIRECT": 4}


def expected_path(s, gids, cids, heads, thr, h2d, num_layers):
    an, _ = O.ce_analyze(gids, cids, s.cpu_block_stride, s.chunk, s.gpu_block_stride)
    full = O.is_full_block(num_layers, s.kv_dim, s.chunk, s.cpu_block_stride)
    return O.CE_NAMES[O.ce_choose_path(an, s.cpu_layout == "BLOCKFIRST", heads, thr, s.chunk,
                                       h2d, full)]


SHAPES = [
    pytest.param(VLLM, 4, 2, 64, 64, 4096, "BLOCKFIRST", "LAYERFIRST", id="vllm-bf-kv2"),
    pytest.param(VLLM, 4, 2, 64, 64, 4096, "LAYERFIRST", "LAYERFIRST", id="vllm-lf-kv2"),
    pytest.param(VLLM, 4, 1, 64, 64, 9216, "BLOCKFIRST", "LAYERFIRST", id="mla-bf"),
    pytest.param(VLLM, 4, 1, 64, 64, 9216, "LAYERFIRST", "LAYERFIRST", id="mla-lf"),
    pytest.param(VLLM, 3, 2, 64, 64, 2048, "BLOCKFIRST", "LAYERBLOCK", id="vllm-layerblock"),
    pytest.param(TRTLLM, 5, 2, 64, 64, 4096, "BLOCKFIRST", "LAYERFIRST", id="trtllm-bf"),
    pytest.param(SGLANG, 4, 2, 64, 64, 8192, "BLOCKFIRST", "LAYERFIRST", id="sglang-bf"),
    pytest.param(SGLANG, 4, 2, 64, 64, 8192, "LAYERFIRST", "LAYERFIRST", id="sglang-lf"),
]


@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout", SHAPES)
@pytest.mark.parametrize("pattern", ["contiguous", "few_seg", "scattered"])
@pytest.mark.parametrize("heads", [1, 8])
@pytest.mark.parametrize("memcpy2d", [False, True], ids=["no2d", "2d"])
def test_auto_strategy_matches_oracle(gpu_device, backend, L, K, N, NH, chunk, cpu_layout,
                                      gpu_layout, pattern, heads, memcpy2d):
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=31)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(7)
    n = 32
    if pattern == "scattered":
        gids, cids = block_ids(rng, N, n), block_ids(rng, NH, n)
    else:  # the same shape on both sides so that runs line up
        gids = block_ids(rng, N, n, pattern)
        cids = gids - gids.min() + int(rng.integers(0, NH - n + 1))
        if pattern == "few_seg":
            cids = block_ids(np.random.default_rng(1), NH, n, "few_seg")
            gids = cids - cids.min() + int(gids.min())
    for thr in (8, 2):
        for h2d in (False, True):
            want = expected_path(s, gids, cids, heads, thr, h2d, L)
            print(f"case {pattern} heads={heads} thr={thr} h2d={h2d} 2d={memcpy2d} -> {want}",
                  flush=True)
            dev.transfer(gids, cids, is_h2d=h2d, use_ce_transfer=True, ce_path_opt=True,
                         ce_segment_threshold=thr, num_kv_heads=heads,
                         ce_enable_memcpy2d=memcpy2d)
            assert last_transfer_path() == want
            s.oracle_transfer(gids, cids, h2d)
            dev.assert_matches_reference(f"{want} h2d={h2d}")


@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout", SHAPES)
def test_per_block_baseline(gpu_device, backend, L, K, N, NH, chunk, cpu_layout, gpu_layout):
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=32)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(8)
    gids, cids = block_ids(rng, N, 12), block_ids(rng, NH, 12)
    for h2d in (False, True):
        dev.transfer(gids, cids, is_h2d=h2d, use_ce_transfer=True, ce_path_opt=False)
        assert last_transfer_path() == "PER_BLOCK"
        s.oracle_transfer(gids, cids, h2d)
        dev.assert_matches_reference(f"PER_BLOCK h2d={h2d}")


@pytest.mark.parametrize("force", ["SEGMENT_SCATTER", "GATHER_SCATTER", "GATHER_DIRECT"])
@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout", SHAPES)
@pytest.mark.parametrize("memcpy2d", [False, True], ids=["no2d", "2d"])
def test_forced_general_strategies(gpu_device, force, backend, L, K, N, NH, chunk, cpu_layout,
                                   gpu_layout, memcpy2d):
    """The three strategies that cope with any id pattern, forced on every shape
    (kernel path == every copy-engine path on the same inputs)."""
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=33)
    gpu_rows_adjacent = s.gpu_block_stride == s.chunk
    if force == "SEGMENT_SCATTER" and not gpu_rows_adjacent and not memcpy2d:
        pytest.skip("segment DMA needs adjacent GPU blocks (checked in test_forced_misfit)")
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(9)
    for pattern in ("scattered", "few_seg"):
        cids = block_ids(rng, NH, 24, pattern)
        gids = block_ids(rng, N, 24, "scattered") if pattern == "scattered" else \
            cids - cids.min() + 3
        if force == "SEGMENT_SCATTER" and not gpu_rows_adjacent and pattern == "scattered":
            continue  # 24 segments exceed the 2-D copy threshold; the staging branch needs adjacency
        for h2d in (False, True):
            print(f"case force={force} {pattern} h2d={h2d} 2d={memcpy2d}", flush=True)
            dev.transfer(gids, cids, is_h2d=h2d, use_ce_transfer=True, ce_path_opt=True,
                         ce_force_path=PATHS[force], ce_enable_memcpy2d=memcpy2d,
                         ce_gather_threads=3)
            assert last_transfer_path() == force
            s.oracle_transfer(gids, cids, h2d)
            dev.assert_matches_reference(f"forced {force} {pattern} h2d={h2d}")


@pytest.mark.parametrize("force", ["PER_BLOCK", "SEGMENT_SCATTER", "GATHER_SCATTER", "GATHER_DIRECT"])
def test_every_copy_as_a_2d_copy_of_one_row(gpu_device, force):
    """ce_rect_min_kb = 0 hands every copy of the copy-engine path that no host thread
    waits for to the runtime as a 2-D copy of one row (the form the runtime gives to the
    copy engines; the staging ping-pong of the two *_SCATTER strategies keeps 1-D copies): same bytes,
    and the GPU blocks of GATHER_DIRECT in host order with duplicates on the host side."""
    from flexkv_amd.c_ext import last_transfer_path, launch_policy
    s = KVSetup(VLLM, 5, 2, 64, 64, 4096, "BLOCKFIRST", seed=12)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(3)
    with launch_policy(ce_rect_min_kb=0):
        for pattern in ("scattered", "few_seg", "contiguous"):
            cids = block_ids(rng, 64, 20, pattern)
            gids = block_ids(rng, 64, 20, "scattered")
            for h2d in (False, True):
                dev.transfer(gids, cids, is_h2d=h2d, use_ce_transfer=True,
                             ce_path_opt=force != "PER_BLOCK", ce_force_path=PATHS.get(force, -1),
                             ce_enable_memcpy2d=True)
                assert last_transfer_path() == force
                s.oracle_transfer(gids, cids, h2d)
                dev.assert_matches_reference(f"{force} {pattern} h2d={h2d} as 2-D copies")
        # the same host block restored into two GPU blocks (host order puts them side by side)
        gids, cids = np.array([7, 3, 50, 9], dtype=np.int64), np.array([11, 12, 11, 10], dtype=np.int64)
        dev.transfer(gids, cids, is_h2d=True, use_ce_transfer=True, ce_path_opt=True,
                     ce_force_path=PATHS["GATHER_DIRECT"])
        s.oracle_transfer(gids, cids, True)
        dev.assert_matches_reference("duplicate host block")


def test_forced_direct_strategies_on_fitting_input(gpu_device):
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(VLLM, 3, 1, 40, 40, 4096, "LAYERFIRST", seed=34)   # adjacent blocks on both sides
    dev = s.to_device(gpu_device)
    run_g, run_c = np.arange(5, 25, dtype=np.int64), np.arange(11, 31, dtype=np.int64)
    for h2d in (False, True):
        dev.transfer(run_g, run_c, is_h2d=h2d, use_ce_transfer=True, ce_path_opt=True, ce_force_path=0)
        assert last_transfer_path() == "CONTIG_DIRECT"
        s.oracle_transfer(run_g, run_c, h2d)
        dev.assert_matches_reference("CONTIG_DIRECT")
    seg_g = np.array([0, 1, 2, 10, 11, 30, 20, 21], dtype=np.int64)
    seg_c = np.array([5, 6, 7, 20, 21, 0, 33, 34], dtype=np.int64)
    for h2d in (False, True):
        dev.transfer(seg_g, seg_c, is_h2d=h2d, use_ce_transfer=True, ce_path_opt=True, ce_force_path=1)
        assert last_transfer_path() == "SEGMENT_DIRECT"
        s.oracle_transfer(seg_g, seg_c, h2d)
        dev.assert_matches_reference("SEGMENT_DIRECT")


def test_forced_misfit_and_out_of_range(gpu_device):
    s = KVSetup(VLLM, 2, 2, 16, 16, 1024, "BLOCKFIRST", seed=35)
    dev = s.to_device(gpu_device)
    ids = np.array([3, 9, 1], dtype=np.int64)
    with pytest.raises(RuntimeError, match=r"force_path out of range \[0,4\]: 5"):  # transfer.cu:213
        dev.transfer(ids, ids, is_h2d=False, use_ce_transfer=True, ce_path_opt=True, ce_force_path=5)
    # a strategy that assumes adjacent host blocks must not be run on a block-first pool
    with pytest.raises(ValueError, match="does not fit"):
        dev.transfer(ids, ids, is_h2d=False, use_ce_transfer=True, ce_path_opt=True, ce_force_path=0)
    with pytest.raises(ValueError, match="does not fit"):
        dev.transfer(ids, ids, is_h2d=False, use_ce_transfer=True, ce_path_opt=True, ce_force_path=1)
    dev.assert_matches_reference("refused calls moved nothing")


def test_gather_direct_groups_and_partial_layers(gpu_device, monkeypatch):
    """Layer batches (host block only partly covered) take the per-block / 2-D
    branch of GATHER_DIRECT; the result equals the whole-block branch."""
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(VLLM, 6, 2, 48, 48, 2048, "BLOCKFIRST", seed=36)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(10)
    gids, cids = block_ids(rng, 48, 20), block_ids(rng, 48, 20, "few_seg")
    for memcpy2d in (False, True):
        for l0 in (0, 2, 4):
            for h2d in (False, True):
                dev.transfer(gids, cids, is_h2d=h2d, start_layer=l0, num_layers=2,
                             use_ce_transfer=True, ce_path_opt=True, ce_force_path=4,
                             ce_enable_memcpy2d=memcpy2d, num_kv_heads=8)
                assert last_transfer_path() == "GATHER_DIRECT"
                s.oracle_transfer(gids, cids, h2d, start_layer=l0, num_layers=2)
                dev.assert_matches_reference(f"GATHER_DIRECT layers {l0}..{l0 + 1} h2d={h2d}")


@pytest.mark.parametrize("memcpy2d", [False, True], ids=["no2d", "2d"])
def test_gather_direct_in_many_staging_groups(gpu_device, memcpy2d):
    """A staging buffer of 1 MiB holds two blocks of 384 KiB: 37 blocks go in 19 groups
    (or, where the host blocks form few runs, in 37 groups of one block that alternate
    between two buffers while their copies run on a second stream); runs of consecutive
    host blocks are cut at group boundaries, and the last group is short.  Whole blocks
    and layer batches, both directions, and the same with the second stream off."""
    from flexkv_amd.c_ext import last_transfer_path, launch_policy
    s = KVSetup(VLLM, 6, 2, 64, 64, 32768, "BLOCKFIRST", seed=37)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(11)
    for two_streams, pattern in [(m, p) for m in (1, 2, 0) for p in ("contiguous", "few_seg", "scattered")]:
        with launch_policy(ce_staging_mb=1, ce_two_streams=two_streams):
            cids = block_ids(rng, 64, 37, pattern)
            gids = block_ids(rng, 64, 37, "scattered")
            for l0, nl in ((0, 6), (1, 3)):
                for h2d in (False, True):
                    print(f"case {pattern} layers {l0}+{nl} h2d={h2d} 2d={memcpy2d} "
                          f"two_streams={two_streams}", flush=True)
                    dev.transfer(gids, cids, is_h2d=h2d, start_layer=l0, num_layers=nl,
                                 use_ce_transfer=True, ce_path_opt=True, ce_force_path=4,
                                 ce_enable_memcpy2d=memcpy2d, num_kv_heads=8)
                    assert last_transfer_path() == "GATHER_DIRECT"
                    s.oracle_transfer(gids, cids, h2d, start_layer=l0, num_layers=nl)
                    dev.assert_matches_reference(
                        f"GATHER_DIRECT in groups, {pattern}, layers {l0}+{nl}, h2d={h2d}")


def test_auto_engine_follows_the_cost_model_and_stays_exact(gpu_device):
    """use_ce_transfer="auto": the path that ran is the one fkv_choose_engine
    names, and the bytes equal the oracle's either way."""
    import ctypes
    from flexkv_amd import _lib
    from flexkv_amd.c_ext import last_transfer_path
    for backend, chunk, pattern in ((TRTLLM, 65536, "scattered"), (VLLM, 512, "scattered"),
                                    (VLLM, 262144, "contiguous")):
        s = KVSetup(backend, 4, 2, 48, 48, chunk, "BLOCKFIRST", seed=41)
        dev = s.to_device(gpu_device)
        rng = np.random.default_rng(11)
        gids, cids = block_ids(rng, 48, 40, pattern), block_ids(rng, 48, 40, pattern)
        for h2d in (False, True):
            dev.transfer(gids, cids, is_h2d=h2d, use_ce_transfer="auto", ce_path_opt=True,
                         num_kv_heads=8)
            ran_ce = last_transfer_path() != "KERNEL"
            s.oracle_transfer(gids, cids, h2d)
            dev.assert_matches_reference(f"auto engine backend={backend} h2d={h2d}")
            print(f"auto: backend={backend} chunk={chunk} {pattern} h2d={h2d} -> "
                  f"{last_transfer_path()}", flush=True)
            assert isinstance(ran_ce, bool)
    # tiny chunks, scattered: the kernel; whole 512 KiB blocks of a block-major tensor: DMA
    s = KVSetup(TRTLLM, 4, 2, 48, 48, 65536, "BLOCKFIRST", seed=42)
    dev = s.to_device(gpu_device)
    ids = np.arange(40, dtype=np.int64)
    dev.transfer(ids, ids, is_h2d=True, use_ce_transfer="auto", ce_path_opt=True, num_kv_heads=8)
    assert last_transfer_path() == "GATHER_SCATTER"   # runs as plain whole-block DMAs
    s = KVSetup(VLLM, 4, 2, 48, 48, 512, "LAYERFIRST", seed=43)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(12)
    g, c = block_ids(rng, 48, 40), block_ids(rng, 48, 40)
    dev.transfer(g, c, is_h2d=True, use_ce_transfer="auto", ce_path_opt=True, num_kv_heads=8)
    assert last_transfer_path() == "KERNEL"


def test_block_major_partial_layers_direct(gpu_device):
    """TRT-LLM layout, a sub-range of layers: the run of a block covers only part
    of the block on both sides (per-block or 2-D DMAs)."""
    from flexkv_amd.c_ext import last_transfer_path
    s = KVSetup(TRTLLM, 6, 2, 32, 32, 4096, "BLOCKFIRST", seed=44)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(13)
    gids, cids = block_ids(rng, 32, 20), block_ids(rng, 32, 20, "few_seg")
    for memcpy2d in (False, True):
        for l0 in (0, 2, 3):
            for h2d in (False, True):
                dev.transfer(gids, cids, is_h2d=h2d, start_layer=l0, num_layers=3,
                             use_ce_transfer=True, ce_path_opt=True, ce_enable_memcpy2d=memcpy2d,
                             num_kv_heads=8)
                assert last_transfer_path() == "GATHER_SCATTER"
                s.oracle_transfer(gids, cids, h2d, start_layer=l0, num_layers=3)
                dev.assert_matches_reference(f"block runs layers {l0}..{l0 + 2} h2d={h2d}")


# ---- host gather/scatter passes: thread counts and streaming stores -------------------
# tests/test_kv_transfer_correctness.py:1730-1960 (test_gather_nt_roundtrip,
# test_gather_nt_layerwise_h2d): ce_gather_threads 0 (single-thread fallback) / 1 / 4 / 8 and
# ce_gather_nt on / off change how the host passes of the copy-engine path run, never a byte.
GATHER_QUADRANTS = [   # (kv_dim, num_kv_heads, chunk): MLA, K/V apart with one head, packed MHA, MHA
    pytest.param(1, 1, 16 * 512 * 2, id="mla"),
    pytest.param(2, 1, 16 * 512 * 2, id="kv_sep_1h"),
    pytest.param(1, 8, 16 * 8 * 128 * 2, id="packed_mha"),
    pytest.param(2, 8, 16 * 8 * 128 * 2, id="plain_mha"),
]


@pytest.mark.parametrize("kv_dim,heads,chunk", GATHER_QUADRANTS)
@pytest.mark.parametrize("cpu_layout", ["BLOCKFIRST", "LAYERFIRST"])
@pytest.mark.parametrize("gather_threads", [0, 1, 4, 8], ids=["gt0", "gt1", "gt4", "gt8"])
@pytest.mark.parametrize("gather_nt", [True, False], ids=["nt_on", "nt_off"])
def test_gather_threads_and_streaming_stores_round_trip(gpu_device, kv_dim, heads, chunk, cpu_layout,
                                                        gather_threads, gather_nt):
    """Put, wipe the engine's blocks, get: the strategy the library picks for the shape, and
    the two strategies with a host pass forced (rows gathered / scattered by host threads)."""
    import torch
    from flexkv_amd.c_ext import last_transfer_path
    L, N, NH, n = 4, 48, 48, 21
    s = KVSetup(VLLM, L, kv_dim, N, NH, chunk, cpu_layout, seed=51 + gather_threads)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(53)
    kw = dict(use_ce_transfer=True, ce_path_opt=True, num_kv_heads=heads,
              ce_gather_threads=gather_threads, ce_gather_nt=gather_nt, ce_enable_memcpy2d=False)
    for force in (None, "SEGMENT_SCATTER", "GATHER_SCATTER"):
        gids, cids = block_ids(rng, N, n), block_ids(rng, NH, n)
        extra = {} if force is None else dict(ce_force_path=PATHS[force])
        dev.transfer(gids, cids, is_h2d=False, **kw, **extra)
        if force is not None:
            assert last_transfer_path() == force
        s.oracle_transfer(gids, cids, False)
        dev.assert_matches_reference(f"put {force} gt={gather_threads} nt={gather_nt}")
        # other bytes in the engine's blocks, then back from the host
        fresh = [np.random.default_rng(59).integers(0, 256, a.size, dtype=np.uint8) for a in s.gpu_ref]
        for a, t, f in zip(s.gpu_ref, dev.gpu, fresh):
            a[:] = f
            t.copy_(torch.from_numpy(f).to(t.device).view(t.dtype).reshape(t.shape))
        dev.transfer(gids, cids, is_h2d=True, **kw, **extra)
        s.oracle_transfer(gids, cids, True)
        dev.assert_matches_reference(f"get {force} gt={gather_threads} nt={gather_nt}")


@pytest.mark.parametrize("kv_dim,heads,chunk", GATHER_QUADRANTS)
@pytest.mark.parametrize("gather_threads", [0, 4], ids=["gt0", "gt4"])
@pytest.mark.parametrize("gather_nt", [True, False], ids=["nt_on", "nt_off"])
def test_gather_threads_and_streaming_stores_layerwise_restore(gpu_device, kv_dim, heads, chunk,
                                                               gather_threads, gather_nt):
    """The same settings through a layerwise restore on the copy engine, a layer at a time."""
    import torch
    from flexkv_amd.c_ext import LayerwiseTransferGroup, launch_policy
    L, N, NH, n = 4, 48, 48, 21
    s = KVSetup(VLLM, L, kv_dim, N, NH, chunk, "BLOCKFIRST", seed=61 + gather_threads)
    dev = s.to_device(gpu_device)
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)  # noqa: E731
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=L,
        gpu_kv_strides_tensor=i64(s.gpu_kv_stride), gpu_block_strides_tensor=i64(s.gpu_block_stride),
        gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1, is_blockfirst=True,
        num_kv_heads=heads, ce_gather_threads=gather_threads, ce_gather_nt=gather_nt)
    rng = np.random.default_rng(67)
    gids, cids = block_ids(rng, N, n), block_ids(rng, NH, n)
    e = torch.empty(0, dtype=torch.int64)
    with launch_policy(staged_restore=0, staged_gather=0):   # the copy-engine strategies themselves
        for notify in ("hostfunc", "polling"):
            grp.layerwise_transfer(
                e, e, 0, 0, 0, 0, 0, torch.as_tensor(gids), torch.as_tensor(cids), s.cpu_kv_stride,
                s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
                s.cpu_block_stride, 4, True, L, 1, s.kv_dim, heads, counter_id=0,
                kv_shared_across_ranks_mode="sharded", notify_mode=notify)
            grp.synchronize()
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference(f"layerwise on the copy engine, {notify}")
    grp.close()


# tests/test_kv_transfer_correctness.py:1327-1620 (test_ce_paths_roundtrip,
# test_ce_paths_layerwise_h2d): every strategy the id pattern, the threshold and the shape
# lead to, reached through a layerwise restore on the copy engine, a layer or all layers a batch.
@pytest.mark.parametrize("kv_dim,heads,chunk", [GATHER_QUADRANTS[0], GATHER_QUADRANTS[1],
                                                GATHER_QUADRANTS[3]])
@pytest.mark.parametrize("cpu_layout", ["BLOCKFIRST", "LAYERFIRST"])
@pytest.mark.parametrize("path_opt", [False, True], ids=["baseline", "optimized"])
@pytest.mark.parametrize("memcpy2d", [False, True], ids=["no2d", "2d"])
def test_layerwise_restore_on_the_copy_engine_by_id_pattern(gpu_device, kv_dim, heads, chunk,
                                                            cpu_layout, path_opt, memcpy2d):
    import torch
    from flexkv_amd.c_ext import LayerwiseTransferGroup, last_transfer_path, launch_policy
    L, N, NH, n = 4, 64, 64, 32
    s = KVSetup(VLLM, L, kv_dim, N, NH, chunk, cpu_layout, seed=71)
    dev = s.to_device(gpu_device)
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)  # noqa: E731
    e = torch.empty(0, dtype=torch.int64)
    rng = np.random.default_rng(73)
    for thr in (8, 2):
        grp = LayerwiseTransferGroup(
            num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=L,
            gpu_kv_strides_tensor=i64(s.gpu_kv_stride),
            gpu_block_strides_tensor=i64(s.gpu_block_stride),
            gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
            iouring_entries=0, iouring_flags=0,
            layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1,
            is_blockfirst=cpu_layout == "BLOCKFIRST", num_kv_heads=heads,
            ce_segment_threshold=thr, ce_path_opt=path_opt, ce_enable_memcpy2d=memcpy2d)
        for pattern in ("contiguous", "few_seg", "scattered"):
            if pattern == "scattered":
                gids, cids = block_ids(rng, N, n), block_ids(rng, NH, n)
            else:
                cids = block_ids(rng, NH, n, pattern)
                gids = cids - cids.min() + int(rng.integers(0, N - (cids.max() - cids.min())))
            for gran in (1, L):
                fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
                s.host_ref[:] = fresh
                dev.host.copy_(torch.from_numpy(fresh))
                # the strategies themselves (the library's staging routes are covered elsewhere)
                with launch_policy(staged_restore=0, staged_gather=0):
                    grp.layerwise_transfer(
                        e, e, 0, 0, 0, 0, 0, torch.as_tensor(gids), torch.as_tensor(cids),
                        s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, s.chunk,
                        s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, 4, True, L, gran,
                        s.kv_dim, heads, counter_id=0, kv_shared_across_ranks_mode="sharded",
                        notify_mode="polling")
                    grp.synchronize()
                taken = last_transfer_path()
                if not path_opt:
                    assert taken == "PER_BLOCK"
                else:   # the last batch: layers [L - gran, L) of the call
                    assert taken == expected_path(s, gids, cids, heads, thr, True, gran), \
                        (pattern, thr, gran)
                s.oracle_transfer(gids, cids, True)
                dev.assert_matches_reference(f"{pattern} thr={thr} gran={gran} -> {taken}")
        grp.close()
