"""Copy-engine analysis and strategy choice: library (C ABI) vs oracle, both
vs definitions that do not restate their code."""
import ctypes

import numpy as np
import pytest

from flexkv_amd import _lib
from flexkv_amd.layout import KVCacheLayout, KVCacheLayoutType
from oracle import fkv_oracle as O

L = _lib.load()
NAMES = _lib.CE_PATH_NAMES


def lib_analyze(g, c, cbs, chunk, gbs):
    g = np.ascontiguousarray(g, dtype=np.int64)
    c = np.ascontiguousarray(c, dtype=np.int64)
    out = _lib.CEAnalysis()
    segs = (_lib.CESegment * max(1, g.size))()
    _lib.check(L.fkv_ce_analyze(g.ctypes.data, c.ctypes.data, g.size, cbs, chunk, gbs,
                                ctypes.byref(out), ctypes.cast(segs, ctypes.c_void_p),
                                max(1, g.size)))
    return out, [(segs[i].start_k, segs[i].nr_blocks) for i in range(out.num_segments)]


def lib_choose(an, blockfirst, heads, thr, chunk, h2d, full):
    cfg = _lib.default_ce_config()
    cfg.is_blockfirst, cfg.num_kv_heads, cfg.segment_threshold = int(blockfirst), heads, thr
    return int(L.fkv_ce_choose_path(ctypes.byref(an), ctypes.byref(cfg), chunk, int(h2d), int(full)))


def brute_segments(g, c):
    """Maximal runs in which BOTH id lists step by exactly +1."""
    n = len(g)
    cuts = [0] + [k for k in range(1, n) if not (g[k] == g[k - 1] + 1 and c[k] == c[k - 1] + 1)] + [n]
    return [(a, b - a) for a, b in zip(cuts[:-1], cuts[1:]) if b > a]


def test_segments_random_vs_brute_force_and_oracle():
    rng = np.random.default_rng(0)
    for trial in range(300):
        n = int(rng.integers(0, 40))
        # mixtures of runs and jumps on both sides
        g = np.cumsum(rng.choice([1, 1, 1, 2, -3, 7], size=n)).astype(np.int64) + 100
        c = np.cumsum(rng.choice([1, 1, 1, 1, 5, -2], size=n)).astype(np.int64) + 100
        chunk = 64
        cbs = int(rng.choice([64, 128]))
        gbs = int(rng.choice([0, 64, 256]))
        a, segs = lib_analyze(g, c, cbs, chunk, gbs)
        oa, osegs = O.ce_analyze(g, c, cbs, chunk, gbs)
        want = brute_segments(list(g), list(c)) if n else []
        assert segs == want == osegs
        assert a.num_segments == len(want) == oa.num_segments
        assert bool(a.gpu_log_contig) == all(g[k] == g[k - 1] + 1 for k in range(1, n))
        assert bool(a.cpu_log_contig) == all(c[k] == c[k - 1] + 1 for k in range(1, n))
        assert bool(a.cpu_phys_contig) == (cbs == chunk)
        assert bool(a.gpu_phys_contig) == (gbs in (0, chunk))
        for f in ("gpu_log_contig", "cpu_log_contig", "cpu_phys_contig", "gpu_phys_contig"):
            assert getattr(a, f) == getattr(oa, f)
        assert sum(nr for _, nr in segs) == n


def test_choose_path_library_equals_oracle_exhaustively():
    an = _lib.CEAnalysis()
    oan = O.Analysis()
    for bits in range(16):
        for nseg in (1, 4, 8, 9, 64):
            for bf in (0, 1):
                for heads in (1, 8):
                    for thr in (2, 8):
                        for chunk in (32768, 37440, 100):
                            for h2d in (0, 1):
                                for full in (0, 1):
                                    vals = [(bits >> i) & 1 for i in range(4)]
                                    for obj in (an, oan):
                                        (obj.gpu_log_contig, obj.cpu_log_contig,
                                         obj.cpu_phys_contig, obj.gpu_phys_contig) = vals
                                        obj.num_segments = nseg
                                    assert lib_choose(an, bf, heads, thr, chunk, h2d, full) == \
                                        O.ce_choose_path(oan, bf, heads, thr, chunk, h2d, full)


# ---- the strategy matrix of the reference's own test predictor ---------------
# Restated from tests/test_kv_transfer_correctness.py:1247-1317 in terms of the
# *names* of the block-id pattern, host layout and sharing mode (not of the
# analysis results), then compared with choose_path run on real ids and the real
# strides of those layouts.

def make_pattern(name, n):
    if name == "contiguous":
        return np.arange(n, dtype=np.int64)
    if name == "few_seg":
        q = n // 4
        b = np.arange(n, dtype=np.int64)
        return np.concatenate([b[0:q], b[2 * q:3 * q], b[q:2 * q], b[3 * q:4 * q]])
    # stand-in for torch.randperm(seed 42): any permutation without adjacent
    # ascending neighbours gives the same segment count (n)
    return np.concatenate([np.arange(1, n, 2), np.arange(0, n, 2)])[::-1].astype(np.int64).copy()


def predicted(pattern, cpu_layout, kv_dim, num_kv_heads, mode, h2d, n=64, thr=8):
    # The reference predictor also demands kv_dim == 1 here, reasoning that a
    # layer-first block stride is kv_dim * chunk; storage.py:222-234 gives
    # T*H*D == chunk for every kv_dim, so choose_path sees adjacent host blocks
    # for kv_dim == 2 as well.  (The predictor only feeds a coverage assert in
    # the reference and is never compared with the C++ choice.)
    dst_phys = cpu_layout == "LAYERFIRST"
    blockfirst = cpu_layout == "BLOCKFIRST"
    sharded_d2h = num_kv_heads == 1 and mode == "sharded" and not h2d
    src_phys = not sharded_d2h
    nseg = {"contiguous": 1, "few_seg": 4}.get(pattern, n)
    full_block = mode in ("rank0_only", "all_write")
    if not dst_phys and blockfirst and src_phys:
        if not h2d and num_kv_heads == 1 and not full_block:
            # the predictor returns SEGMENT_SCATTER here; choose_path first sends
            # more-than-threshold segment counts to GATHER_SCATTER
            # (csrc/ce_transfer.cu:80-84), which the reference's sweep never hits
            return "GATHER_SCATTER" if nseg > thr else "SEGMENT_SCATTER"
        if not h2d and num_kv_heads == 1 and nseg > thr:
            return "GATHER_SCATTER"
        return "GATHER_DIRECT"
    if pattern == "contiguous" and dst_phys and src_phys:
        return "CONTIG_DIRECT"
    if not src_phys:
        return "GATHER_SCATTER"
    if nseg <= thr:
        return "SEGMENT_DIRECT" if dst_phys else "SEGMENT_SCATTER"
    return "GATHER_SCATTER"


MODES = ["sharded", "all_write", "rank0_only", "layer_parallel", "rank_rotate"]


@pytest.mark.parametrize("pattern", ["contiguous", "few_seg", "scattered"])
@pytest.mark.parametrize("cpu_layout", ["LAYERFIRST", "BLOCKFIRST"])
@pytest.mark.parametrize("kv_dim,num_kv_heads", [(1, 1), (2, 1), (1, 8), (2, 8)])
@pytest.mark.parametrize("thr", [8, 2])
def test_strategy_matrix(pattern, cpu_layout, kv_dim, num_kv_heads, thr):
    Lyr, n, T, H, D, es, tp = 4, 64, 16, (1 if num_kv_heads == 1 else 8), 128, 2, 4
    ids = make_pattern(pattern, n)
    cpu = KVCacheLayout(KVCacheLayoutType[cpu_layout], Lyr, n, T, H, D, kv_dim=kv_dim)
    # multi-head KV is modelled on one GPU (no head split): its chunk equals the
    # host chunk; `tp` only shapes the shared-KV (num_kv_heads == 1) modes below
    gpu = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, Lyr, n, T, H, D, kv_dim=kv_dim)
    seen = set()
    for mode in (MODES if num_kv_heads == 1 else ["sharded"]):
        for h2d in (False, True):
            chunk = gpu.get_chunk_size() * es
            gbs = gpu.get_block_stride() * es
            layers_in_call = Lyr
            if num_kv_heads == 1 and not h2d:
                if mode == "sharded":
                    chunk //= tp                      # a rank moves 1/tp of every chunk
                elif mode == "layer_parallel":
                    layers_in_call = Lyr // tp        # a rank moves 1/tp of the layers
            cbs = cpu.get_block_stride() * es
            an, _ = lib_analyze(ids, ids, cbs, chunk, gbs)
            full = O.is_full_block(layers_in_call, kv_dim, chunk, cbs)
            got = NAMES[lib_choose(an, cpu_layout == "BLOCKFIRST", num_kv_heads, thr, chunk, h2d,
                                   full)]
            want = predicted(pattern, cpu_layout, kv_dim, num_kv_heads, mode, h2d, n, thr)
            if (num_kv_heads == 1 and not h2d and cpu_layout == "BLOCKFIRST"
                    and mode == "rank_rotate"):
                # one designated rank moves whole blocks: choose_path sees a full
                # block, the name-based predictor files rank_rotate under "shard"
                want = predicted(pattern, cpu_layout, kv_dim, num_kv_heads, "rank0_only", h2d, n, thr)
            assert got == want, (pattern, cpu_layout, kv_dim, num_kv_heads, mode, h2d, thr)
            seen.add(got)
    assert seen  # at least one strategy exercised per cell


def test_every_strategy_is_reachable():
    """Counterpart of test_ce_strategy_coverage (:1697-1727)."""
    seen = set()
    for pattern in ("contiguous", "few_seg", "scattered"):
        for cpu_layout in ("LAYERFIRST", "BLOCKFIRST"):
            for kv_dim, heads in ((1, 1), (2, 1), (1, 8), (2, 8)):
                for mode in MODES:
                    for h2d in (False, True):
                        seen.add(predicted(pattern, cpu_layout, kv_dim, heads, mode, h2d))
    assert seen == {"CONTIG_DIRECT", "SEGMENT_DIRECT", "SEGMENT_SCATTER", "GATHER_SCATTER",
                    "GATHER_DIRECT"}


def test_baseline_configs_route_as_documented():
    cfg = _lib.default_ce_config()
    cfg.is_blockfirst = 1
    rng = np.random.default_rng(1)
    # Llama-3-8B vLLM layout -> block-first host, kv_dim 2, 8 heads: GATHER_DIRECT
    ids = rng.permutation(4096)[:256]
    an, _ = lib_analyze(ids, rng.permutation(1024)[:256], 2097152, 32768, 32768)
    assert NAMES[lib_choose(an, True, 8, 8, 32768, False, True)] == "GATHER_DIRECT"
    # TRT-LLM GPU (block stride 5 MiB != chunk) -> GATHER_SCATTER
    an, _ = lib_analyze(ids, np.arange(256), 5242880, 32768, 5242880)
    assert NAMES[lib_choose(an, True, 8, 8, 32768, False, True)] == "GATHER_SCATTER"
    # layer-first host, packed KV, one contiguous run -> CONTIG_DIRECT
    an, _ = lib_analyze(np.arange(64), np.arange(64) + 5, 73728, 73728, 73728)
    assert NAMES[lib_choose(an, False, 1, 8, 73728, True, False)] == "CONTIG_DIRECT"
