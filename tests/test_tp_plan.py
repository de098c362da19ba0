"""Per-rank placement of a tensor-parallel transfer: library vs oracle over the
whole grid, and the partition properties any correct rule must have."""
import ctypes
import itertools

import pytest

from flexkv_amd import _lib
from oracle import fkv_oracle as O

L = _lib.load()
MODES = ["sharded", "all_write", "rank0_only", "layer_parallel", "rank_rotate", "bogus"]


def lib_plan(rank, n, heads, h2d, mode, designated, rotate, layer_id, gran, nblocks, chunk,
             cbs, tps):
    out = _lib.TPRankPlan()
    rc = L.fkv_tp_rank_plan_compute(rank, n, heads, int(h2d), mode.encode(), designated, rotate,
                                    layer_id, gran, nblocks, chunk, cbs, tps, ctypes.byref(out))
    _lib.check(rc)
    return out


def as_tuple(p):
    if not p.active:
        return (0,)
    return (1, p.start_layer, p.num_layers, p.cpu_startoff, p.gpu_startoff, p.chunk_size)


@pytest.mark.parametrize("n", [1, 2, 4, 8])
@pytest.mark.parametrize("heads", [1, 8])
@pytest.mark.parametrize("h2d", [False, True])
@pytest.mark.parametrize("mode", MODES)
def test_library_equals_oracle(n, heads, h2d, mode):
    chunk, cbs, nblocks = 73728, 73728 * 61, 17
    for gran, designated, rotate in itertools.product((1, 3, 7, 61), (0, n - 1), (0, n // 2)):
        for rank in range(n):
            a = lib_plan(rank, n, heads, h2d, mode, designated, rotate, 5, gran, nblocks, chunk,
                         cbs, cbs // n)
            b = O.tp_rank_plan(rank, n, heads, h2d, mode, designated, rotate, 5, gran, nblocks,
                               chunk, cbs, cbs // n)
            assert as_tuple(a) == as_tuple(b), (rank, gran, designated, rotate)


def plans(n, heads, h2d, mode, gran=7, designated=0, rotate=0, chunk=4096, cbs=4096 * 14,
          nblocks=5):
    return [lib_plan(r, n, heads, h2d, mode, designated, rotate, 2, gran, nblocks, chunk, cbs,
                     cbs // n) for r in range(n)]


@pytest.mark.parametrize("n", [2, 4, 8])
def test_sharded_d2h_shards_tile_every_chunk(n):
    ps = plans(n, 1, False, "sharded")
    spans = sorted((p.gpu_startoff, p.gpu_startoff + p.chunk_size) for p in ps)
    assert spans[0][0] == 0 and spans[-1][1] == 4096
    assert all(a[1] == b[0] for a, b in zip(spans, spans[1:]))       # no gap, no overlap
    assert all(p.cpu_startoff == p.gpu_startoff and p.active for p in ps)
    assert all((p.start_layer, p.num_layers) == (2, 7) for p in ps)


def test_sharded_d2h_rejects_indivisible_chunk():
    with pytest.raises(RuntimeError, match="divisible by num_gpus"):
        lib_plan(0, 3, 1, False, "sharded", 0, 0, 0, 1, 4, 4096, 4096, 4096)
    with pytest.raises(ValueError):
        O.tp_rank_plan(0, 3, 1, False, "sharded", 0, 0, 0, 1, 4, 4096, 4096, 4096)
    # H2D and one GPU are unaffected
    assert lib_plan(0, 3, 1, True, "sharded", 0, 0, 0, 1, 4, 4096, 4096, 4096).chunk_size == 4096
    assert lib_plan(0, 1, 1, False, "sharded", 0, 0, 0, 1, 4, 4097, 4097, 4097).chunk_size == 4097


@pytest.mark.parametrize("n,gran", [(4, 7), (4, 2), (8, 61), (2, 1), (8, 8)])
def test_layer_parallel_slices_tile_the_layer_range(n, gran):
    ps = plans(n, 1, False, "layer_parallel", gran=gran)
    act = [p for p in ps if p.active]
    assert len(act) == min(n, gran)
    spans = [(p.start_layer, p.start_layer + p.num_layers) for p in act]
    assert spans[0][0] == 2 and spans[-1][1] == 2 + gran
    assert all(a[1] == b[0] for a, b in zip(spans, spans[1:]))
    sizes = [p.num_layers for p in act]
    assert max(sizes) - min(sizes) <= 1 and sizes == sorted(sizes, reverse=True)
    assert all(p.chunk_size == 4096 and p.cpu_startoff == 0 and p.gpu_startoff == 0 for p in act)
    # the mode only splits GPU->host puts
    assert all(p.active and p.num_layers == gran for p in plans(n, 1, True, "layer_parallel", gran=gran))


@pytest.mark.parametrize("mode,designated,rotate,writer", [("rank0_only", 2, 1, 2),
                                                           ("rank_rotate", 2, 1, 1)])
def test_single_writer_modes(mode, designated, rotate, writer):
    ps = plans(4, 1, False, mode, designated=designated, rotate=rotate)
    assert [p.active for p in ps] == [int(r == writer) for r in range(4)]
    w = ps[writer]
    assert (w.cpu_startoff, w.gpu_startoff, w.chunk_size, w.num_layers) == (0, 0, 4096, 7)
    assert all(p.active for p in plans(4, 1, True, mode, designated=designated, rotate=rotate))


def test_all_write_regions_are_disjoint_and_whole():
    ps = plans(4, 1, False, "all_write", nblocks=5, cbs=4096 * 14)
    region = 5 * 4096 * 14
    assert [p.cpu_startoff for p in ps] == [r * region for r in range(4)]
    assert all(p.gpu_startoff == 0 and p.chunk_size == 4096 for p in ps)
    assert [p.cpu_startoff for p in plans(4, 1, True, "all_write")] == [r * region for r in range(4)]


def test_multi_head_ranks_take_head_slices():
    ps = plans(4, 8, False, "sharded", cbs=4096 * 14 * 4)
    assert [p.cpu_startoff for p in ps] == [r * 4096 * 14 for r in range(4)]
    assert all(p.gpu_startoff == 0 and p.chunk_size == 4096 and p.active for p in ps)
    # the sharing mode is ignored for multi-head KV
    assert [as_tuple(p) for p in plans(4, 8, False, "rank0_only", cbs=4096 * 14 * 4)] == \
        [as_tuple(p) for p in ps]


def test_unknown_mode_degrades_to_sharded():
    assert [as_tuple(p) for p in plans(4, 1, False, "bogus")] == \
        [as_tuple(p) for p in plans(4, 1, False, "sharded")]


def test_single_gpu_moves_everything_in_place():
    for mode in MODES:
        for h2d in (False, True):
            for heads in (1, 8):
                (p,) = plans(1, heads, h2d, mode)
                assert as_tuple(p) == (1, 2, 7, 0, 0, 4096)


def test_layerwise_restore_offsets():
    lib = O.lib()
    f = lambda r, heads, mode: lib.fkv_oracle_layerwise_cpu_startoff(r, heads, mode.encode(), 5,
                                                                      1000, 250)
    assert [f(r, 8, "sharded") for r in range(4)] == [0, 250, 500, 750]
    assert [f(r, 1, "sharded") for r in range(4)] == [0, 0, 0, 0]
    assert [f(r, 1, "rank0_only") for r in range(4)] == [0, 0, 0, 0]
    assert [f(r, 1, "all_write") for r in range(4)] == [0, 5000, 10000, 15000]
    assert [f(r, 1, "layer_parallel") for r in range(4)] == [0, 0, 0, 0]  # not valid for restore
