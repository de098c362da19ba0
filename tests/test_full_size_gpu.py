"""The benchmark configurations at their full sizes, checked through properties
that do not need a CPU pass over gigabytes: the host image equals torch's own
index_select of the engine tensors (compared on the GPU), gather -> erase ->
scatter restores every byte, and a checksum over whole tensors shows that no
other block was touched."""
import gc
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402

pytestmark = pytest.mark.gpu


def checksums(w):
    """One 64-bit wrap-around sum per engine tensor."""
    return [int(t.contiguous().view(torch.uint8).view(torch.int64).sum()) for t in w.tensors]


@pytest.fixture
def workload(request, gpu_device):
    w = bench.Workload(request.param, torch, gpu_device)
    yield w
    del w
    bench.release_cached_memory(torch)   # device and pinned host memory torch keeps cached


@pytest.mark.parametrize("workload,use_ce", [("c0", False), ("c0", True), ("c1", False),
                                             ("c1", True), ("c2", False), ("c2", True)],
                         indirect=["workload"], ids=["c0-kernel", "c0-ce", "c1-kernel", "c1-ce",
                                                     "c2-kernel", "c2-ce"])
def test_gather_erase_scatter_at_full_size(workload, use_ce):
    w = workload
    kw = dict(transfer_num_cta=4, use_ce_transfer=use_ce, ce_path_opt=True, sync=True)
    before = checksums(w)
    w.host.zero_()
    w.transfer(w.gpu_ids, w.cpu_ids, False, **kw)
    assert w.verify_host_image(w.gpu_ids, w.cpu_ids)
    assert checksums(w) == before                         # a put does not write the engine's tensors
    gi = w.gpu_ids.to(w.device)
    back = getattr(w, "gpu_ids_reload", w.gpu_ids)        # c2 reloads into another permutation
    bi = back.to(w.device)
    saved = [[w.gpu_rows(l, kv).index_select(0, gi) for kv in range(w.kv_dim)]
             for l in range(w.L)]
    for l in range(w.L):
        for kv in range(w.kv_dim):
            w.gpu_rows(l, kv).index_fill_(0, bi, 0)
    w.transfer(back, w.cpu_ids, True, **kw)
    for l in range(w.L):
        for kv in range(w.kv_dim):
            assert torch.equal(w.gpu_rows(l, kv).index_select(0, bi), saved[l][kv]), (l, kv)
    if back is w.gpu_ids:
        assert checksums(w) == before                     # every other block is as it was


@pytest.fixture(scope="module")
def c3(gpu_device):
    """One c3 workload (68 GiB of engine tensors) for all its cases; the cases with
    scattered host blocks re-make its host pool in place when they are reached."""
    w = bench.Workload("c3", torch, gpu_device)
    yield w
    del w
    bench.release_cached_memory(torch)   # device and pinned host memory torch keeps cached


# every route the library can take for a layerwise restore, forced through the launch policy
ROUTES = {"default": {},
          "kernel": dict(staged_restore=0, staged_gather=0),
          "copy_per_run": dict(staged_restore=2, staged_gather=0),
          "gathered": dict(staged_restore=0, staged_gather=2)}


@pytest.mark.parametrize("host_ids,route,notify", [
    ("one_run", "default", "polling"), ("one_run", "default", "hostfunc"),
    ("one_run", "kernel", "polling"), ("one_run", "copy_per_run", "hostfunc"),
    ("one_run", "gathered", "polling"),
    ("scattered", "default", "polling"), ("scattered", "default", "hostfunc"),
    ("scattered", "kernel", "polling"), ("scattered", "copy_per_run", "polling"),
    ("scattered", "gathered", "hostfunc")])
def test_layerwise_restore_at_full_size(c3, host_ids, route, notify):
    """c3 (61 layers x 512 blocks of 72 KiB) out of a host pool whose 512 blocks are one
    run, and out of a 4096-block pool with the 512 blocks scattered over it, on every
    route: after put -> erase -> restore the checksum of every engine tensor is what it
    was, and the counters say which route ran."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup, get_stats, launch_policy, reset_stats
    w = c3
    if host_ids == "scattered" and w.name == "c3":
        w.fragment_host_pool()
    assert (w.name == "c3f") == (host_ids == "scattered")   # the cases run in the order given
    before = checksums(w)
    w.transfer(w.gpu_ids, w.cpu_ids, False, transfer_num_cta=4, sync=True)
    assert w.verify_host_image(w.gpu_ids, w.cpu_ids)
    gi = w.gpu_ids.to(w.device)
    for l in range(w.L):
        w.gpu_rows(l, 0).index_fill_(0, gi, 0)
    assert checksums(w) != before
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)  # noqa: E731
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[w.tensors], cpu_blocks=w.host, ssd_files={}, num_layers=w.L,
        gpu_kv_strides_tensor=i64(w.gks), gpu_block_strides_tensor=i64(w.gbs),
        gpu_layer_strides_tensor=i64(w.gls), gpu_chunk_sizes_tensor=i64(w.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    e = torch.empty(0, dtype=torch.int64)
    with launch_policy(**ROUTES[route]):
        reset_stats()
        grp.layerwise_transfer(e, e, 0, 0, 0, 0, 0, w.gpu_ids, w.cpu_ids, w.cks, w.cls, w.cbs,
                               w.chunk, w.cks, w.cls, w.cbs, 4, False, w.L, 1, w.kv_dim, 1,
                               counter_id=0, kv_shared_across_ranks_mode="sharded",
                               notify_mode=notify)
        grp.synchronize()
        st = get_stats()
    torch.cuda.synchronize()
    assert checksums(w) == before
    taken = (st["staged_batches"], st["gathered_batches"])
    want = {("one_run", "default"): (w.L, 0), ("scattered", "default"): (w.L - 1, w.L - 1),
            "kernel": (0, 0), "copy_per_run": (w.L, 0), "gathered": (w.L - 1, w.L - 1)}
    assert taken == want.get((host_ids, route), want.get(route)), (host_ids, route, st)
    grp.close()


@pytest.mark.parametrize("workload", ["c4"], indirect=True)
@pytest.mark.parametrize("streams_per_direction", [32, 1])
def test_concurrent_requests_at_full_size(workload, streams_per_direction):
    """c4: 32 puts and 32 gets from 64 threads at once on a 32768-block pool, a
    stream per request or one per direction.  The engine blocks of the puts are
    changed and those of the gets wiped beforehand; afterwards the host image of
    every block equals its engine block, and blocks of no request are untouched."""
    w = workload
    used = torch.zeros(w.num_gpu_blocks, dtype=torch.bool)
    used[w.gpu_ids] = True
    idle = (~used).nonzero().flatten()[:4096].to(w.device)
    before = [int(w.gpu_rows(l, kv).index_select(0, idle).view(torch.int64).sum())
              for l in (0, w.L // 2, w.L - 1) for kv in range(w.kv_dim)]
    r = bench.run_concurrent(w, torch, steps=2, warmup=1, num_cta=4,
                             streams_per_direction=streams_per_direction, verify=True)
    assert r["bit_exact"] is True
    after = [int(w.gpu_rows(l, kv).index_select(0, idle).view(torch.int64).sum())
             for l in (0, w.L // 2, w.L - 1) for kv in range(w.kv_dim)]
    assert before == after
