"""Layerwise restore through the copy engines against the oracle, next to the same
restore on the kernel path: host rows -> staging buffer -> scatter kernel with one
copy command per run of host blocks, and host rows -> pinned buffer (gathered by host
threads) -> staging buffer -> scatter kernel with one copy command per batch.

The choice among the three is a matter of the launch policy; the tests force it,
so which route a case runs does not depend on the box."""
import numpy as np
import pytest
import torch

from kvsetup import KVSetup, SGLANG, TRTLLM, VLLM

pytestmark = pytest.mark.gpu


def group_of(s, dev):
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)
    return LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=s.num_layers,
        gpu_kv_strides_tensor=i64(s.gpu_kv_stride), gpu_block_strides_tensor=i64(s.gpu_block_stride),
        gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1,
        is_blockfirst=s.cpu_layout == "BLOCKFIRST")


def restore(grp, s, gids, cids, gran, notify="polling", num_layers=None, use_ce=False):
    e = torch.empty(0, dtype=torch.int64)
    grp.layerwise_transfer(
        e, e, 0, 0, 0, 0, 0, torch.as_tensor(gids), torch.as_tensor(cids), s.cpu_kv_stride,
        s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
        s.cpu_block_stride, 4, use_ce, s.num_layers if num_layers is None else num_layers, gran,
        s.kv_dim, 1, counter_id=0, kv_shared_across_ranks_mode="sharded", notify_mode=notify)
    grp.synchronize()


def host_ids(rng, pool, n, pattern):
    if pattern == "one_run":
        a = int(rng.integers(0, pool - n + 1))
        ids = np.arange(a, a + n)
    elif pattern == "runs_and_holes":  # runs of 1-6 blocks, holes of 1-3 blocks between them
        ids, at = [], 0
        while len(ids) < n and at < pool:
            run = int(rng.integers(1, 7))
            ids.extend(range(at, min(pool, at + run)))
            at += run + int(rng.integers(1, 4))
        ids = np.array(ids[:n])
    else:  # scattered
        ids = rng.permutation(pool)[:n]
    return rng.permutation(ids).astype(np.int64)  # positions in any order


ROUTES = {"copy_engines": dict(staged_restore=2, staged_gather=0),
          "gathered": dict(staged_restore=0, staged_gather=2, gather_first_by_kernel=0),
          "gathered_first_by_kernel": dict(staged_restore=0, staged_gather=2, gather_first_by_kernel=1),
          "kernel": dict(staged_restore=0, staged_gather=0),
          # every batch on the group's one stream (by default small batches alternate over two)
          "kernel_one_stream": dict(staged_restore=0, staged_gather=0, kernel_alt_stream_kb=0),
          "copy_engines_one_stream": dict(staged_restore=2, staged_gather=0, staged_dma_streams=1)}


@pytest.mark.parametrize("route", list(ROUTES))
@pytest.mark.parametrize("pattern", ["one_run", "runs_and_holes", "scattered"])
@pytest.mark.parametrize("backend,kv_dim,cpu_layout,gran", [
    (VLLM, 1, "BLOCKFIRST", 1), (VLLM, 2, "BLOCKFIRST", 3), (VLLM, 2, "LAYERFIRST", 2),
    (TRTLLM, 2, "BLOCKFIRST", 2), (SGLANG, 2, "BLOCKFIRST", 1), (SGLANG, 2, "LAYERFIRST", 4)])
def test_restore_matches_the_oracle(gpu_device, route, pattern, backend, kv_dim, cpu_layout, gran):
    """Seven layers (more batches than staging or pinned buffers), three restores in a
    row through the same group with fresh host bytes each time: a stale buffer or a
    buffer reused too early would show up as old bytes."""
    from flexkv_amd.c_ext import get_stats, launch_policy, reset_stats
    L, NG, NC, n, chunk = 7, 96, 80, 41, 4608
    s = KVSetup(backend, L, kv_dim, NG, NC, chunk, cpu_layout, seed=17 + gran)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    rng = np.random.default_rng(5 * gran + kv_dim)
    with launch_policy(staged_ring=3, gather_ring=2, gather_threads=3, **ROUTES[route]):
        reset_stats()
        for rep in range(3):
            fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
            s.host_ref[:] = fresh
            dev.host.copy_(torch.from_numpy(fresh))
            gids = rng.permutation(NG)[:n].astype(np.int64)
            cids = host_ids(rng, NC, n, pattern)
            restore(grp, s, gids, cids, gran, notify="hostfunc" if rep == 1 else "polling")
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference(f"restore {rep} ({pattern})")
        st = get_stats()
    batches = (L + gran - 1) // gran
    want_staged = {"copy_engines": 3 * batches, "gathered": 3 * batches,
                   "gathered_first_by_kernel": 3 * (batches - 1), "kernel": 0,
                   "kernel_one_stream": 0, "copy_engines_one_stream": 3 * batches}[route]
    assert st["staged_batches"] == want_staged, st
    assert st["gathered_batches"] == (want_staged if route.startswith("gathered") else 0), st
    grp.close()


def test_restore_of_a_layer_prefix_and_duplicate_host_blocks(gpu_device):
    """num_layers below the group's, a short last batch, and two GPU blocks that
    take the same host block."""
    from flexkv_amd.c_ext import get_stats, launch_policy, reset_stats
    s = KVSetup(VLLM, 9, 2, 64, 64, 2048, "BLOCKFIRST", seed=3)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    gids = np.array([5, 9, 60, 2, 33, 34], dtype=np.int64)
    cids = np.array([10, 11, 10, 12, 40, 13], dtype=np.int64)
    with launch_policy(staged_restore=2):
        reset_stats()
        restore(grp, s, gids, cids, gran=4, num_layers=7)   # batches of 4 + 3 layers
        assert get_stats()["staged_batches"] == 2
    s.oracle_transfer(gids, cids, True, num_layers=7)
    dev.assert_matches_reference("prefix of 7 layers")
    grp.close()


@pytest.mark.parametrize("route", ["copy_engines", "gathered_first_by_kernel", "kernel"])
@pytest.mark.parametrize("notify", ["polling", "hostfunc"])
def test_restore_asked_for_on_the_copy_engine_takes_the_staged_routes(gpu_device, route, notify):
    """use_ce_transfer chooses what the batches that do not go through a staging buffer
    fall back to; the staged routes themselves are open to it (with scattered host blocks
    the copy-engine strategies issue a copy command per block and layer).  No batch of
    such a restore goes by kernel, the first one included."""
    from flexkv_amd.c_ext import get_stats, last_transfer_path, launch_policy, reset_stats
    L, NG, NC, n, chunk, gran = 7, 96, 80, 41, 4608, 2
    s = KVSetup(VLLM, L, 2, NG, NC, chunk, "BLOCKFIRST", seed=23)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    rng = np.random.default_rng(29)
    batches = (L + gran - 1) // gran
    with launch_policy(staged_ring=3, gather_ring=2, gather_threads=3, **ROUTES[route]):
        reset_stats()
        for rep, pattern in enumerate(("scattered", "one_run", "runs_and_holes")):
            fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
            s.host_ref[:] = fresh
            dev.host.copy_(torch.from_numpy(fresh))
            gids = rng.permutation(NG)[:n].astype(np.int64)
            cids = host_ids(rng, NC, n, pattern)
            restore(grp, s, gids, cids, gran, notify=notify, use_ce=True)
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference(f"restore {rep} ({pattern}) on the copy engine")
        st = get_stats()
    staged = 0 if route == "kernel" else 3 * batches
    assert st["staged_batches"] == staged, st
    assert st["gathered_batches"] == (staged if route.startswith("gathered") else 0), st
    if route == "kernel":
        assert last_transfer_path() != "KERNEL"    # one of the copy-engine strategies
    else:
        assert st["kernel_launches"] == staged, st   # the scatter launches and nothing else
    grp.close()


@pytest.mark.parametrize("use_ce", [False, True])
def test_restore_from_a_pageable_host_pool(gpu_device, use_ce):
    """Ordinary host memory is not visible to the device: the kernel path and the copy
    per run cannot take it, rows gathered by host threads into pinned buffers can.  A
    restore that was asked for on the kernel and has no such route says what is wrong;
    one on the copy engine falls back to the engine's own strategies."""
    from flexkv_amd.c_ext import get_stats, launch_policy, reset_stats
    L, NG, NC, n, chunk, gran = 6, 64, 72, 33, 9216, 1
    s = KVSetup(SGLANG, L, 2, NG, NC, chunk, "BLOCKFIRST", seed=31)
    dev = s.to_device(gpu_device)
    dev.host = torch.empty(s.host_bytes, dtype=torch.uint8)   # pageable
    assert not dev.host.is_pinned()
    dev.host.copy_(torch.from_numpy(s.host_ref))
    grp = group_of(s, dev)
    rng = np.random.default_rng(37)
    gids = rng.permutation(NG)[:n].astype(np.int64)
    cids = host_ids(rng, NC, n, "scattered")
    with launch_policy(staged_restore=2, staged_gather=2, gather_ring=2, gather_threads=3):
        reset_stats()
        restore(grp, s, gids, cids, gran, use_ce=use_ce)
        st = get_stats()
    assert (st["staged_batches"], st["gathered_batches"]) == (L, L), st   # no batch by kernel or per run
    s.oracle_transfer(gids, cids, True)
    dev.assert_matches_reference("gathered out of pageable memory")
    # no staged route open
    fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
    s.host_ref[:] = fresh
    dev.host.copy_(torch.from_numpy(fresh))
    with launch_policy(staged_restore=2, staged_gather=0):
        reset_stats()
        if use_ce:
            restore(grp, s, gids, cids, gran, use_ce=True)
            assert get_stats()["staged_batches"] == 0
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference("copy-engine strategies out of pageable memory")
        else:
            before = [t.clone() for t in dev.gpu]
            with pytest.raises(ValueError, match="not device-visible"):
                restore(grp, s, gids, cids, gran, use_ce=False)
            torch.cuda.synchronize()
            assert all(torch.equal(a, b) for a, b in zip(before, dev.gpu))   # nothing was enqueued
    # and the group works afterwards
    with launch_policy(staged_gather=2):
        restore(grp, s, gids, cids, gran, use_ce=use_ce)
    if not use_ce:
        s.oracle_transfer(gids, cids, True)
    dev.assert_matches_reference("after the refused restore")
    grp.close()


@pytest.mark.parametrize("notify", ["polling", "hostfunc"])
def test_small_batches_by_kernel_alternate_over_two_streams(gpu_device, notify):
    """A restore by kernel in many small batches launches every other batch from the third
    on on a second stream.  Bytes against the oracle, the eventfds of the layers in order
    (the poller and the HOSTFUNC loop look at the batch events in order whichever stream
    recorded them), a consumer stream gated per layer with wait_layer, three restores in a
    row through one group, and the same with everything on one stream."""
    import os
    from flexkv_amd.c_ext import LayerwiseTransferGroup, get_stats, launch_policy, reset_stats
    from flexkv_amd.transfer.eventfd_channel import make_eventfd
    L, NG, NC, n, chunk = 17, 64, 64, 29, 8192
    s = KVSetup(VLLM, L, 2, NG, NC, chunk, "BLOCKFIRST", seed=41)
    dev = s.to_device(gpu_device)
    fds = [make_eventfd() for _ in range(L)]
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)  # noqa: E731
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=L,
        gpu_kv_strides_tensor=i64(s.gpu_kv_stride), gpu_block_strides_tensor=i64(s.gpu_block_stride),
        gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.tensor(fds, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    rng = np.random.default_rng(43)
    comp = torch.cuda.Stream()
    e = torch.empty(0, dtype=torch.int64)
    for rep, alt_kb in enumerate((4096, 4096, 0, 4096)):
        fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
        s.host_ref[:] = fresh
        dev.host.copy_(torch.from_numpy(fresh))
        gids = rng.permutation(NG)[:n].astype(np.int64)
        cids = host_ids(rng, NC, n, "scattered")
        gi = torch.as_tensor(gids).to(gpu_device)
        seen = []
        with launch_policy(staged_restore=0, staged_gather=0, kernel_alt_stream_kb=alt_kb):
            reset_stats()
            torch.cuda.synchronize()
            grp.layerwise_transfer(
                e, e, 0, 0, 0, 0, 0, torch.as_tensor(gids), torch.as_tensor(cids), s.cpu_kv_stride,
                s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
                s.cpu_block_stride, 4, False, L, 1, s.kv_dim, 1, counter_id=0,
                kv_shared_across_ranks_mode="sharded", notify_mode=notify)
            with torch.cuda.stream(comp):
                for l in range(L):      # what an engine does: gate layer l's kernels on layer l
                    grp.wait_layer(l, comp)
                    seen.append(dev.gpu[l].view(torch.uint8).reshape(2, NG, -1)
                                .index_select(1, gi).clone())
            grp.synchronize()
            comp.synchronize()
            st = get_stats()
        # batches 2, 4, .. 16 of 17
        assert st["second_stream_batches"] == (8 if alt_kb else 0), st
        s.oracle_transfer(gids, cids, True)
        dev.assert_matches_reference(f"restore {rep}, second stream {'on' if alt_kb else 'off'}")
        for l in range(L):
            want = torch.from_numpy(s.gpu_ref[l].view(np.uint8).reshape(2, NG, -1)[:, gids])
            assert torch.equal(seen[l].cpu(), want), (rep, l)
        for l, fd in enumerate(fds):       # one unit per layer and restore
            os.set_blocking(fd, False)
            assert int.from_bytes(os.read(fd, 8), "little") == 1, (rep, l)
    grp.close()
    for fd in fds:
        os.close(fd)


def test_gathered_restore_announces_layers_in_order_and_serves_waiting_streams(gpu_device):
    """The gathered route launches batch by batch from a thread of its own.  A consumer
    stream that asks for a layer before its batch has been enqueued must still see the
    layer's bytes (fkv_layerwise_wait_layer waits for the record first), the eventfds
    count one unit per layer, and the caller's id lists may be dropped right after the
    call returns."""
    import os
    import select
    from flexkv_amd.c_ext import LayerwiseTransferGroup, get_stats, launch_policy, reset_stats
    L, NG, NC, n, chunk = 9, 128, 160, 77, 18432
    s = KVSetup(VLLM, L, 1, NG, NC, chunk, "BLOCKFIRST", seed=41)
    dev = s.to_device(gpu_device)
    fds = [os.eventfd(0, os.EFD_SEMAPHORE | os.EFD_NONBLOCK) for _ in range(L)]
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=L,
        gpu_kv_strides_tensor=i64(s.gpu_kv_stride), gpu_block_strides_tensor=i64(s.gpu_block_stride),
        gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.tensor(fds, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    rng = np.random.default_rng(8)
    e = torch.empty(0, dtype=torch.int64)
    comp = torch.cuda.Stream()
    with launch_policy(staged_restore=0, staged_gather=2, gather_ring=2, gather_threads=2):
        for notify in ("polling", "hostfunc", "polling"):
            gids = rng.permutation(NG)[:n].astype(np.int64)
            cids = rng.permutation(NC)[:n].astype(np.int64)
            reset_stats()
            g_t, c_t = torch.from_numpy(gids.copy()), torch.from_numpy(cids.copy())
            grp.layerwise_transfer(
                e, e, 0, 0, 0, 0, 0, g_t, c_t, s.cpu_kv_stride, s.cpu_layer_stride,
                s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
                s.cpu_block_stride, 4, False, L, 1, 1, 1, counter_id=0,
                kv_shared_across_ranks_mode="sharded", notify_mode=notify)
            g_t.zero_()   # the library keeps what it needs of the id lists
            c_t.zero_()
            del g_t, c_t
            # every layer, read on a consumer stream right behind its event
            seen = []
            gi = torch.from_numpy(gids).to(gpu_device)
            with torch.cuda.stream(comp):
                for l in range(L):
                    grp.wait_layer(l, comp)
                    seen.append(dev.gpu[l].view(torch.uint8).view(NG, -1).index_select(0, gi).clone())
            comp.synchronize()
            grp.synchronize()
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference(f"gathered restore, {notify}")
            for l in range(L):
                want = s.host_ref.reshape(NC, L, chunk)[cids, l]
                assert np.array_equal(seen[l].cpu().numpy(), want), (notify, l)
            assert get_stats()["gathered_batches"] == L - 1   # the first batch by kernel
            for l, fd in enumerate(fds):
                assert select.select([fd], [], [], 5.0)[0], (notify, l)
                assert os.eventfd_read(fd) == 1
                assert not select.select([fd], [], [], 0)[0], (notify, l)
    grp.close()
    for fd in fds:
        os.close(fd)


@pytest.mark.parametrize("notify", ["polling", "hostfunc"])
@pytest.mark.parametrize("route", ["gathered", "kernel"])
def test_a_restore_that_gives_up_part_way_is_reported_and_the_group_stays_usable(gpu_device, route,
                                                                                notify):
    """The launch of a restore can fail part-way (here the launch policy makes it give up
    before its fourth batch; nothing faults).  The layers enqueued before that land and are
    announced, the others are not; whoever waits for one of them is told instead of waiting
    for good; the failure is reported by the call (when it happens inside the call) or by
    synchronize and the waiters (when the library's own thread launches the restore); and
    the next restore through the same group gives the oracle's bytes."""
    import os
    import select
    from flexkv_amd.c_ext import LayerwiseTransferGroup, launch_policy
    L, NG, NC, n, chunk = 7, 96, 120, 50, 9216
    s = KVSetup(VLLM, L, 1, NG, NC, chunk, "BLOCKFIRST", seed=52)
    dev = s.to_device(gpu_device)
    fds = [os.eventfd(0, os.EFD_SEMAPHORE | os.EFD_NONBLOCK) for _ in range(L)]
    i64 = lambda v: torch.tensor([v], dtype=torch.int64)
    grp = LayerwiseTransferGroup(
        num_gpus=1, gpu_blocks=[dev.gpu], cpu_blocks=dev.host, ssd_files={}, num_layers=L,
        gpu_kv_strides_tensor=i64(s.gpu_kv_stride), gpu_block_strides_tensor=i64(s.gpu_block_stride),
        gpu_layer_strides_tensor=i64(s.gpu_layer_stride), gpu_chunk_sizes_tensor=i64(s.chunk),
        iouring_entries=0, iouring_flags=0,
        layer_eventfds_tensor=torch.tensor(fds, dtype=torch.int32), tp_size=1, is_blockfirst=True)
    rng = np.random.default_rng(13)
    gids = rng.permutation(NG)[:n].astype(np.int64)
    cids = rng.permutation(NC)[:n].astype(np.int64)
    e = torch.empty(0, dtype=torch.int64)

    def call():
        grp.layerwise_transfer(
            e, e, 0, 0, 0, 0, 0, torch.from_numpy(gids), torch.from_numpy(cids), s.cpu_kv_stride,
            s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
            s.cpu_block_stride, 4, False, L, 1, 1, 1, counter_id=0,
            kv_shared_across_ranks_mode="sharded", notify_mode=notify)

    forced = dict(ROUTES[route], gather_first_by_kernel=0) if route == "gathered" else ROUTES[route]
    in_the_call = route == "kernel" or notify == "hostfunc"
    with launch_policy(test_fail_restore_batch=4, **forced):
        if in_the_call:
            with pytest.raises(RuntimeError, match="give up before batch 3"):
                call()
        else:
            call()                                  # returns while the restore is being launched
            comp = torch.cuda.Stream()
            for l in range(3):
                grp.wait_layer(l, comp)             # these land
            with pytest.raises(RuntimeError, match="will not land"):
                grp.wait_layer(3, comp)
            with pytest.raises(RuntimeError, match="give up before batch 3"):
                grp.synchronize()
        torch.cuda.synchronize()
    announced = [bool(select.select([fd], [], [], 0.5 if l < 3 else 0)[0]) for l, fd in enumerate(fds)]
    if route == "gathered":                         # announced as they landed, in order
        assert announced == [True] * 3 + [False] * 4, announced
    else:                                           # a call that fails on its own thread announces nothing
        assert announced == [False] * L, announced
    for l, fd in enumerate(fds):
        if announced[l]:
            assert os.eventfd_read(fd) == 1
    # the layers before the failure are where the oracle puts them; then a whole restore
    s.oracle_transfer(gids, cids, True, num_layers=3)
    dev.assert_matches_reference("layers enqueued before the restore gave up")
    with launch_policy(**forced):
        call()
        grp.synchronize()
    s.oracle_transfer(gids, cids, True)
    dev.assert_matches_reference("the next restore through the same group")
    for fd in fds:
        assert os.eventfd_read(fd) == 1
        os.close(fd)
    grp.close()


def test_the_choice_follows_the_runs_of_host_blocks(gpu_device):
    """With the default policy a restore whose host blocks form one run goes through
    the copy engines with one copy command, one whose host blocks are scattered has its
    rows gathered by host threads first (or stays on the kernel path where that route
    is switched off); all give the oracle's bytes.  (The choice is arithmetic on the id
    list: no timing.)"""
    from flexkv_amd.c_ext import get_stats, launch_policy, reset_stats
    L, n, chunk = 4, 256, 73728
    s = KVSetup(VLLM, L, 1, 300, 300, chunk, "BLOCKFIRST", seed=9)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    rng = np.random.default_rng(2)
    for gather, pattern, want, want_gathered in ((1, "one_run", L, 0), (1, "scattered", L - 1, L - 1),
                                                 (0, "scattered", 0, 0)):
        with launch_policy(staged_restore=1, staged_gather=gather):
            gids = rng.permutation(300)[:n].astype(np.int64)
            cids = host_ids(rng, 300, n, pattern)
            reset_stats()
            restore(grp, s, gids, cids, gran=1)
            st = get_stats()
            assert (st["staged_batches"], st["gathered_batches"]) == (want, want_gathered), (pattern, st)
            s.oracle_transfer(gids, cids, True)
            dev.assert_matches_reference(pattern)
    grp.close()


@pytest.mark.parametrize("seed", range(40))
def test_seeded_random_restores(gpu_device, seed):
    """Shape, host layout, id pattern, granularity, layer prefix, route, engine asked for,
    notify mode and ring sizes drawn from a seed; two restores through the same group with
    fresh host bytes, every byte against the oracle."""
    from flexkv_amd.c_ext import launch_policy
    rng = np.random.default_rng(3000 + seed)
    backend = int(rng.choice([VLLM, TRTLLM, SGLANG]))
    L = int(rng.integers(1, 21))
    kv_dim = 2 if backend == SGLANG else int(rng.choice([1, 2]))
    NG, NC = int(rng.integers(8, 100)), int(rng.integers(8, 100))
    gran16 = rng.random() < 0.8
    chunk = 16 * int(rng.integers(1, 700)) if gran16 else 8 * int(rng.integers(1, 60)) + int(rng.choice([0, 4, 2]))
    cpu_layout = str(rng.choice(["BLOCKFIRST", "LAYERFIRST"]))
    n = int(rng.integers(1, min(NG, NC) + 1))
    gran = int(rng.integers(1, L + 1))
    layers = int(rng.integers(1, L + 1))
    route = str(rng.choice(list(ROUTES) + ["default"]))
    use_ce = bool(rng.random() < 0.3) and chunk % 8 == 0
    policy = dict(ROUTES.get(route, {}), staged_ring=int(rng.integers(2, 5)),
                  gather_ring=int(rng.integers(2, 5)), gather_threads=int(rng.integers(2, 6)))
    s = KVSetup(backend, L, kv_dim, NG, NC, chunk, cpu_layout, seed=4000 + seed)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    print("case", dict(backend=backend, L=L, kv_dim=kv_dim, NG=NG, NC=NC, chunk=chunk,
                       cpu_layout=cpu_layout, n=n, gran=gran, layers=layers, route=route,
                       use_ce=use_ce, policy=policy), flush=True)
    with launch_policy(**policy):
        for rep in range(2):
            fresh = rng.integers(0, 256, s.host_bytes, dtype=np.uint8)
            s.host_ref[:] = fresh
            dev.host.copy_(torch.from_numpy(fresh))
            gids = rng.permutation(NG)[:n].astype(np.int64)
            cids = host_ids(rng, NC, n, str(rng.choice(["one_run", "runs_and_holes", "scattered"])))
            if cids.size < n:           # runs_and_holes may run out of pool
                gids = gids[:cids.size]
            restore(grp, s, gids, cids, gran, notify=str(rng.choice(["polling", "hostfunc"])),
                    num_layers=layers, use_ce=use_ce)
            s.oracle_transfer(gids, cids, True, num_layers=layers)
            dev.assert_matches_reference(f"restore {rep}")
    grp.close()


@pytest.mark.parametrize("route", ["kernel", "copy_engines", "gathered"])
def test_named_compute_stream_keeps_the_restore_beside_the_forward_pass(gpu_device, route):
    """Streams of a process share a few hardware queues, and two streams on one queue run
    one after the other.  Once the engine has named its forward stream, the group's own
    streams sit on other queues: for eight forward streams in a row (torch hands them out
    over all queues, the null stream among them) no stream of the group shares the queue, a
    restore with a per-layer consumer gated on wait_layer still equals the oracle, and a
    restore next to a forward pass of about its own length takes well under the two
    one after the other."""
    from flexkv_amd.c_ext import get_stats, launch_policy, reset_stats
    L, NG, NC, n, chunk = 16, 320, 320, 256, 32768
    s = KVSetup(VLLM, L, 2, NG, NC, chunk, "BLOCKFIRST", seed=71)
    dev = s.to_device(gpu_device)
    grp = group_of(s, dev)
    rng = np.random.default_rng(72)
    gids = rng.permutation(NG)[:n].astype(np.int64)
    cids = host_ids(rng, NC, n, "one_run" if route == "copy_engines" else "scattered")
    s.oracle_transfer(gids, cids, True)
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731
    e = torch.empty(0, dtype=torch.int64)

    def launch():
        grp.layerwise_transfer(
            e, e, 0, 0, 0, 0, 0, torch.as_tensor(gids), torch.as_tensor(cids), s.cpu_kv_stride,
            s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride, s.cpu_layer_stride,
            s.cpu_block_stride, 4, False, L, 1, s.kv_dim, 1, counter_id=0,
            kv_shared_across_ranks_mode="sharded", notify_mode="polling")

    with launch_policy(**ROUTES[route]):
        launch()            # buffers, code objects
        grp.synchronize()
        launch()
        grp.synchronize()
        restore_ms = grp.batch_times_ms()[-1]
        cycles = 200_000
        streams = [torch.cuda.default_stream()] + [torch.cuda.Stream() for _ in range(7)]
        for k, comp in enumerate(streams):
            assert grp.set_compute_stream(comp) == 0, k
            with torch.cuda.stream(comp):   # a forward pass of about the restore's length
                torch.cuda._sleep(cycles)
                a, b = ev(), ev()
                a.record(comp)
                for _ in range(L):
                    torch.cuda._sleep(cycles)
                b.record(comp)
                b.synchronize()
                if k == 0:
                    cycles = max(1000, int(cycles * restore_ms / max(a.elapsed_time(b), 1e-3)))
                a, b = ev(), ev()
                a.record(comp)
                for _ in range(L):
                    torch.cuda._sleep(cycles)
                b.record(comp)
                b.synchronize()
                forward_ms = a.elapsed_time(b)
            for t in dev.gpu:
                t.zero_()
            torch.cuda.synchronize()
            reset_stats()
            t0, t1 = ev(), ev()
            with torch.cuda.stream(comp):
                t0.record(comp)
            launch()
            with torch.cuda.stream(comp):
                for l in range(L):
                    grp.wait_layer(l, comp)
                    torch.cuda._sleep(cycles)
                t1.record(comp)
            grp.synchronize()
            t1.synchronize()
            both_ms = t0.elapsed_time(t1)
            st = get_stats()
            assert (st["staged_batches"] > 0) == (route != "kernel"), st
            assert (st["gathered_batches"] > 0) == (route == "gathered"), st
            got = [t.cpu() for t in dev.gpu]
            for l in range(L):
                want = torch.from_numpy(s.gpu_ref[l].view(np.uint8).reshape(2, NG, -1)[:, gids])
                have = got[l].view(torch.uint8).reshape(2, NG, -1)[:, torch.as_tensor(gids)]
                assert torch.equal(have, want), (k, l)
            assert both_ms < 0.8 * (restore_ms + forward_ms), (k, both_ms, restore_ms, forward_ms)
    grp.close()
