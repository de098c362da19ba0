"""HIP gather/scatter kernel vs the CPU oracle, through the C ABI, bit-exact."""
import os
import time

import numpy as np
import pytest

from kvsetup import KVSetup, VLLM, TRTLLM, SGLANG, block_ids

pytestmark = pytest.mark.gpu

# (backend, L, kv_dim, N_gpu, N_cpu, chunk, cpu_layout, gpu_layout)
KERNEL_CASES = [
    pytest.param(VLLM, 4, 2, 64, 48, 16 * 8 * 128 * 2, "BLOCKFIRST", "LAYERFIRST", id="vllm-llama-bf"),
    pytest.param(VLLM, 4, 2, 64, 48, 16 * 8 * 128 * 2, "LAYERFIRST", "LAYERFIRST", id="vllm-llama-lf"),
    pytest.param(VLLM, 3, 2, 40, 40, 4096, "BLOCKFIRST", "LAYERBLOCK", id="vllm-layerblock"),
    pytest.param(VLLM, 5, 1, 32, 32, 64 * 576 * 2, "BLOCKFIRST", "LAYERFIRST", id="mla-packed"),
    pytest.param(TRTLLM, 6, 2, 32, 32, 8 * 32 * 128, "BLOCKFIRST", "LAYERFIRST", id="trtllm-fp8"),
    pytest.param(SGLANG, 4, 2, 64, 32, 64 * 8 * 128 * 2, "BLOCKFIRST", "LAYERFIRST", id="sglang-page64"),
    pytest.param(SGLANG, 4, 2, 64, 32, 1024, "LAYERFIRST", "LAYERFIRST", id="sglang-lf"),
]


@pytest.mark.parametrize("backend,L,K,N,NH,chunk,cpu_layout,gpu_layout", KERNEL_CASES)
@pytest.mark.parametrize("pattern", ["scattered", "contiguous", "few_seg"])
def test_kernel_d2h_then_h2d_matches_oracle(gpu_device, backend, L, K, N, NH, chunk, cpu_layout,
                                            gpu_layout, pattern):
    s = KVSetup(backend, L, K, N, NH, chunk, cpu_layout, gpu_layout, seed=11)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(5)
    n = 24
    gids, cids = block_ids(rng, N, n, pattern), block_ids(rng, NH, n, pattern)
    print(f"case backend={backend} L={L} kv={K} chunk={chunk} {cpu_layout} {pattern}", flush=True)
    # D2H gather
    dev.transfer(gids, cids, is_h2d=False)
    s.oracle_transfer(gids, cids, is_h2d=False)
    dev.assert_matches_reference("after D2H")
    # H2D scatter into different GPU blocks
    gids2 = block_ids(rng, N, n, "scattered")
    dev.transfer(gids2, cids, is_h2d=True)
    s.oracle_transfer(gids2, cids, is_h2d=True)
    dev.assert_matches_reference("after H2D")


# ---- alignment fallbacks, offsets, edge shapes (straight through the C ABI) ----

@pytest.mark.parametrize("chunk,gpu_off,cpu_off,sub", [
    (4680 * 8, 4680, 4680, 4680),   # 8-aligned shard of a 16-aligned chunk (the reference's 8-byte kernel)
    (40, 0, 0, 40),                  # chunk % 16 == 8
    (48, 8, 24, 16),                 # offsets differ on the two sides
    (20, 0, 0, 20),                  # 4-byte granularity (outside the reference's domain)
    (6, 2, 2, 4),
    (7, 0, 0, 7),                    # odd bytes
    (3 * 8192 + 48, 0, 0, 3 * 8192 + 48),  # several full slices and a short tail
])
@pytest.mark.parametrize("backend", [VLLM, TRTLLM, SGLANG])
def test_offsets_and_narrow_alignment(gpu_device, backend, chunk, gpu_off, cpu_off, sub):
    s = KVSetup(backend, 3, 2, 20, 16, chunk, "BLOCKFIRST", seed=21)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(2)
    gids, cids = block_ids(rng, 20, 9), block_ids(rng, 16, 9)
    print(f"case backend={backend} chunk={chunk} offs=({gpu_off},{cpu_off}) sub={sub}", flush=True)
    for h2d in (False, True):
        assert dev.transfer_raw(gids, cids, h2d, gpu_off=gpu_off, cpu_off=cpu_off, chunk=sub) == 0
        s.oracle_transfer(gids, cids, h2d, gpu_off=gpu_off, cpu_off=cpu_off, chunk=sub)
        dev.assert_matches_reference(f"h2d={h2d}")
        gids = block_ids(rng, 20, 9)


def test_padded_gpu_blocks_and_partial_layer_range(gpu_device):
    s = KVSetup(VLLM, 6, 2, 24, 24, 2048, "LAYERFIRST", seed=5, gpu_block_pad=256)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(3)
    gids, cids = block_ids(rng, 24, 10), block_ids(rng, 24, 10)
    dev.transfer(gids, cids, is_h2d=False, start_layer=2, num_layers=3)
    s.oracle_transfer(gids, cids, False, start_layer=2, num_layers=3)
    dev.assert_matches_reference("layers 2..4 D2H")
    dev.transfer(cids, gids, is_h2d=True, start_layer=4, num_layers=2)
    s.oracle_transfer(cids, gids, True, start_layer=4, num_layers=2)
    dev.assert_matches_reference("layers 4..5 H2D")


def test_sglang_partial_layers_address_v_tensors(gpu_device):
    """A call that covers only some layers must still find V_l at ptrs[L + l]."""
    s = KVSetup(SGLANG, 5, 2, 12, 12, 512, "BLOCKFIRST", seed=6)
    dev = s.to_device(gpu_device)
    ids = np.array([3, 9, 1], dtype=np.int64)
    dev.transfer(ids, ids, is_h2d=False, start_layer=3, num_layers=2)
    s.oracle_transfer(ids, ids, False, start_layer=3, num_layers=2)
    dev.assert_matches_reference("sglang layers 3..4")


def test_empty_single_and_duplicate_ids(gpu_device):
    s = KVSetup(VLLM, 2, 2, 8, 8, 1024, "BLOCKFIRST", seed=7)
    dev = s.to_device(gpu_device)
    none = np.empty(0, dtype=np.int64)
    dev.transfer(none, none, is_h2d=False)
    dev.transfer(none, none, is_h2d=True, use_ce_transfer=True, ce_path_opt=True)
    dev.assert_matches_reference("empty transfer must not touch anything")
    one = np.array([5], dtype=np.int64)
    dev.transfer(one, np.array([2], dtype=np.int64), is_h2d=False)
    s.oracle_transfer(one, np.array([2], dtype=np.int64), False)
    dev.assert_matches_reference("single block")
    # one GPU block fanned out to two host blocks (duplicate source ids are legal)
    dup, dst = np.array([6, 6, 1], dtype=np.int64), np.array([0, 7, 3], dtype=np.int64)
    dev.transfer(dup, dst, is_h2d=False)
    s.oracle_transfer(dup, dst, False)
    dev.assert_matches_reference("duplicate source ids")


def test_many_blocks_cross_id_tiles(gpu_device):
    """More block positions than one LDS id tile holds, few bytes each."""
    s = KVSetup(VLLM, 2, 2, 5000, 5000, 64, "BLOCKFIRST", seed=8)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(4)
    gids, cids = block_ids(rng, 5000, 4500), block_ids(rng, 5000, 4500)
    for cta in (1, 4, 64):
        assert dev.transfer_raw(gids, cids, False, num_cta=cta) == 0
    s.oracle_transfer(gids, cids, False)
    dev.assert_matches_reference("4500 blocks D2H")
    assert dev.transfer_raw(cids, gids, True, num_cta=3) == 0
    s.oracle_transfer(cids, gids, True)
    dev.assert_matches_reference("4500 blocks H2D")


@pytest.mark.parametrize("backend,L,K,chunk,n", [
    (VLLM, 31, 1, 2 * 576 * 2, 512),      # a 128x-compressed latent group: 2304-byte chunks
    (VLLM, 3, 2, 144, 700),                # 9 vectors per chunk, more positions than an id tile holds
    (SGLANG, 5, 2, 8176, 40),              # one vector short of a full slice
    (TRTLLM, 7, 2, 520, 300),              # 8-byte vectors (520 = 8 * 65)
    (VLLM, 2, 2, 1028, 90),                # 4-byte vectors
])
def test_short_chunks_are_packed(gpu_device, backend, L, K, chunk, n):
    """Chunks shorter than a slice travel as one flat sequence of vectors: pieces,
    workgroup ranges and id tiles all cut through chunks at arbitrary places."""
    N = n + n // 2
    s = KVSetup(backend, L, K, N, N, chunk, "BLOCKFIRST", seed=31)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(6)
    for cta in (1, 4, 37):
        gids, cids = block_ids(rng, N, n), block_ids(rng, N, n)
        print(f"case backend={backend} chunk={chunk} n={n} cta={cta}", flush=True)
        assert dev.transfer_raw(gids, cids, False, num_cta=cta) == 0
        s.oracle_transfer(gids, cids, False)
        dev.assert_matches_reference(f"D2H cta={cta}")
        gids2 = block_ids(rng, N, n)
        assert dev.transfer_raw(gids2, cids, True, num_cta=cta) == 0
        s.oracle_transfer(gids2, cids, True)
        dev.assert_matches_reference(f"H2D cta={cta}")


@pytest.mark.parametrize("chunk", [16 * 8 * 128 * 2, 1152, 24], ids=["32k", "packed", "narrow"])
def test_puts_and_gets_at_the_same_time(gpu_device, chunk):
    """A GPU->host and a host->GPU transfer in flight together on two streams: a
    launch that finds the other direction busy confines itself to half of the
    XCDs.  Which workgroups take part must not change a byte (also for chunks
    shorter than a slice, which are packed, and for 8-byte vectors)."""
    import threading
    import torch
    s = KVSetup(VLLM, 8, 2, 600, 600, chunk, "BLOCKFIRST", seed=41)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(8)
    perm_g, perm_c = rng.permutation(600), rng.permutation(600)
    # disjoint blocks on both sides, so the two directions never touch the same bytes
    put_g, put_c = perm_g[:250], perm_c[:250]
    get_g, get_c = perm_g[250:500], perm_c[250:500]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    errors = []
    from flexkv_amd.c_ext import get_stats, reset_stats
    reset_stats()

    def run(i):
        try:
            for _ in range(6):
                rc = dev.transfer_raw(put_g if i == 0 else get_g, put_c if i == 0 else get_c,
                                      i == 1, sync=False, stream=streams[i].cuda_stream)
                assert rc == 0
            streams[i].synchronize()
        except Exception as e:  # noqa: BLE001
            errors.append(e)
    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors, errors
    torch.cuda.synchronize()
    st = get_stats()
    print("launch counters (reported, not asserted):", st)
    s.oracle_transfer(put_g, put_c, False)
    s.oracle_transfer(get_g, get_c, True)
    dev.assert_matches_reference("concurrent put and get")


def test_confined_launches_one_after_another_each_do_their_work(gpu_device):
    """Confined launches share counters that each launch must leave zeroed: 24
    transfers of different blocks, alternating directions with a wait after each,
    reuse the same plan memory, and every one of them has to move its blocks."""
    from flexkv_amd.c_ext import get_stats, reset_stats
    s = KVSetup(VLLM, 4, 2, 520, 520, 4096, "BLOCKFIRST", seed=43)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(12)
    perm_g, perm_c = rng.permutation(520), rng.permutation(520)
    import torch
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]  # work of the launching stream never counts as busy
    reset_stats()
    for k in range(24):
        h2d = k % 2 == 1
        g, c = perm_g[k * 20:(k + 1) * 20 + (k % 3)], perm_c[k * 20:(k + 1) * 20 + (k % 3)]
        with torch.cuda.stream(streams[k % 2]):
            dev.transfer(g, c, is_h2d=h2d)
        s.oracle_transfer(g, c, h2d)
    st = get_stats()
    print("launch counters (reported, not asserted):", st)
    dev.assert_matches_reference("24 confined launches in a row")


def test_more_layer_kv_pairs_than_one_launch_holds(gpu_device):
    """700 layers x 2 = 1400 (layer, kv) pairs: split over two launches."""
    s = KVSetup(VLLM, 700, 2, 6, 6, 32, "BLOCKFIRST", seed=9)
    dev = s.to_device(gpu_device)
    ids = np.array([4, 0, 5, 2], dtype=np.int64)
    dev.transfer(ids, ids[::-1].copy(), is_h2d=False)
    s.oracle_transfer(ids, ids[::-1].copy(), False)
    dev.assert_matches_reference("1400 pairs D2H")
    dev.transfer(ids[::-1].copy(), ids, is_h2d=True, use_ce_transfer=True, ce_path_opt=True)
    s.oracle_transfer(ids[::-1].copy(), ids, True)
    dev.assert_matches_reference("1400 pairs H2D via copy engine")


def test_async_call_owns_its_id_arrays(gpu_device):
    """sync=False returns before the copy runs; the caller may reuse its id
    tensors at once (they are copied into library-owned plan memory)."""
    import torch
    from flexkv_amd.c_ext import transfer_kv_blocks
    s = KVSetup(VLLM, 8, 2, 256, 256, 32768, "BLOCKFIRST", seed=10)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(6)
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        for rep in range(6):
            gids, cids = block_ids(rng, 256, 200), block_ids(rng, 256, 200)
            g, c = torch.from_numpy(gids.copy()), torch.from_numpy(cids.copy())
            h2d = bool(rep % 2)
            transfer_kv_blocks(g, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride,
                               c, dev.host, s.cpu_kv_stride, s.cpu_layer_stride,
                               s.cpu_block_stride, s.chunk, 0, 8, is_host_to_device=h2d,
                               sync=False, is_blockfirst=True)
            g.fill_(255)   # scribble over the caller's arrays while the copy is in flight
            c.fill_(255)
            s.oracle_transfer(gids, cids, h2d)
    st.synchronize()
    dev.assert_matches_reference("six back-to-back async transfers")


def test_pageable_host_tensor_is_refused_by_the_kernel_path(gpu_device):
    import torch
    from flexkv_amd.c_ext import transfer_kv_blocks
    s = KVSetup(VLLM, 2, 2, 8, 8, 1024, "BLOCKFIRST", seed=11)
    dev = s.to_device(gpu_device)
    pageable = torch.zeros(s.host_bytes, dtype=torch.uint8)
    ids = torch.arange(4, dtype=torch.int64)
    with pytest.raises(ValueError, match="not device-visible"):
        transfer_kv_blocks(ids, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride,
                           ids, pageable, s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride,
                           s.chunk, 0, 2, is_host_to_device=False)
    # the copy-engine path reads ids and data through the runtime and accepts pageable memory
    # (also when every copy of pinned memory would go out as a 2-D copy)
    from flexkv_amd.c_ext import launch_policy
    for rect_min_kb in (-1, 0):
        pageable.zero_()
        with launch_policy(ce_rect_min_kb=rect_min_kb):
            transfer_kv_blocks(ids, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride,
                               ids, pageable, s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride,
                               s.chunk, 0, 2, is_host_to_device=False, use_ce_transfer=True)
            torch.cuda.synchronize()
        s.host_ref[:] = 0
        s.oracle_transfer(ids.numpy(), ids.numpy(), False)
        np.testing.assert_array_equal(pageable.numpy(), s.host_ref)


def test_streams_run_concurrently_tells_hardware_queue_sharing(gpu_device):
    """The same stream never overlaps with itself.  Which of six streams share a
    hardware queue is a property of the box (with four queues some pair does not):
    the table is printed, not asserted."""
    import torch
    from flexkv_amd.c_ext import streams_run_concurrently
    streams = [torch.cuda.Stream() for _ in range(6)]
    assert streams_run_concurrently(streams[0], streams[0]) is False
    table = [[streams_run_concurrently(a, b) for b in streams] for a in streams]
    print("streams that run concurrently:", table)
    assert all(not table[i][i] for i in range(6))


def test_streams_hand_over_us_times_an_event_chain_on_the_device(gpu_device):
    """The round trip of an event between two streams, timed on the device: a stream with
    itself gives the floor, another stream is at least as slow and (on different hardware
    queues of a device with four of them) within a few times the floor; the streams are left
    idle and usable.  Which pairs are slow is a property of the box: printed, not asserted."""
    import torch
    from flexkv_amd.c_ext import streams_hand_over_us
    streams = [torch.cuda.Stream() for _ in range(5)]
    floor = streams_hand_over_us(streams[0], streams[0])
    assert 1.0 < floor < 500.0, floor
    pairs = [streams_hand_over_us(streams[0], b) for b in streams[1:]]
    print("event round trips in microseconds: same stream %.1f, others" % floor,
          [round(p, 1) for p in pairs])
    assert all(0.5 * floor < p < 2000.0 for p in pairs), (floor, pairs)
    x = torch.zeros(8, device=gpu_device)
    for s in streams:
        with torch.cuda.stream(s):
            x.add_(1)
    torch.cuda.synchronize()
    assert float(x[0]) == 5.0


def test_a_put_in_another_process_confines_the_gets_of_this_one(gpu_device):
    """Two processes on one GPU: a child keeps posting puts, and the gets of this
    process (too small to keep to home XCDs by themselves) confine themselves
    because the board the processes share says that the other direction is busy.
    Once the child has gone they run on all XCDs again."""
    import subprocess
    import sys
    from flexkv_amd.c_ext import (get_launch_policy, get_stats, launch_policy,
                                  link_activity_elsewhere, reset_stats)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if os.environ.get("FKV_LINK_BOARD_KEY"):
        pytest.skip("the board key of this process is fixed from outside")
    script = (
        "import sys, time; sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + '/tests')\n"
        "import numpy as np, torch\n"
        "from kvsetup import KVSetup\n"
        "dev = KVSetup(0, 4, 2, 64, 64, 65536, 'BLOCKFIRST', seed=3).to_device('cuda:0')\n"
        "ids = np.arange(64)\n"
        "dev.transfer(ids, ids, is_h2d=False)\n"
        "print('putting', flush=True)\n"
        "end = time.time() + 60\n"
        "import select\n"
        "while time.time() < end and not select.select([sys.stdin], [], [], 0)[0]:\n"
        "    dev.transfer(ids, ids, is_h2d=False)\n")
    # both processes address the GPU by its PCI address: no key in the environment
    child = subprocess.Popen([sys.executable, "-c", script, root], stdin=subprocess.PIPE,
                             stdout=subprocess.PIPE, text=True)
    try:
        assert child.stdout.readline().strip() == "putting"
        s = KVSetup(VLLM, 4, 2, 64, 64, 4096, "BLOCKFIRST", seed=44)
        dev = s.to_device(gpu_device)
        rng = np.random.default_rng(3)
        # the child posts a put every millisecond or so: within a window of a second its
        # activity is always in sight (the default window of 20 ms is a matter of timing)
        assert link_activity_elsewhere(False, window_ms=1000)
        split = get_launch_policy()["xcd_count"] >= 4
        with launch_policy(arbiter=1, busy_window_ms=1000, lane_streams=0):
            reset_stats()
            for _ in range(5):
                g, c = rng.permutation(64)[:40], rng.permutation(64)[:40]
                dev.transfer(g, c, is_h2d=True)
                s.oracle_transfer(g, c, True)
            st = get_stats()
        assert st["kernel_launches"] == 5 and st["confined_launches"] == (5 if split else 0), st
        dev.assert_matches_reference("gets next to another process's puts")
    finally:
        child.stdin.write("\n")
        child.stdin.close()
        assert child.wait(60) == 0
    time.sleep(0.1)
    g = np.arange(40)
    with launch_policy(arbiter=1, busy_window_ms=0, lane_streams=0):
        reset_stats()
        dev.transfer(g, g, is_h2d=True)
        st = get_stats()
    # what the child posted has ended, and nothing of this process runs the other way
    assert st["kernel_launches"] == 1 and st["confined_launches"] == 0, st
    s.oracle_transfer(g, g, True)
    dev.assert_matches_reference("get after the other process has gone")


def test_the_arbiter_confines_a_launch_while_the_other_direction_counts_as_busy(gpu_device):
    """arbiter = 1, the setting production runs with: a get launched within the busy window
    of a put on another stream confines itself to the host->GPU XCDs; with no window and
    the put long finished it runs on all XCDs.  A long window makes the first case
    independent of timing."""
    import torch
    from flexkv_amd.c_ext import get_launch_policy, get_stats, launch_policy, reset_stats
    if get_launch_policy()["xcd_count"] < 4:
        pytest.skip("a device with fewer than four XCDs is not split")
    s = KVSetup(VLLM, 4, 2, 96, 96, 4096, "BLOCKFIRST", seed=47)   # 1.3 MB a transfer: below
    dev = s.to_device(gpu_device)                                    # the home threshold
    rng = np.random.default_rng(6)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()

    def move(stream, h2d):
        g, c = rng.permutation(96)[:40], rng.permutation(96)[:40]
        with torch.cuda.stream(stream):
            dev.transfer(g, c, is_h2d=h2d)       # synchronous
        s.oracle_transfer(g, c, h2d)

    with launch_policy(arbiter=1, busy_window_ms=10000, lane_streams=0):
        move(a, False)                            # a put: GPU->host counts as busy from now on
        reset_stats()
        for _ in range(3):
            move(b, True)
        st = get_stats()
        assert st["kernel_launches"] == 3 and st["confined_launches"] == 3, st
        reset_stats()
        move(a, False)                            # and the gets make host->GPU busy for the puts
        st = get_stats()
        assert st["kernel_launches"] == 1 and st["confined_launches"] == 1, st
    torch.cuda.synchronize()
    with launch_policy(arbiter=1, busy_window_ms=0, lane_streams=0):
        reset_stats()
        move(b, True)
        st = get_stats()
        assert st["kernel_launches"] == 1 and st["confined_launches"] == 0, st
    dev.assert_matches_reference("confined and unconfined launches")


@pytest.mark.parametrize("mode", ["arbiter_off", "confined", "home", "safety_net", "claims_on_all_xcds"])
def test_every_way_a_launch_can_share_out_its_work(gpu_device, mode):
    """The launch policy forces each way the workgroups of a launch come by their
    work, whatever the link is doing: fixed shares on all XCDs (arbiter off),
    confined to the XCDs of a busy link, confined to the home XCDs, no workgroup on
    a selected XCD so that the safety-net workgroup copies everything, and ranges
    claimed on all XCDs.  Normal, packed and long chunks, both directions, several
    transfers through the same counters: the oracle's bytes every time."""
    from flexkv_amd.c_ext import get_launch_policy, get_stats, launch_policy, reset_stats
    fields = {"arbiter_off": dict(arbiter=0), "confined": dict(arbiter=2),
              "home": dict(arbiter=1, home_min_kb=0, busy_window_ms=0),
              "safety_net": dict(arbiter=3, safety_net_wait_us=5),
              "claims_on_all_xcds": dict(arbiter=0, all_claims_per_wg=8)}[mode]
    xcds = get_launch_policy()["xcd_count"]
    launches = 0
    with launch_policy(**fields):
        reset_stats()
        before = get_stats()["safety_net_ranges"]
        for chunk, n in ((32768, 120), (1152, 700), (73728, 60)):
            s = KVSetup(VLLM, 6, 2, n + 50, n + 50, chunk, "BLOCKFIRST", seed=chunk)
            dev = s.to_device(gpu_device)
            rng = np.random.default_rng(chunk)
            for h2d in (False, True, False, True):
                g, c = rng.permutation(n + 50)[:n], rng.permutation(n + 50)[:n]
                dev.transfer(g, c, is_h2d=h2d)
                s.oracle_transfer(g, c, h2d)
                launches += 1
            dev.assert_matches_reference(f"{mode}, chunk {chunk}")
        st = get_stats()
    assert st["kernel_launches"] == launches
    if mode in ("arbiter_off", "claims_on_all_xcds") or xcds < 4:
        assert st["confined_launches"] == 0 or mode == "safety_net", st
    if mode in ("confined", "home") and xcds >= 4:
        assert st["confined_launches"] == launches, st
    if mode == "safety_net":
        assert st["confined_launches"] == launches, st
        assert st["safety_net_ranges"] - before > 0, st   # the fallback workgroup did the work


@pytest.mark.parametrize("lane_runs", [0, 1, 2])
def test_both_store_orders_towards_host_memory(gpu_device, lane_runs):
    """GPU->host launches with 16-byte vectors store either 1 KiB per wavefront access
    or 128 adjacent bytes per lane (d2h_lane_runs: never / unless the link is busy the
    other way / always, here also with launches forced into the busy shape).  Whole
    slices, chunks that end in a short slice, chunks shorter than a slice, 8-byte
    vectors and the fused launch of several groups: the oracle's bytes every time."""
    from flexkv_amd.c_ext import launch_policy
    for arbiter in (1, 2):
        with launch_policy(d2h_lane_runs=lane_runs, arbiter=arbiter):
            for chunk, n in ((32768, 90), (18432, 70), (8192 + 16, 64), (2304, 300), (4104, 80)):
                s = KVSetup(VLLM, 5, 2, n + 20, n + 20, chunk, "BLOCKFIRST", seed=chunk + lane_runs)
                dev = s.to_device(gpu_device)
                rng = np.random.default_rng(chunk)
                for h2d in (False, True, False):
                    g, c = rng.permutation(n + 20)[:n], rng.permutation(n + 20)[:n]
                    print(f"case lane_runs={lane_runs} arbiter={arbiter} chunk={chunk} h2d={h2d}",
                          flush=True)
                    dev.transfer(g, c, is_h2d=h2d)
                    s.oracle_transfer(g, c, h2d)
                dev.assert_matches_reference(f"lane_runs={lane_runs}, chunk {chunk}")


def test_the_launch_policy_follows_the_device(gpu_device):
    """Masks are derived from the XCDs the device exposes: disjoint halves for the
    two directions, the home XCDs of a direction include its busy XCDs, and a set
    never names an XCD the device lacks."""
    from flexkv_amd.c_ext import get_launch_policy, reset_launch_policy, set_launch_policy
    p = get_launch_policy()
    present = p["xcd_present_mask"]
    assert p["xcd_count"] == bin(present).count("1") >= 1
    for name in ("d2h_busy_mask", "h2d_busy_mask", "d2h_home_mask", "h2d_home_mask"):
        assert p[name] and p[name] & ~present == 0, (name, p)
    if p["xcd_count"] >= 4:
        assert p["d2h_busy_mask"] & p["h2d_busy_mask"] == 0
        assert p["d2h_home_mask"] & p["h2d_home_mask"] == 0
        assert p["d2h_busy_mask"] & ~p["d2h_home_mask"] == 0
    q = set_launch_policy(d2h_busy_mask=0xffff0000 | present, busy_window_ms=-5, staged_ring=99)
    assert q["d2h_busy_mask"] == present and q["busy_window_ms"] == 0 and q["staged_ring"] == 8
    with pytest.raises(ValueError):
        set_launch_policy(no_such_field=1)
    reset_launch_policy()
    assert get_launch_policy() == p


def test_the_cost_model_is_rebased_on_this_device(gpu_device):
    """The figures of the cost model that depend on the host link come from a
    measurement of the device, taken once: plausible for any PCIe slot, stable across
    calls, kept by a reset, and a figure the caller has set beforehand stays."""
    from flexkv_amd.c_ext import (get_launch_policy, reset_launch_policy, seed_launch_policy,
                                  set_launch_policy)
    p = seed_launch_policy()
    assert p["model_seeded"] == 1
    assert 5000 < p["model_link_mbps"] < 130000, p
    for k in ("model_kernel_d2h_mbps", "model_kernel_h2d_mbps"):
        assert 0.8 * p["model_link_mbps"] < p[k] < 1.25 * p["model_link_mbps"], (k, p)
    assert abs(p["link_gbps_estimate"] - p["model_link_mbps"] * 45 / 57200e0) <= 1.0
    assert 1 <= p["staged_copy_overhead_us"] <= 200, p
    assert seed_launch_policy() == p                  # measured once
    set_launch_policy(model_link_mbps=12345)
    assert seed_launch_policy()["model_link_mbps"] == 12345
    reset_launch_policy()
    assert get_launch_policy() == p                   # the reset keeps the measurement


def test_lane_streams_keep_the_order_of_the_callers_stream(gpu_device):
    """FKV_LANE_STREAMS=1 (read once per process, hence a child process): transfers
    run on the library's own two streams.  What the caller's stream held before a
    call is finished before the transfer starts, and work queued on the caller's
    stream behind an asynchronous call sees the transferred bytes; puts and gets
    from several threads and streams at once still land where they belong."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = (
        "import sys, threading; sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + '/tests')\n"
        "import numpy as np, torch\n"
        "from kvsetup import KVSetup\n"
        "s = KVSetup(0, 4, 2, 96, 96, 65536, 'BLOCKFIRST', seed=5)\n"
        "dev = s.to_device('cuda:0')\n"
        "st = torch.cuda.Stream()\n"
        "big = torch.empty(1 << 28, dtype=torch.uint8, device='cuda')\n"
        "ids = np.arange(8)\n"
        "with torch.cuda.stream(st):\n"
        "    for rep in range(5):\n"
        "        # (1) the stream is busy, then overwrites the blocks; the put must see that\n"
        "        for _ in range(4): big.add_(1)\n"
        "        for l, t in enumerate(dev.gpu):\n"
        "            t.view(torch.uint8).view(2, 96, -1)[:, :8] = rep * 16 + l\n"
        "            s.gpu_ref[l].view(np.uint8).reshape(2, 96, -1)[:, :8] = rep * 16 + l\n"
        "        dev.transfer(ids, ids + 40, is_h2d=False)          # synchronous\n"
        "        s.oracle_transfer(ids, ids + 40, False)\n"
        "        # (2) asynchronous get; a copy queued behind it on the stream must see it\n"
        "        dev.transfer(ids + 20, ids + 40, is_h2d=True, sync=False)\n"
        "        s.oracle_transfer(ids + 20, ids + 40, True)\n"
        "        seen = [t.view(torch.uint8).view(2, 96, -1)[:, 20:28].clone() for t in dev.gpu]\n"
        "        st.synchronize()\n"
        "        for l, x in enumerate(seen):\n"
        "            assert int(x.min()) == int(x.max()) == rep * 16 + l, (rep, l, int(x.min()), int(x.max()))\n"
        "dev.assert_matches_reference('ordering')\n"
        "# (3) eight threads, eight streams, puts and gets of disjoint blocks\n"
        "rng = np.random.default_rng(2)\n"
        "pg, pc = rng.permutation(96), rng.permutation(96)\n"
        "errs = []\n"
        "def work(i):\n"
        "    try:\n"
        "        with torch.cuda.stream(torch.cuda.Stream()):\n"
        "            for k in range(3):\n"
        "                lo = (i * 3 + k) * 4\n"
        "                dev.transfer(pg[lo:lo + 4], pc[lo:lo + 4], is_h2d=(i % 2 == 1))\n"
        "    except Exception as e:\n"
        "        errs.append(e)\n"
        "ths = [threading.Thread(target=work, args=(i,)) for i in range(8)]\n"
        "[t.start() for t in ths]; [t.join() for t in ths]\n"
        "assert not errs, errs\n"
        "for i in range(8):\n"
        "    for k in range(3):\n"
        "        lo = (i * 3 + k) * 4\n"
        "        s.oracle_transfer(pg[lo:lo + 4], pc[lo:lo + 4], i % 2 == 1)\n"
        "torch.cuda.synchronize()\n"
        "dev.assert_matches_reference('threads')\n"
        "print('ok')\n")
    env = dict(os.environ, FKV_LANE_STREAMS="1")
    r = subprocess.run([sys.executable, "-c", script, root], env=env, capture_output=True,
                       text=True, timeout=170)
    assert r.returncode == 0 and r.stdout.split()[-1:] == ["ok"], r.stdout + r.stderr


@pytest.mark.parametrize("chunk,n", [(64, 200000), (16384, 12000)], ids=["200k-x-64B", "12k-x-16KiB"])
def test_very_many_blocks_in_one_call(gpu_device, chunk, n):
    """Hundreds of thousands of block positions in one call: plan memory of several
    MiB, hundreds of id tiles per workgroup, work-unit counts beyond 2^21 (packed
    mode for the short chunks)."""
    s = KVSetup(VLLM, 2, 2, n + 1000, n + 1000, chunk, "BLOCKFIRST", seed=n)
    dev = s.to_device(gpu_device)
    rng = np.random.default_rng(n)
    gids, cids = rng.permutation(n + 1000)[:n], rng.permutation(n + 1000)[:n]
    dev.transfer(gids, cids, is_h2d=False)
    s.oracle_transfer(gids, cids, False)
    dev.assert_matches_reference(f"{n} blocks D2H")
    back = rng.permutation(n + 1000)[:n]
    dev.transfer(back, cids, is_h2d=True)
    s.oracle_transfer(back, cids, True)
    dev.assert_matches_reference(f"{n} blocks H2D")


# ---- several transfers in one call (fkv_transfer_kv_blocks_multi) ----------------------

def _multi_call(devs, gids, cids, h2d, engines=None, sync=True, **kw):
    """One descriptor per device-side setup, all with the same block ids."""
    import torch
    from flexkv_amd.c_ext import transfer_kv_blocks_multi
    g = torch.as_tensor(np.asarray(gids, dtype=np.int64))
    c = torch.as_tensor(np.asarray(cids, dtype=np.int64))
    calls = []
    for i, dev in enumerate(devs):
        s = dev.s
        calls.append(((g, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride, c,
                       dev.host, s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride,
                       s.chunk, 0, s.num_layers),
                      dict(kw, is_host_to_device=h2d, kv_dim=s.kv_dim, gpu_block_type=s.backend,
                           is_blockfirst=s.cpu_layout == "BLOCKFIRST", sync=sync,
                           use_ce_transfer=engines[i] if engines else False)))
    transfer_kv_blocks_multi(calls)


@pytest.mark.parametrize("case", ["alike", "mixed_widths", "six_groups", "with_copy_engine"])
def test_several_transfers_in_one_call_match_oracle(gpu_device, case):
    from flexkv_amd.c_ext import get_stats, reset_stats
    setups = {
        # same vector width and launch shape: one launch
        "alike": [KVSetup(VLLM, 5, 2, 40, 40, 4096, "BLOCKFIRST", seed=21),
                  KVSetup(VLLM, 3, 1, 40, 40, 1024, "LAYERFIRST", seed=22),
                  KVSetup(SGLANG, 2, 2, 40, 40, 2048, "BLOCKFIRST", seed=23)],
        # a 200-byte chunk needs 8-byte vectors: launches of its own
        "mixed_widths": [KVSetup(VLLM, 4, 2, 40, 40, 4096, "BLOCKFIRST", seed=24),
                         KVSetup(VLLM, 4, 1, 40, 40, 200, "BLOCKFIRST", seed=25),
                         KVSetup(TRTLLM, 2, 2, 40, 40, 512, "BLOCKFIRST", seed=26)],
        # more than one launch holds
        "six_groups": [KVSetup(VLLM, 2 + i, 1 + i % 2, 40, 40, 256 << i, "BLOCKFIRST", seed=30 + i)
                       for i in range(6)],
        "with_copy_engine": [KVSetup(VLLM, 3, 2, 40, 40, 4096, "BLOCKFIRST", seed=27),
                             KVSetup(VLLM, 3, 2, 40, 40, 8192, "LAYERFIRST", seed=28)],
    }[case]
    engines = [False, True] if case == "with_copy_engine" else None
    devs = [s.to_device(gpu_device) for s in setups]
    rng = np.random.default_rng(9)
    gids, cids = block_ids(rng, 40, 17), block_ids(rng, 40, 17)
    for h2d in (False, True):
        reset_stats()
        _multi_call(devs, gids, cids, h2d, engines)
        for s in setups:
            s.oracle_transfer(gids, cids, h2d)
        for i, dev in enumerate(devs):
            dev.assert_matches_reference(f"{case} member {i} h2d={h2d}")
        st = get_stats()
        assert st["calls"] == len(setups)
        want = sum(17 * s.num_layers * s.kv_dim * s.chunk for s in setups)
        assert st["bytes_h2d" if h2d else "bytes_d2h"] == want
        if case == "alike":
            assert st["kernel_launches"] == 1
        elif case == "six_groups":
            assert st["kernel_launches"] == 2
        gids, cids = block_ids(rng, 40, 17), block_ids(rng, 40, 17)


def test_several_transfers_in_one_call_edge_cases(gpu_device):
    import torch
    from flexkv_amd.c_ext import transfer_kv_blocks_multi
    a = KVSetup(VLLM, 2, 2, 16, 16, 1024, "BLOCKFIRST", seed=41)
    b = KVSetup(VLLM, 3, 2, 16, 16, 2048, "BLOCKFIRST", seed=42)
    da, db = a.to_device(gpu_device), b.to_device(gpu_device)
    transfer_kv_blocks_multi([])
    none = np.empty(0, dtype=np.int64)
    _multi_call([da, db], none, none, False)
    da.assert_matches_reference("no blocks")
    db.assert_matches_reference("no blocks")

    # the last descriptor's sync flag governs: without it the caller waits on the stream
    ids, host_ids = np.array([3, 1, 8], dtype=np.int64), np.array([0, 5, 2], dtype=np.int64)
    _multi_call([da, db], ids, host_ids, False, sync=False)
    torch.cuda.synchronize()
    for s in (a, b):
        s.oracle_transfer(ids, host_ids, False)
    da.assert_matches_reference("asynchronous")
    db.assert_matches_reference("asynchronous")

    # an empty member between two others is skipped
    g = torch.as_tensor(ids)
    c = torch.as_tensor(host_ids)
    e = torch.as_tensor(none)

    def call(dev, gi, ci, h2d):
        s = dev.s
        return ((gi, dev.ptrs, s.gpu_kv_stride, s.gpu_block_stride, s.gpu_layer_stride, ci,
                 dev.host, s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, s.chunk, 0,
                 s.num_layers), dict(is_host_to_device=h2d, kv_dim=s.kv_dim, sync=True))
    transfer_kv_blocks_multi([call(da, c, g, True), call(db, e, e, True), call(db, c, g, True)])
    for s in (a, b):
        s.oracle_transfer(host_ids, ids, True)
    da.assert_matches_reference("empty member in the middle")
    db.assert_matches_reference("empty member in the middle")

    # both directions in one call are refused before anything moves
    with pytest.raises(ValueError, match="direction"):
        transfer_kv_blocks_multi([call(da, g, c, False), call(db, c, g, True)])
    da.assert_matches_reference("refused call")
    db.assert_matches_reference("refused call")


# ---- seeded random cases: every engine and entry point against the oracle ---------------
def _random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    backend = int(rng.choice([VLLM, TRTLLM, SGLANG]))
    L, K = int(rng.integers(1, 7)), int(rng.choice([1, 2]))
    if backend == SGLANG:
        K = 2
    N, NH = int(rng.integers(4, 90)), int(rng.integers(4, 90))
    gran = int(rng.choice([16, 16, 16, 8, 4, 2, 1]))          # vector width the chunk allows
    chunk = gran * int(rng.integers(1, 1 + 20000 // gran)) if rng.random() < 0.7 else \
        gran * int(rng.integers(1, 40))
    if gran < 16 and chunk % (2 * gran) == 0:
        chunk += gran
    cpu_layout = str(rng.choice(["BLOCKFIRST", "LAYERFIRST"]))
    gpu_layout = str(rng.choice(["LAYERFIRST", "LAYERBLOCK"])) if backend == VLLM else "LAYERFIRST"
    pad = int(rng.choice([0, 0, 16 * int(rng.integers(1, 9))])) if gran == 16 else 0
    n = int(rng.integers(1, min(N, NH) + 1))
    start = int(rng.integers(0, L))
    nl = int(rng.integers(1, L - start + 1))
    # an in-chunk window, as a rank that moves its share of every chunk would ask for
    if rng.random() < 0.3 and chunk >= 4 * gran:
        sub = gran * int(rng.integers(1, chunk // gran))
        g_off = gran * int(rng.integers(0, (chunk - sub) // gran + 1))
        c_off = gran * int(rng.integers(0, (chunk - sub) // gran + 1))
    else:
        sub, g_off, c_off = chunk, 0, 0
    return dict(backend=backend, L=L, K=K, N=N, NH=NH, chunk=chunk, cpu_layout=cpu_layout,
                gpu_layout=gpu_layout, pad=pad, n=n, start=start, nl=nl, sub=sub, g_off=g_off,
                c_off=c_off, rng=rng)


@pytest.mark.parametrize("seed", range(48))
def test_seeded_random_cases_on_every_engine(gpu_device, seed):
    """Shapes, strides, id lists, layer ranges and in-chunk windows drawn from a seed: a put
    and a get on the kernel path (two workgroup counts), through the copy-engine strategies
    (the library's choice and per-block copies; whole chunks with 8-byte granularity, which
    is their domain) and through the entry point that allocates nothing, each compared with
    the oracle byte for byte on the whole host pool and every engine tensor."""
    c = _random_case(seed)
    rng = c["rng"]
    s = KVSetup(c["backend"], c["L"], c["K"], c["N"], c["NH"], c["chunk"], c["cpu_layout"],
                c["gpu_layout"], seed=2000 + seed, gpu_block_pad=c["pad"])
    dev = s.to_device(gpu_device)
    print("case", {k: v for k, v in c.items() if k != "rng"}, flush=True)
    engines = [dict(num_cta=1), dict(num_cta=int(rng.integers(2, 40))),
               dict(entry="fkv_transfer_kv_blocks_noalloc")]
    if c["sub"] == c["chunk"] and c["chunk"] % 8 == 0:
        engines += [dict(use_ce=True, ce=dict(path_opt_enabled=1)),
                    dict(use_ce=True, ce=dict(path_opt_enabled=1, enable_memcpy2d=1,
                                              segment_threshold=2)),
                    dict(use_ce=True, ce=dict(path_opt_enabled=0))]
    for kw in engines:
        gids = rng.permutation(c["N"])[:c["n"]].astype(np.int64)
        cids = rng.permutation(c["NH"])[:c["n"]].astype(np.int64)
        for h2d in (False, True):
            rc = dev.transfer_raw(gids, cids, h2d, start_layer=c["start"], num_layers=c["nl"],
                                  gpu_off=c["g_off"], cpu_off=c["c_off"], chunk=c["sub"], **kw)
            assert rc == 0, (kw, h2d, _last_error())
            s.oracle_transfer(gids, cids, h2d, start_layer=c["start"], num_layers=c["nl"],
                              gpu_off=c["g_off"], cpu_off=c["c_off"], chunk=c["sub"])
            dev.assert_matches_reference(f"{kw} h2d={h2d}")
            gids = rng.permutation(c["N"])[:c["n"]].astype(np.int64)   # the get lands elsewhere


def _last_error():
    from flexkv_amd import _lib
    return _lib.last_error()
