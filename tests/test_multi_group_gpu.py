"""Layerwise restore of heterogeneous layer groups and sliding-window sidecars on
the GPU: the known-answer cases of the reference's tests
(tests/test_layerwise_multi_group_swa.py, test_layerwise_eventfd_timing.py,
test_layerwise_dsv4_multi_group_swa_roundtrip.py) and comparisons with the
oracle on seeded random pools."""
import ctypes
import os
import struct

import numpy as np
import pytest
import torch

from flexkv_amd.layout import LayerGroupSpec, TransferStrides
from mgsetup import (CPU_SRC, GPU_DST, INDEXER_HEAD_SIZE, MAIN_HEAD_SIZE, SWA_CPU_SRC,
                     SWA_GPU_DST, MGCase, main_seed, swa_layout_of, swa_seed)

pytestmark = pytest.mark.gpu

ENGINES = [False, True, "auto"]


@pytest.fixture(autouse=True, params=[
    dict(staged_restore=1, staged_gather=1), dict(staged_restore=2, staged_gather=0),
    dict(staged_restore=0, staged_gather=2, gather_first_by_kernel=0, gather_threads=3, gather_ring=2),
    dict(staged_restore=0, staged_gather=2, gather_first_by_kernel=1, gather_threads=2)],
    ids=["restore_as_chosen", "restore_by_copy_engines", "restore_gathered",
         "restore_gathered_first_by_kernel"])
def _staged_restore(request):
    """Every case four times: with the library's own choice of route (the small pools here
    stay on the kernel path), with the kernel-path restores forced through the copy engines
    and a staging ring one copy per run of host blocks, and with the rows of every group
    member and sidecar gathered by host threads first (batches launched one by one from the
    library's own thread; with and without the first batch by kernel)."""
    from flexkv_amd.c_ext import launch_policy
    with launch_policy(**request.param):
        yield


def _t6_groups(num_layers=4):
    main = LayerGroupSpec(num_layers, 1, MAIN_HEAD_SIZE, tuple(range(num_layers)), itemsize=1)
    indexer = LayerGroupSpec(3, 1, INDEXER_HEAD_SIZE, (1, 2, 3), itemsize=1)
    return [main, indexer]


def _t4_groups():
    return [LayerGroupSpec(3, 1, MAIN_HEAD_SIZE, (1, 2, 3), itemsize=1)]


def _check_known_answers(dev, exp_main, exp_swa):
    for (orig, gi, local), exp in exp_main.items():
        got = dev.main_block(gi, local, GPU_DST)
        assert np.array_equal(got, exp), f"main group={gi} orig={orig} local={local}"
        rest = np.delete(dev.gpu[gi][local].cpu().numpy(), GPU_DST, axis=0)
        assert not rest.any(), "bytes outside the destination block were written"
    for orig, exp in exp_swa.items():
        assert np.array_equal(dev.swa_block(orig, SWA_GPU_DST), exp), f"SWA orig={orig}"
        assert not np.delete(dev.swa_gpu[orig].cpu().numpy(), SWA_GPU_DST, axis=0).any()


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("notify", ["hostfunc", "polling"])
def test_t6_main_indexer_and_swa(gpu_device, engine, notify):
    case = MGCase(_t6_groups(), 4)
    exp_main, exp_swa = case.seed_all_main(), case.seed_all_swa()
    dev = case.to_device(gpu_device)
    dev.run_h2d(swa=([SWA_CPU_SRC], [SWA_GPU_DST]), use_ce_transfer=engine, notify_mode=notify)
    _check_known_answers(dev, exp_main, exp_swa)
    dev.group.close()


@pytest.mark.parametrize("engine", ENGINES)
def test_t4_empty_member_layer_swa_only(gpu_device, engine):
    case = MGCase(_t4_groups(), 4)
    exp_main, exp_swa = case.seed_all_main(), case.seed_all_swa()
    dev = case.to_device(gpu_device)
    dev.run_h2d(swa=([SWA_CPU_SRC], [SWA_GPU_DST]), use_ce_transfer=engine)
    _check_known_answers(dev, exp_main, exp_swa)
    dev.group.close()


def test_no_sidecar_ids_leaves_the_sidecar_alone(gpu_device):
    case = MGCase(_t6_groups(), 4)
    exp_main = case.seed_all_main()
    case.seed_all_swa()
    dev = case.to_device(gpu_device)
    dev.run_h2d(swa=None, use_ce_transfer=False)
    _check_known_answers(dev, exp_main, {})
    assert not any(t.any().item() for t in dev.swa_gpu)
    dev.group.close()


# ---- eventfd contract, tests/test_layerwise_eventfd_timing.py ------------------------

_libc = ctypes.CDLL("libc.so.6", use_errno=True)
_EFD_SEMAPHORE, _EFD_NONBLOCK = 0x1, 0x800


def _eventfds(n):
    fds = []
    for _ in range(n):
        fd = _libc.eventfd(ctypes.c_uint(0), ctypes.c_int(_EFD_SEMAPHORE | _EFD_NONBLOCK))
        assert fd >= 0
        fds.append(fd)
    return fds


def _drain(fd):
    total = 0
    while True:
        try:
            data = os.read(fd, 8)
        except BlockingIOError:
            return total
        total += struct.unpack("Q", data)[0]


@pytest.fixture
def fd_table():
    made = []

    def make(num_counters, tp_size, num_layers):
        fds = _eventfds(num_counters * tp_size * num_layers)
        made.extend(fds)
        arr = np.asarray(fds, dtype=np.int32).reshape(num_counters, tp_size, num_layers)
        return torch.from_numpy(arr.copy()), arr
    yield make
    for fd in made:
        os.close(fd)


def _dsv4_like_groups(num_c4_layers):
    # tests/test_layerwise_eventfd_timing.py: c4 main + indexer on the first layers,
    # a c128 group on the rest
    c4 = tuple(range(num_c4_layers))
    rest = tuple(range(num_c4_layers, 2 * num_c4_layers))
    return [LayerGroupSpec(len(c4), 1, MAIN_HEAD_SIZE, c4, 1),
            LayerGroupSpec(len(rest), 1, MAIN_HEAD_SIZE, rest, 1),
            LayerGroupSpec(len(c4), 1, INDEXER_HEAD_SIZE, c4, 1)]


@pytest.mark.parametrize("notify", ["hostfunc", "polling"])
def test_eventfd_idle_then_one_unit_per_layer(gpu_device, fd_table, notify):
    num_layers = 8
    case = MGCase(_dsv4_like_groups(4), num_layers)
    case.seed_all_main()
    case.seed_all_swa()
    table, fds = fd_table(1, 1, num_layers)
    dev = case.to_device(gpu_device, eventfds=table)
    assert all(_drain(fd) == 0 for fd in fds.reshape(-1))  # silent before the transfer
    dev.run_h2d(swa=([SWA_CPU_SRC], [SWA_GPU_DST]), notify_mode=notify)
    for layer, fd in enumerate(fds[0, 0]):
        assert _drain(fd) == 1, f"layer {layer}"
        assert _drain(fd) == 0
    dev.group.close()


def test_dual_member_layer_posts_once(gpu_device, fd_table):
    case = MGCase(_t6_groups(), 4)
    case.seed_all_main()
    case.seed_all_swa()
    table, fds = fd_table(1, 1, 4)
    dev = case.to_device(gpu_device, eventfds=table)
    dev.run_h2d(swa=([SWA_CPU_SRC], [SWA_GPU_DST]))
    assert [_drain(fd) for fd in fds[0, 0]] == [1, 1, 1, 1]
    dev.group.close()


def test_empty_member_layer_immediate_post_without_sidecar_work(gpu_device, fd_table):
    case = MGCase(_t4_groups(), 4)
    case.seed_all_main()
    table, fds = fd_table(1, 1, 4)
    dev = case.to_device(gpu_device, eventfds=table)
    dev.run_h2d(swa=None)
    assert [_drain(fd) for fd in fds[0, 0]] == [1, 1, 1, 1]
    # the in-process wait on a layer nothing is attached to returns at once
    dev.group.wait_layer(0)
    dev.group.wait_layer(3)
    torch.cuda.synchronize()
    dev.group.close()


def test_empty_member_layer_posts_after_its_sidecar_copy(gpu_device, fd_table):
    case = MGCase(_t4_groups(), 4)
    exp_swa = case.seed_all_swa()
    table, fds = fd_table(1, 1, 4)
    dev = case.to_device(gpu_device, eventfds=table)
    dev.run_h2d(swa=([SWA_CPU_SRC], [SWA_GPU_DST]))
    assert [_drain(fd) for fd in fds[0, 0]] == [1, 1, 1, 1]
    assert np.array_equal(dev.swa_block(0, SWA_GPU_DST), exp_swa[0])
    dev.group.close()


def test_counter_and_tp_rank_indexing(gpu_device, fd_table):
    """Entry [counter, rank, layer] of the table, csrc/layerwise.cpp:15-34."""
    case = MGCase(_t4_groups(), 4)
    case.seed_all_main()
    table, fds = fd_table(3, 2, 4)
    dev = case.to_device(gpu_device, eventfds=table, tp_size=2)
    dev.run_h2d(swa=None, counter_id=2)
    units = np.vectorize(_drain)(fds)
    assert units[2].tolist() == [[1, 1, 1, 1], [1, 1, 1, 1]]
    assert not units[:2].any()
    dev.group.close()


# ---- the DSv4-shaped round trip -----------------------------------------------------------

@pytest.mark.parametrize("engine", ENGINES)
def test_dsv4_put_then_layerwise_get_round_trip(gpu_device, engine):
    from flexkv_amd.c_ext import transfer_kv_blocks
    c4, c128 = (0, 1, 2, 3), (4, 5, 6, 7)
    groups = [LayerGroupSpec(4, 1, 64, c4, 1, 4), LayerGroupSpec(4, 1, 32, c128, 1, 128),
              LayerGroupSpec(4, 1, 40, c4, 1, 4)]
    case = MGCase(groups, 8, tpb=128, swa_width=128)
    gpu_src, cpu_dst, gpu_back, swa_cpu_dst, swa_gpu_back = 1, 2, 5, 3, 6
    golden = {}
    for orig in range(8):
        for gi, local in case.members[orig]:
            g = groups[gi]
            golden[(gi, local)] = main_seed(orig, gi, local, 128 // g.compress_ratio, 1,
                                            g.head_size, mul=(97, 13, 7))
            case.gpu[gi][local][gpu_src] = golden[(gi, local)]
    swa_golden = {orig: swa_seed(orig, 128, 128, salt=0xD4) for orig in range(8)}
    for orig, v in swa_golden.items():
        case.swa_gpu[orig][gpu_src] = v
    dev = case.to_device(gpu_device)
    t = case.tables
    flat = dev.host.view(-1)
    for gi, g in enumerate(groups):  # PUT, one call per group into its slice of the block
        ptrs = torch.tensor([x.data_ptr() for x in dev.gpu[gi]], dtype=torch.int64)
        transfer_kv_blocks(
            torch.tensor([gpu_src], dtype=torch.int64), ptrs, t["group_gpu_kv_strides"][gi],
            t["group_gpu_block_strides"][gi], t["group_gpu_layer_strides"][gi],
            torch.tensor([cpu_dst], dtype=torch.int64), flat[t["group_cpu_offset_bytes"][gi]:],
            t["group_cpu_kv_strides"][gi], t["group_cpu_layer_strides"][gi],
            t["group_cpu_block_strides"][gi], t["group_chunk_sizes"][gi], 0, g.num_layers, 4,
            False, engine, 1, 0)
    s, c = case.swa_gpu_strides, case.swa_cpu_strides
    transfer_kv_blocks(
        torch.tensor([gpu_src], dtype=torch.int64),
        torch.tensor([x.data_ptr() for x in dev.swa_gpu], dtype=torch.int64), s.kv, s.block,
        s.layer, torch.tensor([swa_cpu_dst], dtype=torch.int64), dev.swa_host, c.kv, c.layer,
        c.block, c.chunk, 0, 8, 4, False, engine, 1, 0)
    torch.cuda.synchronize()
    for grp in dev.gpu:
        for x in grp:
            x.zero_()
    for x in dev.swa_gpu:
        x.zero_()
    torch.cuda.synchronize()
    dev.run_h2d(cpu_ids=[cpu_dst], gpu_ids=[gpu_back], swa=([swa_cpu_dst], [swa_gpu_back]),
                use_ce_transfer=engine)
    for (gi, local), v in golden.items():
        assert np.array_equal(dev.main_block(gi, local, gpu_back), v), (gi, local)
    for orig, v in swa_golden.items():
        assert np.array_equal(dev.swa_block(orig, swa_gpu_back), v), orig
    dev.group.close()


# ---- seeded random pools against the oracle ---------------------------------------------------

def _randomize(case, rng):
    case.host[:] = rng.integers(0, 256, case.host.size, dtype=np.uint8)
    case.swa_host[:] = rng.integers(0, 256, case.swa_host.shape, dtype=np.uint8)
    for grp in case.gpu:
        for a in grp:
            a[:] = rng.integers(0, 256, a.shape, dtype=np.uint8)
    for a in case.swa_gpu:
        a[:] = rng.integers(0, 256, a.shape, dtype=np.uint8)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("seed,nblk,nswa", [(1, 5, 3), (2, 24, 24), (3, 1, 0), (4, 0, 2), (5, 30, 7)])
def test_random_pools_match_the_oracle(gpu_device, engine, seed, nblk, nswa):
    from oracle import fkv_oracle as O
    rng = np.random.default_rng(seed)
    groups = [LayerGroupSpec(5, 1, 48, (0, 1, 2, 4, 5), 2, 1),     # bf16-wide main KV
              LayerGroupSpec(2, 1, 24, (3, 4), 2, 4),              # compressed group
              LayerGroupSpec(3, 1, 20, (0, 2, 5), 1, 2)]           # byte-wide indexer
    if seed == 5:
        # 200-byte chunks (8 tokens x 25 B): this group moves with 8-byte vectors while the
        # others move with 16, so the members of layers 0 and 2 cannot share a launch
        groups[2] = LayerGroupSpec(2, 1, 25, (0, 2), 1, 4)
    case = MGCase(groups, 7, tpb=32, num_gpu_blocks=40, num_cpu_blocks=48, swa_width=96)
    _randomize(case, rng)
    dev = case.to_device(gpu_device)
    gpu_ids = rng.permutation(40)[:nblk].tolist()
    cpu_ids = rng.permutation(48)[:nblk].tolist()
    swa_g = rng.permutation(40)[:nswa].tolist()
    swa_c = rng.permutation(48)[:nswa].tolist()
    swa = case.oracle_swa(swa_c, swa_g) if nswa else None
    immediate, work = O.layerwise_multi_group(1, case.oracle_groups(), case.members, case.host,
                                              gpu_ids, cpu_ids, 1, 1, "sharded", swa)
    assert immediate == ([6] if not nswa else [])
    from flexkv_amd.c_ext import get_launch_policy, get_stats, reset_stats
    reset_stats()
    dev.run_h2d(cpu_ids=cpu_ids, gpu_ids=gpu_ids, swa=(swa_c, swa_g) if nswa else None,
                use_ce_transfer=engine)
    pol, st = get_launch_policy(), get_stats()
    if engine is False and pol["staged_gather"] == 2 and pol["staged_restore"] == 0:
        # every group member and sidecar of every layer with work had its rows gathered
        # (less the first batch where that one goes by kernel)
        members = sum(len(m) for m in case.members) * (nblk > 0) + 7 * (nswa > 0)
        first = 0
        if pol["gather_first_by_kernel"]:
            first = len(case.members[0]) * (nblk > 0) + (nswa > 0)
        assert st["gathered_batches"] == members - first, (st, members, first)
    for gi, grp in enumerate(case.gpu):
        for local, ref in enumerate(grp):
            assert np.array_equal(dev.gpu[gi][local].cpu().numpy(), ref), (gi, local)
    for orig, ref in enumerate(case.swa_gpu):
        assert np.array_equal(dev.swa_gpu[orig].cpu().numpy(), ref), orig
    assert np.array_equal(dev.host.numpy(), case.host)  # a restore never writes the host pool
    dev.group.close()


@pytest.mark.parametrize("engine", [False, True])
def test_multi_group_sidecar_matches_the_oracle(gpu_device, engine):
    """A sidecar made of its own groups (init_swa_multi_group,
    csrc/layerwise.cpp:355-503): a ring group on every layer plus a state group
    on two of them, with its own host pool and its own block ids."""
    from oracle import fkv_oracle as O
    rng = np.random.default_rng(11)
    main = MGCase(_t6_groups(), 4, num_gpu_blocks=16, num_cpu_blocks=16)
    side = MGCase([LayerGroupSpec(4, 1, 64, (0, 1, 2, 3), 1, 1),
                   LayerGroupSpec(2, 1, 40, (1, 3), 1, 1)], 4, num_gpu_blocks=12,
                  num_cpu_blocks=10)
    _randomize(main, rng)
    _randomize(side, rng)
    dev = main.to_device(gpu_device, has_swa=False)
    side_host = torch.zeros(side.host.size, dtype=torch.uint8, pin_memory=True)
    side_host.copy_(torch.from_numpy(side.host))
    side_gpu = [[torch.from_numpy(a.copy()).to(gpu_device) for a in grp] for grp in side.gpu]
    st = side.tables
    dev.group.init_swa_multi_group(
        swa_gpu_blocks_per_group=[[g] for g in side_gpu], swa_cpu_blocks=side_host,
        swa_ssd_files={}, swa_layer_members=st["layer_members"],
        **{"swa_" + k: v for k, v in st.items() if k.startswith("group_")})
    with pytest.raises(RuntimeError, match="already initialized"):
        dev.group.init_swa_multi_group(
            swa_gpu_blocks_per_group=[[g] for g in side_gpu], swa_cpu_blocks=side_host,
            swa_ssd_files={}, swa_layer_members=st["layer_members"],
            **{"swa_" + k: v for k, v in st.items() if k.startswith("group_")})
    gpu_ids, cpu_ids = [3, 9, 4], [7, 0, 12]
    swa_g, swa_c = [11, 2], [5, 9]
    swa = {"kind": "multi", "groups": side.oracle_groups(), "members": side.members,
           "host": side.host, "gpu_ids": swa_g, "cpu_ids": swa_c}
    O.layerwise_multi_group(1, main.oracle_groups(), main.members, main.host, gpu_ids, cpu_ids,
                            1, 1, "sharded", swa)
    empty = torch.empty(0, dtype=torch.int64)
    dev.group.layerwise_transfer_multi_group(
        empty, empty, 0, 1, 4, torch.tensor(gpu_ids, dtype=torch.int64),
        torch.tensor(cpu_ids, dtype=torch.int64), 4, engine, 1, 1,
        swa_h2d_src=torch.tensor(swa_c, dtype=torch.int64),
        swa_h2d_dst=torch.tensor(swa_g, dtype=torch.int64))
    torch.cuda.synchronize()
    for gi, grp in enumerate(main.gpu):
        for local, ref in enumerate(grp):
            assert np.array_equal(dev.gpu[gi][local].cpu().numpy(), ref), ("main", gi, local)
    for gi, grp in enumerate(side.gpu):
        for local, ref in enumerate(grp):
            assert np.array_equal(side_gpu[gi][local].cpu().numpy(), ref), ("side", gi, local)
    dev.group.close()


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("granularity", [1, 3])
def test_single_group_with_uniform_sidecar(gpu_device, engine, granularity):
    """layerwise_transfer with swa_h2d_src/dst: every batch of layers is followed by
    the same layers of the sidecar (csrc/layerwise.cpp:1202-1209)."""
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    from kvsetup import KVSetup, VLLM
    from oracle import fkv_oracle as O
    rng = np.random.default_rng(21)
    L, nblk = 5, 6
    s = KVSetup(VLLM, num_layers=L, num_gpu_blocks=20, num_cpu_blocks=24, chunk=1536,
                kv_dim=2, cpu_layout="LAYERFIRST", seed=5)
    d = s.to_device(gpu_device)
    gpu_ids = rng.permutation(20)[:nblk].tolist()
    cpu_ids = rng.permutation(24)[:nblk].tolist()
    # the sidecar: a LAYERFIRST host pool and one device tensor per layer
    width, tpb, n_g, n_c = 80, 16, 10, 12
    cl, gl = swa_layout_of(L, n_c, tpb, width), swa_layout_of(L, n_g, tpb, width)
    cs, gs = TransferStrides.from_layout(cl, 1), TransferStrides.from_layout(gl, 1)
    swa_host_ref = rng.integers(0, 256, cl.kv_shape, dtype=np.uint8)
    swa_gpu_ref = [rng.integers(0, 256, (n_g, tpb, 1, width), dtype=np.uint8) for _ in range(L)]
    swa_host = torch.zeros(cl.kv_shape, dtype=torch.uint8, pin_memory=True)
    swa_host.copy_(torch.from_numpy(swa_host_ref))
    swa_gpu = [torch.from_numpy(a.copy()).to(gpu_device) for a in swa_gpu_ref]
    swa_g, swa_c = [7, 1, 4], [0, 11, 5]
    grp = LayerwiseTransferGroup(
        1, [d.gpu], d.host, {}, L, torch.tensor([s.gpu_kv_stride]),
        torch.tensor([s.gpu_block_stride]), torch.tensor([s.gpu_layer_stride]),
        torch.tensor([s.chunk]), 0, 0, torch.empty(0, dtype=torch.int32), 1,
        has_swa=True, swa_gpu_blocks=[swa_gpu], swa_cpu_blocks=swa_host,
        swa_gpu_kv_strides_tensor=torch.tensor([gs.kv]),
        swa_gpu_block_strides_tensor=torch.tensor([gs.block]),
        swa_gpu_layer_strides_tensor=torch.tensor([gs.layer]),
        swa_gpu_chunk_sizes_tensor=torch.tensor([gs.chunk]))
    empty = torch.empty(0, dtype=torch.int64)
    grp.layerwise_transfer(
        empty, empty, 0, 0, 0, 1, 4, torch.tensor(gpu_ids), torch.tensor(cpu_ids),
        s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride,
        s.cpu_layer_stride, 0, 4, engine, L, granularity, 2, 8,
        swa_h2d_src=torch.tensor(swa_c), swa_h2d_dst=torch.tensor(swa_g),
        swa_h2d_cpu_kv_stride_in_bytes=cs.kv, swa_h2d_cpu_layer_stride_in_bytes=cs.layer,
        swa_cpu_block_stride_in_bytes=cs.block)
    torch.cuda.synchronize()
    s.oracle_transfer(gpu_ids, cpu_ids, True)
    d.assert_matches_reference()
    O.transfer_c(O.BACKEND_VLLM, [a.ctypes.data for a in swa_gpu_ref], L, gs.kv, gs.block,
                 gs.layer, 0, swa_host_ref.ctypes.data, cs.kv, cs.layer, cs.block, 0, gs.chunk, 0,
                 L, 1, swa_g, swa_c, True)
    for l in range(L):
        assert np.array_equal(swa_gpu[l].cpu().numpy(), swa_gpu_ref[l]), l
    # the sidecar ids are optional per call
    grp.layerwise_transfer(
        empty, empty, 0, 0, 0, 1, 4, torch.tensor(gpu_ids), torch.tensor(cpu_ids),
        s.cpu_kv_stride, s.cpu_layer_stride, s.cpu_block_stride, s.chunk, s.cpu_kv_stride,
        s.cpu_layer_stride, 0, 4, engine, L, granularity, 2, 8)
    grp.close()


@pytest.mark.parametrize("engine", [False, True])
@pytest.mark.parametrize("entries", [0, 64], ids=["threads", "iouring"])
def test_blocks_and_sidecar_staged_from_ssd_files(gpu_device, tmp_path, engine, entries):
    """Step 0 of the multi-group restore: byte-flat blocks come out of the SSD
    files whole, the uniform sidecar layer by layer, into the host blocks the call
    names; then the restore proper runs on the refreshed pools
    (csrc/layerwise.cpp:1371-1432)."""
    from oracle import fkv_oracle as O
    rng = np.random.default_rng(31)
    case = MGCase(_t6_groups(), 4, num_gpu_blocks=16, num_cpu_blocks=12, swa_width=48)
    _randomize(case, rng)
    B, n_ssd, nfiles = case.block_stride, 18, 3
    main_files = [rng.integers(0, 256, (n_ssd // nfiles) * B, dtype=np.uint8)
                  for _ in range(nfiles)]
    swa_file_layout = swa_layout_of(4, n_ssd, case.tpb, 48).div_block(2, padding=True)
    fs = TransferStrides.from_layout(swa_file_layout, 1)
    swa_files = [rng.integers(0, 256, swa_file_layout.get_total_elements(), dtype=np.uint8)
                 for _ in range(2)]

    def write(arrays, tag):
        paths = []
        for i, a in enumerate(arrays):
            paths.append(str(tmp_path / f"{tag}_{i}.bin"))
            a.tofile(paths[-1])
        return {0: paths}
    dev = case.to_device(gpu_device, ssd_files=write(main_files, "main"),
                         swa_ssd_files=write(swa_files, "swa"), iouring_entries=entries)
    ssd_ids, staged = [17, 3, 10, 5], [11, 0, 6, 2]
    swa_ssd_ids, swa_staged = [9, 14, 0], [4, 10, 1]
    gpu_ids, cpu_ids = [3, 9, 4, 15, 0], [11, 7, 0, 2, 6]
    swa_g, swa_c = [11, 2, 6], [4, 9, 1]
    # expected host pools: whole blocks by the striping rule, sidecar through the oracle
    for sb, cb in zip(ssd_ids, staged):
        f, inf = sb % nfiles, sb // nfiles
        case.host[cb * B:(cb + 1) * B] = main_files[f][inf * B:(inf + 1) * B]
    c = case.swa_cpu_strides
    O.ssd_transfer(swa_files, 1, 2, 0, 4, case.swa_host.reshape(-1), swa_ssd_ids, swa_staged,
                   c.layer, c.kv, fs.layer, fs.kv, c.chunk, c.block, True, 1, 1)
    O.layerwise_multi_group(1, case.oracle_groups(), case.members, case.host, gpu_ids, cpu_ids,
                            1, 1, "sharded", case.oracle_swa(swa_c, swa_g))
    kw = dev.swa_call_kwargs(swa_c, swa_g)
    kw.update(swa_disk2h_src=torch.tensor(swa_ssd_ids), swa_disk2h_dst=torch.tensor(swa_staged),
              swa_ssd_layer_stride_in_bytes=fs.layer, swa_ssd_kv_stride_in_bytes=fs.kv,
              swa_num_blocks_per_file=n_ssd // 2)
    dev.group.layerwise_transfer_multi_group(
        torch.tensor(ssd_ids), torch.tensor(staged), n_ssd // nfiles, 1, 4,
        torch.tensor(gpu_ids), torch.tensor(cpu_ids), 4, engine, 1, 1, **kw)
    torch.cuda.synchronize()
    assert np.array_equal(dev.host.numpy(), case.host)
    assert np.array_equal(dev.swa_host.numpy(), case.swa_host)
    for gi, grp in enumerate(case.gpu):
        for local, ref in enumerate(grp):
            assert np.array_equal(dev.gpu[gi][local].cpu().numpy(), ref), (gi, local)
    for orig, ref in enumerate(case.swa_gpu):
        assert np.array_equal(dev.swa_gpu[orig].cpu().numpy(), ref), orig
    dev.group.close()


# ---- error behaviour ------------------------------------------------------------------------------

def test_wrong_entry_point_for_the_instance(gpu_device):
    case = MGCase(_t6_groups(), 4)
    dev = case.to_device(gpu_device)
    empty = torch.empty(0, dtype=torch.int64)
    ids = torch.tensor([1], dtype=torch.int64)
    with pytest.raises(RuntimeError, match=r"layerwise_transfer\(\) invoked on a multi-group"):
        dev.group.layerwise_transfer(empty, empty, 0, 0, 0, 1, 4, ids, ids, 0, 0, 0, 0, 0, 0, 0,
                                     4, False, 4, 1, 1, 1)
    dev.group.close()
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    from kvsetup import KVSetup, VLLM
    s = KVSetup(VLLM, num_layers=2, num_gpu_blocks=4, num_cpu_blocks=4, chunk=256, kv_dim=2,
                cpu_layout="LAYERFIRST", seed=1)
    d = s.to_device(gpu_device)
    grp = LayerwiseTransferGroup(
        1, [d.gpu], d.host, {}, 2, torch.tensor([s.gpu_kv_stride]),
        torch.tensor([s.gpu_block_stride]), torch.tensor([s.gpu_layer_stride]),
        torch.tensor([s.chunk]), 0, 0, torch.empty(0, dtype=torch.int32), 1)
    with pytest.raises(RuntimeError, match=r"layerwise_transfer_multi_group\(\) invoked on a "
                                           "single-group"):
        grp.layerwise_transfer_multi_group(empty, empty, 0, 1, 4, ids, ids, 4, False, 1, 1)
    grp.close()


def test_constructor_rejects_inconsistent_groups(gpu_device):
    case = MGCase(_t6_groups(), 4)
    dev = case.to_device(gpu_device)
    from flexkv_amd.c_ext import LayerwiseTransferGroup
    t = dict(case.tables)
    ctor = {k: t[k] for k in t if k.startswith("group_")}
    common = dict(num_gpus=1, cpu_blocks=dev.host, ssd_files={}, num_original_layers=4,
                  iouring_entries=512, iouring_flags=0,
                  layer_eventfds_tensor=torch.empty(0, dtype=torch.int32), tp_size=1)
    with pytest.raises(RuntimeError, match="layer_members must have length num_original_layers"):
        LayerwiseTransferGroup(gpu_blocks_per_group=[[g] for g in dev.gpu],
                               layer_members=t["layer_members"][:3], **ctor, **common)
    with pytest.raises(RuntimeError, match="does not match num_groups"):
        LayerwiseTransferGroup(gpu_blocks_per_group=[[dev.gpu[0]]],
                               layer_members=t["layer_members"], **ctor, **common)
    # two tensors for a group of four layers is none of the three device layouts
    with pytest.raises(RuntimeError, match="unsupported tensors_per_gpu=2 for num_layers=4"):
        LayerwiseTransferGroup(gpu_blocks_per_group=[[dev.gpu[0][:2]], [dev.gpu[1]]],
                               layer_members=t["layer_members"], **ctor, **common)
    with pytest.raises(RuntimeError, match="Failed to open file"):
        LayerwiseTransferGroup(gpu_blocks_per_group=[[g] for g in dev.gpu],
                               layer_members=t["layer_members"], **ctor,
                               **{**common, "ssd_files": {0: ["/nonexistent/x"]}})
    dev.group.close()
