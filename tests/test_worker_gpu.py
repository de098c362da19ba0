"""Transfer workers in their own processes, on the GPU: engine tensors shared
through both handle forms, ops submitted through the pipe and the shared op
pool, completions read from the queue, bytes checked against the oracle or by a
put -> erase -> get round trip."""
import os
import queue as pyqueue
import struct
import time

import numpy as np
import pytest
import torch
import torch.multiprocessing as mp

from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec,
                               MultiGroupBlockLayout, TransferStrides)
from flexkv_amd.transfer.eventfd_channel import make_eventfd, send_layer_eventfds
from flexkv_amd.transfer.memory_handle import TensorSharedHandle
from flexkv_amd.transfer.op_pool import SharedOpPool
from flexkv_amd.transfer.ops import LayerwiseTransferOp, TransferOp, TransferType
from flexkv_amd.transfer.worker import (GPUCPUTransferWorker, LayerwiseTransferWorker,
                                        PinnedPoolHandle, tpGPUCPUTransferWorker)

pytestmark = pytest.mark.gpu

I64 = np.int64
L, N_GPU, N_CPU, T, H, D = 4, 24, 32, 8, 2, 64
DT = torch.int16  # two-byte elements, like bf16 KV


def _gpu_layout(kv_dim=2, heads=H, layers=L):
    return KVCacheLayout(KVCacheLayoutType.LAYERFIRST, layers, N_GPU, T, heads, D, kv_dim=kv_dim,
                         num_kv_heads=heads)


def _cpu_layout(kind, kv_dim=2, heads=H, layers=L):
    return KVCacheLayout(kind, layers, N_CPU, T, heads, D, kv_dim=kv_dim, num_kv_heads=heads)


def _engine_tensors(device, seed, kv_dim=2, heads=H, layers=L):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(-30000, 30000, (kv_dim, N_GPU, T, heads, D), dtype=DT, generator=g)
            .to(device) for _ in range(layers)]


def _collect(q, n, timeout=120):
    got = []
    end = time.time() + timeout
    while len(got) < n:
        try:
            got.append(q.get(timeout=max(0.1, end - time.time())))
        except pyqueue.Empty:
            break
    return got


@pytest.fixture
def engine():
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    pool = SharedOpPool(16, 64)
    handles = []

    def start(cls, *args, **kw):
        h = cls.create_worker(ctx, q, pool.get_buffer(), *args, **kw)
        handles.append(h)
        h.wait_ready(180)
        return h
    yield start, q, pool
    for h in handles:
        if h.process.is_alive():
            h.shutdown()


def _op(kind, src, dst, pool=None, graph=0):
    op = TransferOp(graph, kind, np.asarray(src, dtype=I64), np.asarray(dst, dtype=I64))
    if pool is not None:
        op.src_slot_id = pool.allocate_slot(op.src_block_ids, 1)
        op.dst_slot_id = pool.allocate_slot(op.dst_block_ids, 2)
        assert op.src_slot_id >= 0 and op.dst_slot_id >= 0
    return op


@pytest.mark.parametrize("direct_ipc", [False, True])
@pytest.mark.parametrize("engine_kind", [False, True])
def test_worker_owned_pinned_pool_round_trip(gpu_device, engine, direct_ipc, engine_kind):
    """Put through the worker, erase, get into other blocks: the worker's pool is
    its own pinned allocation, so the copy kernel's path runs inside the worker."""
    start, q, pool = engine
    tensors = _engine_tensors(gpu_device, 1)
    want = [t.clone() for t in tensors]
    handles = [TensorSharedHandle(t, force_direct_ipc=direct_ipc) for t in tensors]
    assert handles[0].handle_type == ("hip_ipc" if direct_ipc else "torch_reduce")
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST)
    h = start(GPUCPUTransferWorker, handles, PinnedPoolHandle(cl.kv_shape, DT), _gpu_layout(), cl,
              DT, 0, use_ce_transfer_h2d=engine_kind, use_ce_transfer_d2h=engine_kind)
    assert h.control("ping")["pageable_host"] is False
    rng = np.random.default_rng(3)
    src_blocks = rng.permutation(N_GPU)[:10]
    host_blocks = rng.permutation(N_CPU)[:10]
    back_blocks = np.setdiff1d(np.arange(N_GPU), src_blocks)[:10]
    put = _op(TransferType.D2H, src_blocks, host_blocks, pool)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    get = _op(TransferType.H2D, host_blocks, back_blocks)  # ids travel with the op
    h.submit_transfer(get)
    assert _collect(q, 1) == [(get.op_id, True, None)]
    torch.cuda.synchronize()
    for l in range(L):
        assert torch.equal(tensors[l][:, back_blocks], want[l][:, src_blocks]), l
        untouched = np.setdiff1d(np.arange(N_GPU), back_blocks)
        assert torch.equal(tensors[l][:, untouched], want[l][:, untouched]), l
    # an op this worker cannot run is reported as failed, and the worker keeps serving
    e = np.array([], dtype=I64)
    wrong = LayerwiseTransferOp(0, TransferType.LAYERWISE, e, e)
    h.submit_transfer(wrong)
    assert _collect(q, 1) == [(wrong.op_id, False, None)]
    again = _op(TransferType.D2H, src_blocks[:2], host_blocks[:2])
    h.submit_transfer(again)
    assert _collect(q, 1) == [(again.op_id, True, None)]
    h.shutdown()
    assert h.process.exitcode == 0


@pytest.mark.parametrize("kind", [KVCacheLayoutType.BLOCKFIRST, KVCacheLayoutType.LAYERFIRST])
def test_shared_memory_pool_matches_the_oracle(gpu_device, engine, kind):
    """The reference's arrangement: the pool is a shared-memory tensor the engine
    can read.  The worker does not register foreign memory unless asked to
    (FKV_HOST_REGISTER=1, not set here): the pool stays pageable and everything moves
    with the copy engine."""
    from oracle import fkv_oracle as O
    start, q, pool = engine
    tensors = _engine_tensors(gpu_device, 2)
    cl, gl = _cpu_layout(kind), _gpu_layout()
    host = torch.zeros(cl.kv_shape, dtype=DT).share_memory_()
    h = start(GPUCPUTransferWorker, [TensorSharedHandle(t) for t in tensors], host, gl, cl, DT, 0,
              allow_pageable_host=True)
    assert h.control("ping")["pageable_host"] is True
    rng = np.random.default_rng(5)
    gpu_ids = rng.permutation(N_GPU)[:12]
    cpu_ids = rng.permutation(N_CPU)[:12]
    put = _op(TransferType.D2H, gpu_ids, cpu_ids, pool)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    ref_gpu = [t.cpu().numpy().view(np.uint8).reshape(-1) for t in tensors]
    ref_host = np.zeros(host.numel() * 2, dtype=np.uint8)
    gs, cs = TransferStrides.from_layout(gl, 2), TransferStrides.from_layout(cl, 2)
    O.transfer_c(O.BACKEND_VLLM, [a.ctypes.data for a in ref_gpu], L, gs.kv, gs.block, gs.layer, 0,
                 ref_host.ctypes.data, cs.kv, cs.layer, cs.block, 0, gs.chunk, 0, L, 2,
                 gpu_ids, cpu_ids, False)
    assert np.array_equal(host.numpy().view(np.uint8).reshape(-1), ref_host)
    h.shutdown()
    assert h.process.exitcode == 0


def test_multi_group_worker_round_trip(gpu_device, engine):
    """Layer groups of different width and compression behind one worker
    (worker.py:850-1030 of the reference): one call per group into its byte range of
    the host block."""
    start, q, pool = engine
    tpb = 32
    groups = [LayerGroupSpec(3, 1, 48, (0, 1, 2), 2, 1), LayerGroupSpec(2, 1, 24, (1, 2), 2, 4),
              LayerGroupSpec(2, 1, 40, (0, 2), 1, 2)]
    gpu_layouts = [KVCacheLayout(KVCacheLayoutType.LAYERFIRST, g.num_layers, N_GPU,
                                 tpb // g.compress_ratio, 1, g.head_size, kv_dim=1)
                   for g in groups]
    cl = MultiGroupBlockLayout(N_CPU, tpb, tuple(groups), kv_dim=1)
    gen = torch.Generator().manual_seed(9)
    per_group = [[torch.randint(0, 256, (N_GPU, tpb // g.compress_ratio, 1,
                                         g.head_size * g.itemsize), dtype=torch.uint8,
                                generator=gen).to(gpu_device) for _ in range(g.num_layers)]
                 for g in groups]
    want = [[t.clone() for t in grp] for grp in per_group]
    handles = [[TensorSharedHandle(t) for t in grp] for grp in per_group]
    h = start(GPUCPUTransferWorker, handles[0], PinnedPoolHandle(cl.kv_shape, torch.uint8),
              gpu_layouts[0], cl, torch.uint8, 0, layer_groups=groups,
              gpu_blocks_per_group=handles, gpu_layouts_per_group=gpu_layouts)
    src, mid, back = [1, 7, 3, 20], [9, 0, 31, 4], [11, 12, 13, 2]
    put, get = _op(TransferType.D2H, src, mid), _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(put)
    h.submit_transfer(get)
    assert _collect(q, 2) == [(put.op_id, True, None), (get.op_id, True, None)]
    torch.cuda.synchronize()
    for gi, grp in enumerate(per_group):
        for l, t in enumerate(grp):
            assert torch.equal(t[back], want[gi][l][src]), (gi, l)
    h.shutdown()


@pytest.mark.parametrize("heads,kv_dim,mode", [(4, 2, "sharded"), (1, 1, "sharded"),
                                               (1, 1, "rank0_only")])
def test_tp_worker_two_ranks_round_trip(gpu_device, engine, heads, kv_dim, mode, monkeypatch):
    """Two ranks of a tensor-parallel group (both placed on this GPU) behind one
    worker.  With separate heads each rank owns half the heads of every host
    chunk; with shared KV both ranks hold the same bytes."""
    import flexkv_amd.transfer.env as env
    monkeypatch.setenv("FLEXKV_KV_SHARED_ACROSS_RANKS_MODE", mode)
    monkeypatch.setattr(env, "_ENV", None)
    start, q, pool = engine
    tp = 2
    rank_heads = heads // tp if heads > 1 else 1
    ranks = [_engine_tensors(gpu_device, 20 + r if heads > 1 else 20, kv_dim, rank_heads)
             for r in range(tp)]
    want = [[t.clone() for t in ts] for ts in ranks]
    gl = [KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, N_GPU, T, rank_heads, D, kv_dim=kv_dim,
                        num_kv_heads=heads) for _ in range(tp)]
    cl = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, N_CPU, T, heads, D, kv_dim=kv_dim,
                       num_kv_heads=heads)
    h = start(tpGPUCPUTransferWorker, [[TensorSharedHandle(t) for t in ts] for ts in ranks],
              PinnedPoolHandle(cl.kv_shape, DT), gl, cl, DT, tp)
    src, mid, back = [2, 9, 5], [30, 1, 17], [20, 21, 22]
    put, get = _op(TransferType.D2H, src, mid, pool), _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(put)
    h.submit_transfer(get)
    assert _collect(q, 2) == [(put.op_id, True, None), (get.op_id, True, None)]
    torch.cuda.synchronize()
    for r in range(tp):
        for l in range(L):
            assert torch.equal(ranks[r][l][:, back], want[r][l][:, src]), (r, l)
    h.shutdown()
    monkeypatch.setattr(env, "_ENV", None)


@pytest.mark.parametrize("rank_heads,mode", [(1, "sharded"), (1, "rank0_only"), (2, "sharded")])
def test_tp_worker_layer_groups_round_trip(gpu_device, engine, rank_heads, mode, monkeypatch):
    """Layer groups behind the tensor-parallel worker (worker.py:1240-1383, 1461-1482
    of the reference): one thread group per layer group on its byte range of the host
    block.  One head: both ranks hold the same bytes and share one region of the
    block; two heads per rank: every rank has its own region, groups back to back
    inside it."""
    import flexkv_amd.transfer.env as env
    monkeypatch.setenv("FLEXKV_KV_SHARED_ACROSS_RANKS_MODE", mode)
    monkeypatch.setattr(env, "_ENV", None)
    start, q, pool = engine
    tp, tpb = 2, 32
    shared = rank_heads == 1
    total_heads = 1 if shared else rank_heads * tp
    groups = [LayerGroupSpec(3, rank_heads, 48, (0, 1, 2), 2, 1),
              LayerGroupSpec(2, rank_heads, 24, (1, 2), 2, 4),
              LayerGroupSpec(2, rank_heads, 40, (0, 2), 1, 2)]
    layouts = [[KVCacheLayout(KVCacheLayoutType.LAYERFIRST, g.num_layers, N_GPU,
                              tpb // g.compress_ratio, rank_heads, g.head_size, kv_dim=1,
                              num_kv_heads=total_heads) for _ in range(tp)] for g in groups]
    cl = MultiGroupBlockLayout(N_CPU, tpb, tuple(groups), kv_dim=1, tp_size=1 if shared else tp)
    # per group, per rank, per layer
    tensors = []
    for gi, g in enumerate(groups):
        per_rank = []
        for r in range(tp):
            gen = torch.Generator().manual_seed(100 + gi if shared else 100 + 10 * r + gi)
            per_rank.append([torch.randint(0, 256, (N_GPU, tpb // g.compress_ratio, rank_heads,
                                                    g.head_size * g.itemsize), dtype=torch.uint8,
                                           generator=gen).to(gpu_device)
                             for _ in range(g.num_layers)])
        tensors.append(per_rank)
    want = [[[t.clone() for t in ts] for ts in per_rank] for per_rank in tensors]
    handles = [[[TensorSharedHandle(t) for t in ts] for ts in per_rank] for per_rank in tensors]
    h = start(tpGPUCPUTransferWorker, handles[0], PinnedPoolHandle(cl.kv_shape, torch.uint8),
              layouts[0], cl, torch.uint8, tp, layer_groups=groups, gpu_blocks_per_group=handles,
              gpu_layouts_per_group=layouts)
    src, mid, back = [1, 7, 3, 20], [9, 0, 31, 4], [11, 12, 13, 2]
    put, get = _op(TransferType.D2H, src, mid, pool), _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(put)
    h.submit_transfer(get)
    assert _collect(q, 2) == [(put.op_id, True, None), (get.op_id, True, None)]
    torch.cuda.synchronize()
    for gi, per_rank in enumerate(tensors):
        for r, ts in enumerate(per_rank):
            for l, t in enumerate(ts):
                assert torch.equal(t[back], want[gi][r][l][src]), (gi, r, l)
                rest = [b for b in range(N_GPU) if b not in back]
                assert torch.equal(t[rest], want[gi][r][l][rest]), (gi, r, l, "other blocks")
    h.shutdown()
    monkeypatch.setattr(env, "_ENV", None)


@pytest.mark.parametrize("direct_ipc", [False, True])
def test_suspend_and_resume_gpu_blocks(gpu_device, engine, direct_ipc):
    """The engine frees its KV tensors and comes back with new ones
    (worker.py:928-962 of the reference): what was put before is restored into the
    new tensors; between the two controls an op fails instead of touching memory
    that is gone."""
    start, q, pool = engine
    first = _engine_tensors(gpu_device, 31)
    want = [t.clone() for t in first]
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST)
    h = start(GPUCPUTransferWorker,
              [TensorSharedHandle(t, force_direct_ipc=direct_ipc) for t in first],
              PinnedPoolHandle(cl.kv_shape, DT), _gpu_layout(), cl, DT, 0)
    src, mid, back = [4, 8, 15], [16, 23, 2], [1, 2, 3]
    put = _op(TransferType.D2H, src, mid, pool)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    assert h.control("suspend_gpu") == L
    assert h.control("suspend_gpu") == 0  # nothing left to let go
    lost = _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(lost)
    assert _collect(q, 1) == [(lost.op_id, False, None)]
    del first
    second = [torch.zeros_like(t) for t in want]
    # a handle made by torch's own sharing is good for one receiver: new ones for every send
    # (the worker opens and drops the ones it rejects, so that this process gets them back)
    fresh = lambda ts: [TensorSharedHandle(t, force_direct_ipc=direct_ipc) for t in ts]  # noqa: E731
    with pytest.raises(RuntimeError, match="Expected 4 GPU blocks"):
        h.control("resume_gpu", fresh(second[:2]))
    assert h.control("resume_gpu", fresh(second)) == L
    with pytest.raises(RuntimeError, match="already registered"):
        h.control("resume_gpu", fresh(second))
    get = _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(get)
    assert _collect(q, 1) == [(get.op_id, True, None)]
    torch.cuda.synchronize()
    for l in range(L):
        assert torch.equal(second[l][:, back], want[l][:, src]), l
        assert not second[l][:, [b for b in range(N_GPU) if b not in back]].any()
    h.shutdown()


def test_tp_worker_suspend_and_resume_gpu_blocks(gpu_device, engine):
    """The same for a tensor-parallel group of two ranks (worker.py:1385-1430)."""
    start, q, pool = engine
    tp, heads = 2, 4
    ranks = [_engine_tensors(gpu_device, 40 + r, 2, heads // tp) for r in range(tp)]
    want = [[t.clone() for t in ts] for ts in ranks]
    gl = [KVCacheLayout(KVCacheLayoutType.LAYERFIRST, L, N_GPU, T, heads // tp, D, kv_dim=2,
                        num_kv_heads=heads) for _ in range(tp)]
    cl = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, N_CPU, T, heads, D, kv_dim=2,
                       num_kv_heads=heads)
    h = start(tpGPUCPUTransferWorker, [[TensorSharedHandle(t) for t in ts] for ts in ranks],
              PinnedPoolHandle(cl.kv_shape, DT), gl, cl, DT, tp)
    src, mid, back = [2, 9, 5], [30, 1, 17], [20, 21, 22]
    put = _op(TransferType.D2H, src, mid, pool)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    assert h.control("suspend_gpu") == tp * L
    lost = _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(lost)
    assert _collect(q, 1) == [(lost.op_id, False, None)]
    del ranks
    second = [[torch.zeros_like(t) for t in ts] for ts in want]
    with pytest.raises(RuntimeError, match="Expected GPU block counts"):
        h.control("resume_gpu", [[TensorSharedHandle(t) for t in second[0]]])
    assert h.control("resume_gpu", [[TensorSharedHandle(t) for t in ts] for ts in second]) == tp * L
    get = _op(TransferType.H2D, mid, back, pool)
    h.submit_transfer(get)
    assert _collect(q, 1) == [(get.op_id, True, None)]
    torch.cuda.synchronize()
    for r in range(tp):
        for l in range(L):
            assert torch.equal(second[r][l][:, back], want[r][l][:, src]), (r, l)
    h.shutdown()


def _wait_units(fd, timeout=60.0):
    """Blocks like an engine does: one read per unit of the semaphore eventfd."""
    os.set_blocking(fd, True)
    import select
    r, _, _ = select.select([fd], [], [], timeout)
    assert r, "no notification"
    return struct.unpack("Q", os.read(fd, 8))[0]


@pytest.mark.parametrize("notify", ["hostfunc", "polling"])
def test_layerwise_worker_with_engine_eventfds(gpu_device, engine, tmp_path, notify,
                                               monkeypatch):
    """The engine hands its per-layer eventfds to the worker over the unix socket,
    submits a layerwise op and wakes up once per layer."""
    import threading
    import flexkv_amd.transfer.env as env
    monkeypatch.setenv("FLEXKV_LAYERWISE_NOTIFY_MODE", notify)
    monkeypatch.setattr(env, "_ENV", None)
    start, q, pool = engine
    kv_dim, heads, counters = 1, 1, 3
    tensors = _engine_tensors(gpu_device, 40, kv_dim, heads)
    want = [t.clone() for t in tensors]
    gl = _gpu_layout(kv_dim, heads)
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST, kv_dim, heads)
    sock = str(tmp_path / "lw.sock")
    fds = [[make_eventfd() for _ in range(L)] for _ in range(counters)]
    sender = threading.Thread(target=send_layer_eventfds, args=(sock, 0, 1, fds),
                              kwargs=dict(retry_interval_s=0.2))
    sender.start()
    # the host pool is shared memory, so the engine side of the test can fill it
    host = torch.zeros(cl.kv_shape, dtype=DT).share_memory_()
    src = [3, 8, 1, 15]
    mid = [4, 5, 20, 9]
    back = [10, 11, 12, 13]
    for l in range(L):  # the engine-side image of blocks `src` at host blocks `mid`
        host[mid, l, 0] = tensors[l][0, src].cpu()
    h = start(LayerwiseTransferWorker, [[TensorSharedHandle(t) for t in tensors]], host, [gl], cl,
              DT, 1, layerwise_eventfd_socket=sock, use_ce_transfer_h2d=False,
              allow_pageable_host=True)
    sender.join(60)
    assert not sender.is_alive()
    e = np.array([], dtype=I64)
    op = LayerwiseTransferOp(0, TransferType.LAYERWISE, e, e,
                             src_block_ids_h2d=np.asarray(mid, dtype=I64),
                             dst_block_ids_h2d=np.asarray(back, dtype=I64), counter_id=1)
    h.submit_transfer(op)
    for l in range(L):
        assert _wait_units(fds[1][l]) == 1   # layer l has landed
        assert torch.equal(tensors[l][:, back], want[l][:, src]), l
    assert _collect(q, 1) == [(op.op_id, True, None)]
    for c in (0, 2):  # the other counter sets stayed silent
        for fd in fds[c]:
            os.set_blocking(fd, False)
            with pytest.raises(BlockingIOError):
                os.read(fd, 8)
    h.shutdown()
    assert h.process.exitcode == 0
    for cs in fds:
        for fd in cs:
            os.close(fd)
    monkeypatch.setattr(env, "_ENV", None)


def test_layerwise_worker_stages_ssd_blocks_first(gpu_device, engine, tmp_path):
    """A layerwise op whose disk2h ids name blocks that live only in the SSD files:
    the worker reads them into the host pool, then restores everything."""
    from oracle import fkv_oracle as O
    start, q, pool = engine
    kv_dim, heads, n_ssd, nfiles = 1, 1, 20, 2
    tensors = _engine_tensors(gpu_device, 41, kv_dim, heads)
    gl = _gpu_layout(kv_dim, heads)
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST, kv_dim, heads)
    sl = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, n_ssd, T, heads, D, kv_dim=kv_dim,
                       num_kv_heads=heads)
    fl = sl.div_block(nfiles, padding=True)
    c, s = TransferStrides.from_layout(cl, 2), TransferStrides.from_layout(fl, 2)
    rng = np.random.default_rng(8)
    files = [rng.integers(0, 256, fl.get_total_elements() * 2, dtype=np.uint8)
             for _ in range(nfiles)]
    paths = {0: [str(tmp_path / f"ssd_{i}.bin") for i in range(nfiles)]}
    for a, p in zip(files, paths[0]):
        a.tofile(p)
    host = torch.zeros(cl.kv_shape, dtype=DT).share_memory_()
    host.view(torch.uint8).view(-1).copy_(torch.from_numpy(
        rng.integers(0, 256, host.numel() * 2, dtype=np.uint8)))
    ref_host = host.view(torch.uint8).view(-1).numpy().copy()
    ssd_ids, staged = [19, 4, 11], [30, 2, 7]
    src, dst = [30, 5, 2, 7, 16], [0, 23, 9, 1, 14]
    O.ssd_transfer(files, 1, nfiles, 0, L, ref_host, ssd_ids, staged, c.layer, c.kv, s.layer,
                   s.kv, c.chunk, c.block, True, 1, kv_dim)
    h = start(LayerwiseTransferWorker, [[TensorSharedHandle(t) for t in tensors]], host, [gl], cl,
              DT, 1, enable_eventfd=False, use_ce_transfer_h2d=False, allow_pageable_host=True,
              ssd_files=paths, ssd_kv_layout=sl, num_blocks_per_file=n_ssd // nfiles)
    e = np.array([], dtype=I64)
    op = LayerwiseTransferOp(0, TransferType.LAYERWISE, e, e,
                             src_block_ids_h2d=np.asarray(src, dtype=I64),
                             dst_block_ids_h2d=np.asarray(dst, dtype=I64),
                             src_block_ids_disk2h=np.asarray(ssd_ids, dtype=I64),
                             dst_block_ids_disk2h=np.asarray(staged, dtype=I64))
    h.submit_transfer(op)
    assert _collect(q, 1) == [(op.op_id, True, None)]
    assert np.array_equal(host.view(torch.uint8).view(-1).numpy(), ref_host)
    want = torch.from_numpy(ref_host).view(DT).view(cl.kv_shape)  # [block, layer, kv, ...]
    for l in range(L):
        assert torch.equal(tensors[l][:, dst].cpu(), want[src, l].transpose(0, 1)), l
    h.shutdown()
    assert h.process.exitcode == 0


@pytest.mark.parametrize("entries", [0, 64], ids=["threads", "iouring"])
def test_gpu_worker_that_also_serves_the_ssd_tier(gpu_device, engine, tmp_path, monkeypatch,
                                                  entries):
    """Three tiers behind one worker: the process that owns the pinned pool runs the
    kernel path GPU<->host and the host<->SSD ops on the same pool.  put -> spill ->
    wipe the host blocks -> stage back into other host blocks -> get."""
    monkeypatch.setenv("FLEXKV_IOURING_ENTRIES", str(entries))
    start, q, pool = engine
    n_ssd, nfiles = 40, 2
    tensors = _engine_tensors(gpu_device, 50)
    want = [t.clone() for t in tensors]
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST)
    sl = KVCacheLayout(KVCacheLayoutType.BLOCKFIRST, L, n_ssd, T, H, D, kv_dim=2, num_kv_heads=H)
    fl = sl.div_block(nfiles, padding=True)
    paths = {0: [str(tmp_path / f"tier_{i}.bin") for i in range(nfiles)]}
    for p in paths[0]:
        with open(p, "wb") as fh:
            fh.truncate(fl.get_total_elements() * 2)
    h = start(GPUCPUTransferWorker, [TensorSharedHandle(t) for t in tensors],
              PinnedPoolHandle(cl.kv_shape, DT), _gpu_layout(), cl, DT, 0,
              ssd_files=paths, ssd_kv_layout=sl, num_blocks_per_file=n_ssd // nfiles)
    rng = np.random.default_rng(12)
    gpu_src = rng.permutation(N_GPU)[:9]
    host_a = rng.permutation(N_CPU)[:9]
    ssd_ids = rng.permutation(n_ssd)[:9]
    host_b = np.setdiff1d(np.arange(N_CPU), host_a)[:9]
    gpu_dst = np.setdiff1d(np.arange(N_GPU), gpu_src)[:9]
    zero_src = np.setdiff1d(np.arange(N_GPU), np.concatenate([gpu_src, gpu_dst]))[:1]
    for t in tensors:
        t[:, zero_src] = 0                                      # a block of zeros to wipe with
    torch.cuda.synchronize()
    ops = [_op(TransferType.D2H, gpu_src, host_a, pool),        # put
           _op(TransferType.H2DISK, host_a, ssd_ids),           # spill
           _op(TransferType.D2H, np.repeat(zero_src, 9), host_a),   # wipe the host copies
           _op(TransferType.DISK2H, ssd_ids, host_b),           # stage back elsewhere
           _op(TransferType.H2D, host_b, gpu_dst)]              # get
    for op in ops:
        h.submit_transfer(op)
        assert _collect(q, 1) == [(op.op_id, True, None)]
    torch.cuda.synchronize()
    for l in range(L):
        assert torch.equal(tensors[l][:, gpu_dst], want[l][:, gpu_src]), l
    h.shutdown()
    assert h.process.exitcode == 0


def test_gpu_worker_runs_gets_next_to_puts(gpu_device, engine):
    """overlap_directions: D2H and H2D ops each run on a thread and stream of their
    own.  Five ops are submitted back to back; the put that overwrites host blocks
    an unfinished get still reads has to wait for that get, the get that reads what
    an unfinished put writes for that put, the others may overlap.  Every op is
    reported once, in whatever order."""
    start, q, pool = engine
    tensors = _engine_tensors(gpu_device, 77)
    want = [t.clone() for t in tensors]
    cl = _cpu_layout(KVCacheLayoutType.BLOCKFIRST)
    h = start(GPUCPUTransferWorker, [TensorSharedHandle(t) for t in tensors],
              PinnedPoolHandle(cl.kv_shape, DT), _gpu_layout(), cl, DT, 0,
              overlap_directions=True)
    rng = np.random.default_rng(21)
    perm = rng.permutation(N_GPU)
    P, G1, G2, G3, G4 = perm[:8], perm[8:12], perm[12:16], perm[16:20], perm[20:24]
    hperm = rng.permutation(N_CPU)
    HA, HB = hperm[:8], hperm[8:12]
    first = _op(TransferType.D2H, P, HA, pool)
    h.submit_transfer(first)
    assert _collect(q, 1) == [(first.op_id, True, None)]
    ops = [_op(TransferType.H2D, HA[:4], G1),        # reads host HA[:4]
           _op(TransferType.D2H, P[4:8], HA[:4]),    # overwrites them: after that get
           _op(TransferType.H2D, HA[4:], G2),
           _op(TransferType.D2H, P[:4], HB),
           _op(TransferType.H2D, HB, G4)]            # reads what the put before it writes
    for op in ops:
        h.submit_transfer(op)
    done = _collect(q, 5)
    assert sorted(d[0] for d in done) == sorted(op.op_id for op in ops) and all(d[1] for d in done)
    last = _op(TransferType.H2D, HA[:4], G3)
    h.submit_transfer(last)
    assert _collect(q, 1) == [(last.op_id, True, None)]
    torch.cuda.synchronize()
    for l in range(L):
        assert torch.equal(tensors[l][:, G1], want[l][:, P[:4]]), l   # what was there before the put
        assert torch.equal(tensors[l][:, G2], want[l][:, P[4:8]]), l
        assert torch.equal(tensors[l][:, G3], want[l][:, P[4:8]]), l  # what the put wrote
        assert torch.equal(tensors[l][:, G4], want[l][:, P[:4]]), l   # the get waited for its put
    h.shutdown()
    assert h.process.exitcode == 0
