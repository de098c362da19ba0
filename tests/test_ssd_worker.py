"""The host-pool <-> SSD worker in its own process: H2DISK and DISK2H ops through
the pipe and the shared op pool, file images and read-back checked against the
oracle, failed ops reported.  No GPU involved."""
import queue as pyqueue
import time

import numpy as np
import pytest
import torch
import torch.multiprocessing as mp

from flexkv_amd.layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec,
                               MultiGroupBlockLayout, TransferStrides)
from flexkv_amd.transfer.op_pool import SharedOpPool
from flexkv_amd.transfer.ops import TransferOp, TransferType
from flexkv_amd.transfer.worker import CPUSSDDiskTransferWorker

I64 = np.int64
LAYERS, N_CPU, N_SSD, T, H, D = 3, 16, 24, 4, 2, 32
DT = torch.int16


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


def _files(tmp_path, ndev, nfiles, size):
    paths = {}
    for d in range(ndev):
        (tmp_path / f"dev{d}").mkdir(exist_ok=True)
        paths[d] = []
        for f in range(nfiles):
            p = tmp_path / f"dev{d}" / f"ssd_cache_{d}_{f}.bin"
            with open(p, "wb") as fh:
                fh.truncate(size)
            paths[d].append(str(p))
    return paths


def _images(paths):
    return [np.fromfile(p, dtype=np.uint8) for d in sorted(paths) for p in paths[d]]


def _op(kind, src, dst, pool=None):
    op = TransferOp(0, kind, np.asarray(src, dtype=I64), np.asarray(dst, dtype=I64))
    if pool is not None:
        op.src_slot_id = pool.allocate_slot(op.src_block_ids, 1)
        op.dst_slot_id = pool.allocate_slot(op.dst_block_ids, 2)
        assert op.src_slot_id >= 0 and op.dst_slot_id >= 0
    return op


@pytest.mark.parametrize("kind", [KVCacheLayoutType.LAYERFIRST, KVCacheLayoutType.BLOCKFIRST],
                         ids=["layerfirst", "blockfirst"])
@pytest.mark.parametrize("entries", [0, 64], ids=["threads", "iouring"])
def test_ssd_worker_put_then_get(tmp_path, monkeypatch, engine, kind, entries):
    from oracle import fkv_oracle as O
    monkeypatch.setenv("FLEXKV_IOURING_ENTRIES", str(entries))
    start, q, pool = engine
    ndev, nfiles = 2, 2
    cl = KVCacheLayout(kind, LAYERS, N_CPU, T, H, D, kv_dim=2, num_kv_heads=H)
    sl = KVCacheLayout(kind, LAYERS, N_SSD, T, H, D, kv_dim=2, num_kv_heads=H)
    fl = sl.div_block(ndev * nfiles, padding=True)
    paths = _files(tmp_path, ndev, nfiles, fl.get_total_elements() * 2)
    g = torch.Generator().manual_seed(11)
    host = torch.randint(-30000, 30000, tuple(cl.kv_shape), dtype=DT, generator=g).share_memory_()
    h = start(CPUSSDDiskTransferWorker, host, paths, cl, sl, DT, N_SSD // (ndev * nfiles))
    c, s = TransferStrides.from_layout(cl, 2), TransferStrides.from_layout(fl, 2)
    rng = np.random.default_rng(5)
    cpu_src = rng.permutation(N_CPU)[:9]
    ssd_ids = rng.permutation(N_SSD)[:9]
    cpu_back = np.setdiff1d(np.arange(N_CPU), cpu_src)[:7]
    ref_host = host.numpy().view(np.uint8).reshape(-1).copy()
    ref_files = [np.zeros(fl.get_total_elements() * 2, dtype=np.uint8) for _ in range(ndev * nfiles)]

    put = _op(TransferType.H2DISK, cpu_src, ssd_ids, pool)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    O.ssd_transfer(ref_files, ndev, nfiles, 0, LAYERS, ref_host, ssd_ids, cpu_src, c.layer, c.kv,
                   s.layer, s.kv, c.chunk, c.block, False, 1, 2)
    for got, want in zip(_images(paths), ref_files):
        assert np.array_equal(got, want)

    get = _op(TransferType.DISK2H, ssd_ids[:7], cpu_back)
    h.submit_transfer(get)
    assert _collect(q, 1) == [(get.op_id, True, None)]
    O.ssd_transfer(ref_files, ndev, nfiles, 0, LAYERS, ref_host, ssd_ids[:7], cpu_back, c.layer,
                   c.kv, s.layer, s.kv, c.chunk, c.block, True, 1, 2)
    assert np.array_equal(host.numpy().view(np.uint8).reshape(-1), ref_host)

    # a transfer type this worker does not run fails the op and the worker keeps serving
    wrong = _op(TransferType.H2D, cpu_src[:2], ssd_ids[:2])
    h.submit_transfer(wrong)
    assert _collect(q, 1) == [(wrong.op_id, False, None)]
    again = _op(TransferType.DISK2H, ssd_ids[:2], cpu_back[:2])
    h.submit_transfer(again)
    assert _collect(q, 1) == [(again.op_id, True, None)]


def test_ssd_worker_multi_group_blocks(tmp_path, engine):
    """Byte-flat multi-group blocks move whole: block b of the pool lands at its
    striped place in the files and comes back into another block."""
    start, q, _ = engine
    groups = [LayerGroupSpec(2, 2, 32, [0, 2]), LayerGroupSpec(1, 1, 48, [1], itemsize=1)]
    cl = MultiGroupBlockLayout(N_CPU, T, groups, kv_dim=2)
    sl = MultiGroupBlockLayout(N_SSD, T, groups, kv_dim=2)
    B = cl.get_block_stride()
    ndev, nfiles = 1, 3
    per_file = N_SSD // nfiles
    paths = _files(tmp_path, ndev, nfiles, per_file * B)
    g = torch.Generator().manual_seed(2)
    host = torch.randint(0, 256, (N_CPU * B,), dtype=torch.uint8, generator=g).share_memory_()
    before = host.clone()
    h = start(CPUSSDDiskTransferWorker, host, paths, cl, sl, torch.uint8, per_file,
              layer_groups=groups)
    cpu_src, ssd_ids, cpu_back = [3, 0, 9, 4], [20, 1, 7, 12], [15, 14, 13, 12]
    put = _op(TransferType.H2DISK, cpu_src, ssd_ids)
    h.submit_transfer(put)
    assert _collect(q, 1) == [(put.op_id, True, None)]
    imgs = _images(paths)
    for cb, sb in zip(cpu_src, ssd_ids):
        f, inf = sb % nfiles, sb // nfiles
        assert np.array_equal(imgs[f][inf * B:(inf + 1) * B], before[cb * B:(cb + 1) * B].numpy())
    get = _op(TransferType.DISK2H, ssd_ids, cpu_back)
    h.submit_transfer(get)
    assert _collect(q, 1) == [(get.op_id, True, None)]
    for cb, back in zip(cpu_src, cpu_back):
        assert torch.equal(host[back * B:(back + 1) * B], before[cb * B:(cb + 1) * B])


def test_ssd_worker_reports_missing_files(tmp_path, engine, capfd):
    start, q, _ = engine
    cl = KVCacheLayout(KVCacheLayoutType.LAYERFIRST, LAYERS, N_CPU, T, H, D, kv_dim=2,
                       num_kv_heads=H)
    host = torch.zeros(tuple(cl.kv_shape), dtype=DT).share_memory_()
    with pytest.raises(RuntimeError, match="exited with code 1 before it became ready"):
        start(CPUSSDDiskTransferWorker, host, {0: [str(tmp_path / "nope.bin")]}, cl, cl, DT, N_CPU)
    err = capfd.readouterr().err
    assert "Failed to open file" in err and "SSD Worker init failed" in err
