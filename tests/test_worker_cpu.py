"""The worker-process harness without a device: op records, the shared op pool,
trace lines, the eventfd hand-over and the worker loop's reporting contract."""
import logging
import os
import queue as pyqueue
import re
import threading
import time

import numpy as np
import pytest
import torch
import torch.multiprocessing as mp

from flexkv_amd.transfer import trace
from flexkv_amd.transfer.eventfd_channel import (drain_eventfd, make_eventfd,
                                                 receive_layer_eventfds, send_layer_eventfds)
from flexkv_amd.transfer.op_pool import SharedOpPool
from flexkv_amd.transfer.ops import (LayerwiseTransferOp, TransferOp, TransferType,
                                     WorkerLayerwiseTransferOp, WorkerTransferOp)

I64 = np.int64


# ---- op records ------------------------------------------------------------------

def test_transfer_op_ids_and_checks():
    a = TransferOp(1, TransferType.D2H, np.arange(4, dtype=I64), np.arange(4, dtype=I64) + 10)
    b = TransferOp(1, TransferType.H2D, np.arange(2, dtype=I64), np.arange(2, dtype=I64))
    assert b.op_id == a.op_id + 1 and a.valid_block_num == 4
    with pytest.raises(ValueError, match="same number of physical blocks"):
        TransferOp(1, TransferType.D2H, np.arange(4, dtype=I64), np.arange(3, dtype=I64))
    with pytest.raises(AssertionError):
        TransferOp(1, TransferType.D2H, np.arange(4, dtype=np.int32), np.arange(4, dtype=I64))
    # a virtual op only marks the completion of others and may be empty on one side
    TransferOp(1, TransferType.VIRTUAL, np.arange(0, dtype=I64), np.arange(3, dtype=I64))


def test_worker_op_carries_ids_only_without_slots():
    op = TransferOp(5, TransferType.D2H, np.arange(4, dtype=I64), np.arange(4, dtype=I64))
    w = WorkerTransferOp(op)
    assert w.src_block_ids is op.src_block_ids and w.transfer_graph_id == 5
    op.src_slot_id, op.dst_slot_id = 3, 4
    w = WorkerTransferOp(op)
    assert w.src_block_ids.size == 0 and w.dst_block_ids.size == 0 and w.valid_block_num == 4
    op.dst_slot_id = -1  # one side missing: both lists travel
    assert WorkerTransferOp(op).dst_block_ids.size == 4


def test_layerwise_op_defaults_and_checks():
    e = np.array([], dtype=I64)
    op = LayerwiseTransferOp(2, TransferType.LAYERWISE, e, e,
                             src_block_ids_h2d=np.arange(3, dtype=I64),
                             dst_block_ids_h2d=np.arange(3, dtype=I64), counter_id=2)
    w = WorkerLayerwiseTransferOp(op)
    assert w.counter_id == 2 and w.swa_src_block_ids_h2d.size == 0
    assert w.swa_src_block_ids_h2d.dtype == I64
    with pytest.raises(ValueError):
        LayerwiseTransferOp(2, TransferType.LAYERWISE, e, e,
                            src_block_ids_h2d=np.arange(3, dtype=I64),
                            dst_block_ids_h2d=np.arange(2, dtype=I64))
    with pytest.raises(AssertionError):
        LayerwiseTransferOp(2, TransferType.H2D, e, e)


# ---- shared op pool ----------------------------------------------------------------

def test_op_pool_contract():
    pool = SharedOpPool(3, 8)
    assert pool.get_buffer().is_shared() and pool.get_buffer_size() == (3, 8)
    ids = np.array([5, 1, 9], dtype=I64)
    s0 = pool.allocate_slot(ids)
    assert s0 >= 0 and pool.get_buffer()[s0, :3].tolist() == [5, 1, 9]
    assert pool.allocate_slot(ids) == s0                      # equal lists share a row
    s1 = pool.allocate_slot(ids, device_type_prefix=2)        # ... unless the pool differs
    assert s1 != s0
    assert pool.allocate_slot(np.array([], dtype=I64)) == -1
    assert pool.allocate_slot(np.arange(9, dtype=I64)) == -1  # longer than a row
    s2 = pool.allocate_slot(np.array([5, 1], dtype=I64))      # a prefix is a different list
    assert s2 not in (s0, s1)
    assert pool.allocate_slot(np.array([7], dtype=I64)) == -1  # full
    assert pool.status() == {"used_slots": 3, "free_slots": 0, "capacity": 3}
    pool.free_slot(s0)
    assert pool.status()["used_slots"] == 3                   # still referenced once
    pool.free_slot(s0)
    assert pool.status()["used_slots"] == 2
    with pytest.raises(RuntimeError, match="double free"):
        pool.free_slot(s0)
    s3 = pool.allocate_slot(np.array([7], dtype=I64))
    assert s3 == s0 and pool.get_buffer()[s3, 0] == 7


def test_op_pool_concurrent_allocation_is_consistent():
    pool = SharedOpPool(64, 16)
    lists = [np.arange(i % 7 + 1, dtype=I64) * (i % 5 + 1) for i in range(200)]
    got = [None] * len(lists)

    def work(lo, hi):
        for i in range(lo, hi):
            got[i] = pool.allocate_slot(lists[i])
    ts = [threading.Thread(target=work, args=(k * 50, k * 50 + 50)) for k in range(4)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    for ids, slot in zip(lists, got):
        assert slot >= 0 and pool.get_buffer()[slot, :ids.size].tolist() == ids.tolist()
    by_content = {}
    for ids, slot in zip(lists, got):
        assert by_content.setdefault(ids.tobytes(), slot) == slot
    for slot in got:
        pool.free_slot(slot)
    assert pool.status()["used_slots"] == 0


# ---- trace lines -----------------------------------------------------------------------

XFER_RE = re.compile(
    r"^\[XFER\] op=\d+ type=\w+ nb=\d+ bytes=\d+ h2d=[01] kv_dim=\d+ ipc=[\d.]+ms wait=[\d.]+ms "
    r"xfer=[\d.]+ms e2e=[\d.]+ms bw=\d+MB/s worker=\d+ graph=-?\d+ backlog=\d+$")
SUMMARY_RE = re.compile(
    r"^\[XFER-SUMMARY\] window=\d+s ops=\d+ inflight_max=\d+ wait_p50=[\d.]+ms wait_p99=[\d.]+ms "
    r"xfer_p50=[\d.]+ms xfer_p99=[\d.]+ms type: .*$")


def test_trace_metrics_and_lines():
    lines = []
    t = trace.TransferTrace(True, emit=lines.append)
    op = WorkerTransferOp(TransferOp(9, TransferType.H2D, np.arange(6, dtype=I64),
                                     np.arange(6, dtype=I64)))
    ms = 1_000_000
    m = trace.worker_metrics(op, 10 * ms, 12 * ms, 15 * ms, 19 * ms, worker_id=3,
                             bytes_per_block=1000, kv_dim=2, is_h2d=True)
    assert m == {"type": "H2D", "nb": 6, "graph_id": 9, "worker_id": 3, "is_h2d": True,
                 "kv_dim": 2, "bytes": 6000, "ipc_ms": 2.0, "wait_ms": 3.0, "xfer_ms": 4.0}
    t.op_submitted(op.transfer_op_id, time.perf_counter_ns())
    t.op_submitted(12345, time.perf_counter_ns())
    assert t.inflight() == 2
    t.op_finished(op.transfer_op_id, m)
    assert len(lines) == 1 and XFER_RE.match(lines[0]), lines
    # 6000 bytes in 4 ms = 1.5 MB/s -> "%.0f" -> 2
    assert " bw=2MB/s " in lines[0] and " backlog=1" in lines[0] and " nb=6 " in lines[0]
    line = t.flush_summary()
    assert SUMMARY_RE.match(line) and "ops=1" in line and "inflight_max=2" in line
    assert "xfer_p50=4.000ms" in line and line.endswith("type: H2D=1")
    # a layerwise op has no valid_block_num: the h2d id list counts
    e = np.array([], dtype=I64)
    lw = WorkerLayerwiseTransferOp(LayerwiseTransferOp(
        4, TransferType.LAYERWISE, e, e, src_block_ids_h2d=np.arange(5, dtype=I64),
        dst_block_ids_h2d=np.arange(5, dtype=I64)))
    lw.valid_block_num = 0
    assert trace.worker_metrics(lw, 0, 0, 0, 0, 1, 0, 1, True)["nb"] == 5
    # clocks that run backwards are clamped
    assert trace.worker_metrics(op, 5, 3, 2, 1, 0, 0, 1, False)["ipc_ms"] == 0.0


def test_trace_off_is_silent():
    lines = []
    t = trace.TransferTrace(False, emit=lines.append)
    t.op_submitted(1, 0)
    t.op_finished(1, {"x": 1})
    assert lines == [] and t.inflight() == 0 and t.flush_summary() is None
    trace.configure(False)
    assert trace.build_worker_metrics(None, 0, 0, 0, 0, 0, 0, 1, True) is None


def test_percentile_is_nearest_rank():
    vals = [5.0, 1.0, 3.0, 2.0, 4.0]
    assert trace.percentile(vals) == 3.0 and trace.percentile(vals, 99) == 5.0
    assert trace.percentile(vals, 0) == 1.0 and trace.percentile([]) == 0.0
    assert trace.percentile([1.0, 2.0], 50) == 1.0  # round(0.5) is 0: the lower one


# ---- eventfds over the unix socket ---------------------------------------------------

def test_eventfd_table_arrives_in_counter_rank_layer_order(tmp_path):
    path = str(tmp_path / "lw.sock")
    tp, layers, counters = 2, 3, 2
    sent = {r: [[make_eventfd(nonblocking=True) for _ in range(layers)] for _ in range(counters)]
            for r in range(tp)}
    out = {}
    server = threading.Thread(target=lambda: out.setdefault(
        "t", receive_layer_eventfds(path, tp, layers, deadline_s=20)))
    server.start()
    for r in (1, 0):  # ranks may connect in any order
        send_layer_eventfds(path, r, tp, sent[r], retry_interval_s=0.05)
    server.join(30)
    table = out["t"].reshape(counters, tp, layers)
    assert table.dtype == torch.int32 and not os.path.exists(path)
    # the received descriptors are new numbers for the same kernel objects
    for c in range(counters):
        for r in range(tp):
            for l in range(layers):
                os.write(int(table[c, r, l]), (1).to_bytes(8, "little"))
                assert drain_eventfd(sent[r][c][l]) == 1
                assert all(drain_eventfd(fd) == 0 for rr in sent for cs in sent[rr] for fd in cs)
    for fd in table.reshape(-1).tolist() + [fd for r in sent for cs in sent[r] for fd in cs]:
        os.close(fd)


def test_eventfd_missing_rank_and_no_client(tmp_path):
    path = str(tmp_path / "lw2.sock")
    fds = [[make_eventfd() for _ in range(2)]]
    out = {}
    server = threading.Thread(target=lambda: out.setdefault(
        "t", receive_layer_eventfds(path, 2, 2, deadline_s=1.0, accept_timeout_s=0.2)))
    server.start()
    send_layer_eventfds(path, 1, 2, fds, retry_interval_s=0.05)
    server.join(30)
    table = out["t"].reshape(1, 2, 2)
    assert table[0, 0].tolist() == [-1, -1] and (table[0, 1] >= 0).all()
    assert receive_layer_eventfds(str(tmp_path / "lw3.sock"), 1, 2, deadline_s=0.3,
                                  accept_timeout_s=0.1).numel() == 0
    with pytest.raises(RuntimeError, match="Failed to send eventfds"):
        send_layer_eventfds(str(tmp_path / "nobody.sock"), 0, 1, fds, connect_retries=2,
                            retry_interval_s=0.01, send_retries=1)


# ---- the worker loop in a real process ---------------------------------------------------

def _collect(q, n, timeout=60):
    got = []
    end = time.time() + timeout
    while len(got) < n:
        try:
            got.append(q.get(timeout=max(0.1, end - time.time())))
        except pyqueue.Empty:
            break
    return got


@pytest.fixture
def harness():
    from worker_fakes import RecordingWorker
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    pool = SharedOpPool(8, 16)
    board = torch.zeros(32, dtype=torch.int64).share_memory_()
    handles = []

    def start(**kw):
        h = RecordingWorker.create_worker(ctx, q, pool.get_buffer(), board, **kw)
        handles.append(h)
        return h
    yield start, q, pool, board
    for h in handles:
        if h.process.is_alive():
            h.shutdown()


def test_worker_reports_every_op_in_order(harness):
    start, q, pool, board = harness
    h = start()
    h.wait_ready(120)
    ops = []
    for i in range(6):
        src = np.arange(3, dtype=I64) + i
        dst = np.arange(3, dtype=I64) + 3 * i
        op = TransferOp(i, TransferType.D2H, src, dst)
        if i % 2:  # every other op sends its ids through the shared pool
            op.src_slot_id = pool.allocate_slot(src, 1)
            op.dst_slot_id = pool.allocate_slot(dst, 2)
        ops.append(op)
    bad = TransferOp(0, TransferType.D2H, np.array([-1], dtype=I64), np.array([0], dtype=I64))
    refused = TransferOp(77, TransferType.H2D, np.array([1], dtype=I64), np.array([30], dtype=I64))
    partial = TransferOp(88, TransferType.H2D, np.arange(3, dtype=I64),
                         np.arange(3, dtype=I64) + 20)
    everything = ops + [bad, refused, partial]
    for op in everything:
        h.submit_transfer(op)
    got = _collect(q, len(everything))
    assert len(got) == len(everything)
    ids = [g[0].transfer_op_id if not isinstance(g[0], int) else g[0] for g in got]
    assert ids == [op.op_id for op in everything]          # arrival order, nothing dropped
    for g in got[:6]:
        assert g[1] is True and g[2] is None                # trace is off: no metrics
    assert got[6] == (bad.op_id, False, None)               # raised inside the worker
    assert got[7] == (refused.op_id, False, None)           # launch_transfer said no
    result, ok, _ = got[8]
    assert ok is True and result.block_results == (True, False, True)
    expect = torch.zeros(32, dtype=torch.int64)
    for op in ops + [refused, partial]:
        for s, d in zip(op.src_block_ids.tolist(), op.dst_block_ids.tolist()):
            expect[d] += s + 1
    assert torch.equal(board, expect)
    assert h.control("board_sum") == int(expect.sum())
    assert h.control("ping", {"a": 1})["echo"] == {"a": 1}
    with pytest.raises(RuntimeError, match="does not support control nonsense"):
        h.control("nonsense")
    h.shutdown()
    assert h.process.exitcode == 0


def test_worker_constructor_failure_is_visible(harness):
    start, q, pool, board = harness
    h = start(fail_init=True)
    with pytest.raises(RuntimeError, match="before it became ready"):
        h.wait_ready(120)
    assert h.process.exitcode not in (0, None)


def test_worker_ends_on_sigterm_and_on_closed_pipe(harness):
    start, q, pool, board = harness
    a, b = start(), start()
    a.wait_ready(120)
    b.wait_ready(120)
    a.process.terminate()          # SIGTERM: SystemExit inside the loop, clean exit code
    a.process.join(30)
    assert a.process.exitcode == 0
    b.transfer_conn.close()        # the engine went away
    b.process.join(30)
    assert b.process.exitcode == 0


def test_worker_metrics_when_trace_is_on(harness, monkeypatch):
    import flexkv_amd.transfer.env as env
    monkeypatch.setenv("FLEXKV_TRANSFER_TRACE", "1")   # inherited by the spawned worker
    monkeypatch.setattr(env, "_ENV", None)
    trace.configure(True)
    lines = []
    monkeypatch.setattr(trace.instance(), "_emit", lines.append)
    try:
        start, q, pool, board = harness
        h = start(delay_s=0.02)
        h.wait_ready(120)
        op = TransferOp(3, TransferType.H2D, np.arange(4, dtype=I64), np.arange(4, dtype=I64))
        h.submit_transfer(op)
        (op_id, ok, m), = _collect(q, 1)
        assert ok and op_id == op.op_id
        assert m["type"] == "H2D" and m["nb"] == 4 and m["bytes"] == 4 * 4096 and m["is_h2d"]
        assert m["xfer_ms"] >= 20.0 and m["ipc_ms"] >= 0.0 and m["worker_id"] == h.worker_id
        trace.record_xfer(op_id, m)
        assert XFER_RE.match(lines[0]) and " backlog=0" in lines[0]
        # the process-wide window may have been open for more than its ten seconds
        assert all(SUMMARY_RE.match(x) for x in lines[1:]) and len(lines) <= 2
    finally:
        trace.configure(False)
        monkeypatch.setattr(env, "_ENV", None)


def test_side_lane_runs_in_order_and_holds_back_ops_that_share_blocks():
    """The second thread of a GPU worker that overlaps gets with puts: ops handed
    to it run in order, and the worker's own thread can wait until no unfinished
    op of the lane touches given host or engine blocks."""
    import threading
    from flexkv_amd.transfer.worker import _SideLane
    gate, ran = threading.Event(), []

    def run_op(op):
        if op == "slow":
            gate.wait(10)
        ran.append(op)
    lane = _SideLane("t", run_op, None)
    lane.submit("slow", np.array([1, 2, 3]), np.array([10, 11]))
    lane.submit("next", np.array([7]), np.array([12]))
    t0 = time.time()
    lane.wait_until_clear_of(np.array([4, 5]), np.array([13]))       # shares nothing
    lane.wait_until_clear_of(np.array([], dtype=np.int64), None)     # touches nothing
    assert time.time() - t0 < 0.3
    cleared = []
    for ids in ((np.array([3]), None), (None, np.array([12, 99]))):  # a host block; an engine block
        done = threading.Event()
        threading.Thread(target=lambda i=ids, d=done: (lane.wait_until_clear_of(*i), d.set()),
                         daemon=True).start()
        cleared.append(done)
    time.sleep(0.3)
    assert not cleared[0].is_set() and not cleared[1].is_set()
    gate.set()
    assert cleared[0].wait(5) and cleared[1].wait(5)
    lane.drain()
    assert ran == ["slow", "next"]
    lane.close()


class _PoolAdopter:
    """TransferWorkerBase's host-pool logic without a process, a pipe or a device."""

    def __new__(cls):
        from worker_fakes import RecordingWorker
        w = RecordingWorker.__new__(RecordingWorker)
        w.worker_id = 0
        return w


def test_host_pool_adoption_register_is_opt_in(monkeypatch):
    """A pageable pool is registered only with FKV_HOST_REGISTER=1; without it the
    pool stays pageable when that is allowed and is refused otherwise.  The
    registration itself is replaced by a recorder: no device is involved."""
    from flexkv_amd import host_buffer
    calls = []
    monkeypatch.setattr(host_buffer, "cudaHostRegister", lambda t: calls.append(("reg", t.data_ptr())))
    monkeypatch.setattr(host_buffer, "cudaHostUnregister",
                        lambda t: calls.append(("unreg", t.data_ptr())))
    pool = torch.zeros(1024, dtype=torch.uint8)

    monkeypatch.delenv("FKV_HOST_REGISTER", raising=False)
    w = _PoolAdopter()
    with pytest.raises(RuntimeError, match="neither pinned nor worker-owned"):
        w._adopt_host_pool(pool, "pool", allow_pageable=False)
    assert w._adopt_host_pool(pool, "pool", allow_pageable=True) is pool
    assert w._pageable_host and w._engine(False) is True and calls == []

    monkeypatch.setenv("FKV_HOST_REGISTER", "1")
    w = _PoolAdopter()
    assert w._adopt_host_pool(pool, "pool", allow_pageable=False) is pool
    assert not w._pageable_host and w._engine(False) is False
    assert calls == [("reg", pool.data_ptr())]
    w.shutdown()
    assert calls == [("reg", pool.data_ptr()), ("unreg", pool.data_ptr())]
    w.shutdown()  # idempotent
    assert len(calls) == 2


def test_host_pool_adoption_falls_back_when_registration_is_refused(monkeypatch):
    from flexkv_amd import host_buffer

    def refuse(t):
        raise RuntimeError("registration refused")
    monkeypatch.setattr(host_buffer, "cudaHostRegister", refuse)
    monkeypatch.setenv("FKV_HOST_REGISTER", "1")
    pool = torch.zeros(1024, dtype=torch.uint8)
    w = _PoolAdopter()
    with pytest.raises(RuntimeError, match="registration refused"):
        w._adopt_host_pool(pool, "pool", allow_pageable=False)
    assert w._host_registered == []
    assert w._adopt_host_pool(pool, "pool", allow_pageable=True) is pool
    assert w._pageable_host and w._host_registered == []


# tests/test_transfer_worker_device_selection.py: the device is made current before the host
# pool is registered with the runtime (registration maps the pool for the current device).
class _RegistrationReached(Exception):
    pass


def _stop_at_first_host_registration(monkeypatch, events):
    from flexkv_amd import host_buffer
    from flexkv_amd.transfer import worker
    monkeypatch.setattr(worker.torch.cuda, "set_device",
                        lambda device: events.append(("set_device", device)))

    def register(_tensor):
        events.append(("register", None))
        raise _RegistrationReached
    monkeypatch.setattr(host_buffer, "cudaHostRegister", register)
    monkeypatch.setenv("FKV_HOST_REGISTER", "1")


def test_gpu_cpu_worker_selects_device_before_host_registration(monkeypatch):
    from flexkv_amd.transfer.worker import GPUCPUTransferWorker
    events = []
    _stop_at_first_host_registration(monkeypatch, events)
    with pytest.raises(_RegistrationReached):
        GPUCPUTransferWorker(
            worker_id=0, transfer_conn=None, finished_ops_queue=None,
            op_buffer_tensor=torch.empty(0), gpu_blocks=[], cpu_blocks=torch.zeros(64, dtype=torch.uint8),
            gpu_kv_layout=None, cpu_kv_layout=None, dtype=torch.bfloat16, gpu_device_id=3)
    assert events == [("set_device", 3), ("register", None)]


def test_tp_worker_selects_device_of_its_tensors_before_host_registration(monkeypatch):
    from flexkv_amd.transfer.worker import tpGPUCPUTransferWorker
    events = []
    _stop_at_first_host_registration(monkeypatch, events)
    handle = type("Handle", (), {"device": torch.device("cuda:4")})()
    with pytest.raises(_RegistrationReached):
        tpGPUCPUTransferWorker(
            worker_id=0, transfer_conn=None, finished_ops_queue=None,
            op_buffer_tensor=torch.empty(0), gpu_blocks=[[handle], [handle]],
            cpu_blocks=torch.zeros(64, dtype=torch.uint8), gpu_kv_layouts=[], cpu_kv_layout=None,
            dtype=torch.bfloat16, tp_group_size=2)
    assert events and events[-1] == ("register", None)
    selected = [e[1] for e in events[:-1]]
    assert selected and all(e[0] == "set_device" for e in events[:-1])
    last = selected[-1]                      # the device that is current when the pool is registered
    assert (last.index if isinstance(last, torch.device) else last) == 4
