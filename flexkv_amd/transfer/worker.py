"""Transfer worker processes for the GPU<->CPU path.

One worker process owns one kind of transfer.  The engine submits ops through a
pipe (``WorkerHandle.submit_transfer``), the worker runs them one at a time in
arrival order (a GPU worker with ``overlap_directions`` runs gets next to puts)
and reports every op on a shared queue:

    (op_id, True,  metrics-or-None)      the op ran
    (op_id, False, None)                 the op raised; logged, never dropped

Contract and names follow ``flexkv/transfer/worker.py`` of the reference
(``TransferWorkerBase`` :120-633, ``WorkerHandle`` :635-707,
``GPUCPUTransferWorker`` :709-1097, ``tpGPUCPUTransferWorker`` :1098-1520) and
``flexkv/transfer/layerwise.py`` (``LayerwiseTransferWorker`` :69-1059).  What a
worker of this library does *not* do: compression, remote tiers.

Host pools.  A worker either receives the pool as a shared-memory tensor and
registers it with the runtime (the reference's way), or receives a
``PinnedPoolHandle`` and allocates the pool itself, pinned and device-mapped.
Where the runtime refuses to register existing memory, a worker started with
``allow_pageable_host=True`` (or FKV_WORKER_ALLOW_PAGEABLE_HOST=1) keeps the pool
pageable and moves every transfer with the copy engine, which accepts such
memory; otherwise the refusal is an error, as in the reference.

The shared op buffer is not pinned: the transfer library reads block ids on the
host while it builds a call, never from the device.
"""
from __future__ import annotations

import logging
import os
import signal
import threading
import time
from abc import ABC, abstractmethod
from dataclasses import dataclass
from multiprocessing.connection import Connection
from typing import Any, Dict, List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from .. import _lib
from ..layout import (KVCacheLayout, KVCacheLayoutType, LayerGroupSpec, MultiGroupBlockLayout,
                      TransferStrides, gpu_block_type_from_tensor_count, gpu_strides_from_tensor,
                      multi_group_tables)
from . import trace
from .env import global_env
from .memory_handle import TensorSharedHandle, discard_tensor_handles, import_tensor_handles
from .ops import (LayerwiseTransferOp, TransferOp, TransferType, WorkerLayerwiseTransferOp,
                  WorkerTransferOp, WorkerTransferResult)

logger = logging.getLogger("flexkv")


@dataclass(frozen=True)
class PinnedPoolHandle:
    """A host pool the worker allocates for itself (pinned, device-mapped).  Takes
    the place of a host tensor in a worker's constructor arguments."""
    shape: Tuple[int, ...]
    dtype: torch.dtype

    def numel(self) -> int:
        n = 1
        for e in self.shape:
            n *= int(e)
        return n


def materialize_worker_tensor(pool: Union[torch.Tensor, PinnedPoolHandle]) -> torch.Tensor:
    if isinstance(pool, PinnedPoolHandle):
        from ..host_buffer import alloc_mapped_host_tensor
        return alloc_mapped_host_tensor(pool.numel(), pool.dtype).view(pool.shape)
    return pool


def _allow_pageable(flag: Optional[bool]) -> bool:
    if flag is not None:
        return bool(flag)
    return bool(int(os.getenv("FKV_WORKER_ALLOW_PAGEABLE_HOST", "0")))


def _register_foreign_pools() -> bool:
    """Whether a host pool that is not pinned is handed to hipHostRegister.  Opt-in
    (``FKV_HOST_REGISTER=1``): some platforms refuse registration of memory that
    already exists, and the error such a refusal leaves behind can surface at a
    later device call.  A pool the worker allocates itself (``PinnedPoolHandle``)
    or a tensor that is already pinned needs none."""
    return bool(int(os.getenv("FKV_HOST_REGISTER", "0")))


class _SideLane:
    """A second thread of a worker that runs the ops handed to it in order, next to
    the ops the worker runs itself.  It remembers the block ids of its unfinished ops
    so that the worker can hold back an op of its own that touches the same blocks."""

    def __init__(self, name: str, run_op, device: Optional[int]) -> None:
        import queue
        self.name = name
        self._run_op = run_op
        self._device = device
        self._q: "queue.Queue[Any]" = queue.Queue()
        self._cond = threading.Condition()
        self._inflight: Dict[int, Tuple[np.ndarray, np.ndarray]] = {}
        self._seq = 0
        self._thread = threading.Thread(target=self._loop, name=f"fkv-lane-{name}", daemon=True)
        self._thread.start()

    def submit(self, op: Any, cpu_ids: np.ndarray, gpu_ids: np.ndarray) -> None:
        with self._cond:
            self._seq += 1
            key = self._seq
            self._inflight[key] = (np.array(cpu_ids, copy=True), np.array(gpu_ids, copy=True))
        self._q.put((key, op))

    def wait_until_clear_of(self, cpu_ids: Optional[np.ndarray],
                            gpu_ids: Optional[np.ndarray]) -> None:
        """Returns once no unfinished op of the lane shares a host block with
        `cpu_ids` or an engine block with `gpu_ids` (None: that side is not touched)."""
        def clash() -> bool:
            for c, g in self._inflight.values():
                if cpu_ids is not None and len(cpu_ids) and np.isin(cpu_ids, c).any():
                    return True
                if gpu_ids is not None and len(gpu_ids) and np.isin(gpu_ids, g).any():
                    return True
            return False
        with self._cond:
            while clash():
                self._cond.wait(0.5)

    def drain(self) -> None:
        with self._cond:
            while self._inflight:
                self._cond.wait(0.5)

    def close(self) -> None:
        self._q.put(None)
        self._thread.join(timeout=60)

    def _loop(self) -> None:
        if self._device is not None:
            torch.cuda.set_device(self._device)
        while True:
            item = self._q.get()
            if item is None:
                return
            key, op = item
            try:
                self._run_op(op)   # reports the op itself, never raises
            finally:
                with self._cond:
                    self._inflight.pop(key, None)
                    self._cond.notify_all()


class TransferWorkerBase(ABC):
    _worker_id_counter = 0
    _worker_id_lock = threading.Lock()

    def __new__(cls, *args: Any, **kwargs: Any):
        # Fields shutdown() reads exist before __init__ runs, so the process wrapper
        # can always clean up after a constructor that failed half-way.
        obj = super().__new__(cls)
        obj._host_registered = []
        obj._shutdown_done = False
        obj._pageable_host = False
        obj._lanes = {}
        return obj

    def __init__(self, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                 op_buffer_tensor: torch.Tensor) -> None:
        self.worker_id = worker_id
        self.transfer_conn = transfer_conn
        self.finished_ops_queue = finished_ops_queue
        self.op_buffer_tensor = op_buffer_tensor
        self._host_registered: List[Tuple[torch.Tensor, str]] = []
        self._shutdown_done = False
        self._pageable_host = False
        self._lanes: Dict[str, _SideLane] = {}
        trace.configure(global_env().enable_transfer_trace)

    # ---- host memory --------------------------------------------------------------
    def _adopt_host_pool(self, pool: Union[torch.Tensor, PinnedPoolHandle], label: str,
                         allow_pageable: Optional[bool] = None) -> torch.Tensor:
        """The pool as a tensor the device can reach.  Worker-owned pools are born
        pinned; foreign memory is registered (and tracked for shutdown)."""
        if isinstance(pool, PinnedPoolHandle):
            return materialize_worker_tensor(pool)
        if pool.is_pinned():
            return pool
        if not _register_foreign_pools():
            if not _allow_pageable(allow_pageable):
                raise RuntimeError(
                    f"{label} is neither pinned nor worker-owned: pass a PinnedPoolHandle or a "
                    "pinned tensor, set FKV_HOST_REGISTER=1 to have the worker register it, or "
                    "allow_pageable_host=True to move it with the copy engine")
            logger.info("[worker %s] %s stays pageable: every transfer of this worker goes "
                        "through the copy engine", self.worker_id, label)
            self._pageable_host = True
            return pool
        from ..host_buffer import cudaHostRegister
        size_gb = pool.numel() * pool.element_size() / (1024 ** 3)
        logger.info("[worker %s] hipHostRegister %s: ptr=0x%x size=%.3f GiB", self.worker_id,
                    label, pool.data_ptr(), size_gb)
        try:
            cudaHostRegister(pool)
            self._host_registered.append((pool, label))
        except RuntimeError as e:
            if not _allow_pageable(allow_pageable):
                raise
            logger.warning("[worker %s] %s stays pageable (%s): every transfer of this worker "
                           "goes through the copy engine", self.worker_id, label, e)
            self._pageable_host = True
        return pool

    def _engine(self, use_ce: Any) -> Any:
        return True if self._pageable_host else use_ce

    def shutdown(self) -> None:
        """Wait (bounded) for device work, then unregister host memory in reverse
        order.  Idempotent, and safe after a constructor that failed half-way."""
        if getattr(self, "_shutdown_done", False):
            return
        self._shutdown_done = True
        for lane in (getattr(self, "_lanes", None) or {}).values():
            lane.close()
        registered = getattr(self, "_host_registered", None) or []
        wid = getattr(self, "worker_id", -1)
        logger.info("[worker %s] shutdown: unregistering %d host region(s)", wid, len(registered))
        self._drain_device_bounded(wid, 30.0)
        from ..host_buffer import cudaHostUnregister
        while registered:
            tensor, label = registered.pop()
            try:
                cudaHostUnregister(tensor)
            except Exception as e:  # noqa: BLE001 - best effort, the process is ending
                logger.warning("[worker %s] unregister of %s failed: %s", wid, label, e)
        self._host_registered = registered
        self._release_engine_tensors()

    def _release_engine_tensors(self) -> None:
        """Drop the engine's tensors this process imported, and tell torch's IPC layer at
        once: the owner of a tensor shared through torch keeps its memory (and warns when it
        exits) until every importer has let go, which an importer that simply ends never
        does.  The transfer groups hold addresses only and are gone or idle by now."""
        for name in ("gpu_blocks", "gpu_blocks_ptrs", "swa_gpu_blocks", "_group_tensors"):
            if hasattr(self, name):
                setattr(self, name, None)
        try:
            import gc
            gc.collect()
            if torch.cuda.is_initialized():
                torch.cuda.ipc_collect()
        except Exception as e:  # noqa: BLE001 - best effort, the process is ending
            logger.warning("[worker %s] releasing imported tensors failed: %s",
                           getattr(self, "worker_id", -1), e)

    @staticmethod
    def _drain_device_bounded(worker_id: Any, timeout_s: float) -> bool:
        """torch.cuda.synchronize() with a wall-clock cap: a wedged GPU must not keep
        the host memory pinned forever.  True when the sync completed."""
        if not (torch.cuda.is_available() and torch.cuda.is_initialized()):
            return True
        finished = threading.Event()
        failure: List[BaseException] = []

        def sync() -> None:
            try:
                torch.cuda.synchronize()
            except BaseException as e:  # noqa: BLE001
                failure.append(e)
            finally:
                finished.set()

        threading.Thread(target=sync, name=f"fkv-worker-{worker_id}-drain", daemon=True).start()
        if not finished.wait(timeout_s):
            logger.warning("[worker %s] device synchronize did not finish in %.0fs; "
                           "unpinning anyway", worker_id, timeout_s)
            return False
        if failure:
            logger.warning("[worker %s] device synchronize before unpin failed: %r", worker_id,
                           failure[0])
        return not failure

    # ---- creation -----------------------------------------------------------------
    @classmethod
    def _get_worker_id(cls) -> int:
        with TransferWorkerBase._worker_id_lock:
            wid = TransferWorkerBase._worker_id_counter
            TransferWorkerBase._worker_id_counter += 1
            return wid

    @classmethod
    def create_worker(cls, mp_ctx: Any, finished_ops_queue, op_buffer_tensor: torch.Tensor,
                      *args: Any, **kwargs: Any) -> "WorkerHandle":
        parent_conn, child_conn = mp_ctx.Pipe()
        ready_event = mp_ctx.Event()
        worker_id = cls._get_worker_id()
        process = mp_ctx.Process(
            target=cls._worker_process,
            args=(worker_id, child_conn, finished_ops_queue, op_buffer_tensor, ready_event, *args),
            kwargs=kwargs, daemon=True)
        process.start()
        return WorkerHandle(worker_id, parent_conn, process, ready_event)

    @classmethod
    def _worker_process(cls, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                        op_buffer_tensor: torch.Tensor, ready_event: Any, *args: Any,
                        **kwargs: Any) -> None:
        worker: Optional[TransferWorkerBase] = None

        def on_sigterm(signum: int, frame: Any) -> None:
            logger.warning("[worker %s] received signal %s; exiting", worker_id, signum)
            raise SystemExit(0)  # unwinds through the finally below

        try:
            # Ctrl+C reaches the whole foreground process group; only the parent's
            # sentinel or SIGTERM may end a worker, so that unpinning is never raced.
            signal.signal(signal.SIGINT, signal.SIG_IGN)
            signal.signal(signal.SIGTERM, on_sigterm)
        except Exception as e:  # noqa: BLE001 - e.g. not the main thread
            logger.warning("[worker %s] could not install signal handlers: %s", worker_id, e)
        try:
            worker = cls.__new__(cls)
            worker.__init__(worker_id, transfer_conn, finished_ops_queue, op_buffer_tensor,
                            *args, **kwargs)
            ready_event.set()
            worker.run()
        except Exception as e:
            logger.error("[worker %s] exited with error during init/run: %s", worker_id, e)
            raise
        finally:
            if worker is not None:
                try:
                    worker.shutdown()
                except Exception as e:  # noqa: BLE001
                    logger.error("[worker %s] final shutdown error: %s", worker_id, e)

    # ---- per-op helpers -----------------------------------------------------------
    def get_transfer_block_ids(self, op: WorkerTransferOp) -> Tuple[torch.Tensor, torch.Tensor]:
        """Source and destination ids of an op: rows of the shared op buffer when the
        op names slots, the arrays it carries otherwise (worker.py:393-423)."""
        n = op.valid_block_num

        def side(slot: int, carried: np.ndarray) -> torch.Tensor:
            if slot == -1:
                return torch.from_numpy(np.ascontiguousarray(carried, dtype=np.int64))
            return self.op_buffer_tensor[slot, :n]

        return side(op.src_slot_id, op.src_block_ids), side(op.dst_slot_id, op.dst_block_ids)

    def _log_transfer_performance(self, op, transfer_size: int, start_time: float,
                                  end_time: float) -> None:
        if not logger.isEnabledFor(logging.INFO):
            return
        seconds = max(end_time - start_time, 1e-9)
        layerwise = op.transfer_type == TransferType.LAYERWISE
        logger.info(
            "[FlexKV-IO] operation=transfer act=complete status=success direction=%s blocks=%d "
            "op_id=%d graph_id=%d mode=%s data_size=%.6gGB transfer_time=%.4fs "
            "bandwidth=%.2fGB/s",
            "H2D" if layerwise else op.transfer_type.value,
            len(op.src_block_ids_h2d) if layerwise else op.valid_block_num,
            op.transfer_op_id, op.transfer_graph_id,
            "layerwise" if layerwise else "no-layerwise", transfer_size / (1024 ** 3), seconds,
            transfer_size / seconds / 1e9)

    @abstractmethod
    def launch_transfer(self, transfer_op) -> Union[bool, WorkerTransferResult]:
        ...

    # ---- control messages ---------------------------------------------------------
    def _reply_control(self, msg: Dict[str, Any]) -> None:
        reply: Dict[str, Any] = {"type": "control_ack", "request_id": msg["request_id"]}
        try:
            handler = getattr(self, f"_control_{msg['command']}", None)
            if handler is None:
                raise NotImplementedError(
                    f"{type(self).__name__} does not support control {msg['command']}")
            reply["result"] = handler(msg.get("payload"))
        except Exception as e:  # noqa: BLE001 - reported to the caller
            logger.exception("Worker control %s failed", msg.get("command"))
            reply["error"] = str(e)
        self.transfer_conn.send(reply)

    def _control_ping(self, payload: Any) -> Any:
        return {"worker_id": self.worker_id, "pageable_host": self._pageable_host,
                "echo": payload}

    # ---- the loop -----------------------------------------------------------------
    def _run_one(self, op) -> None:
        ok: Union[bool, WorkerTransferResult] = False
        t_launch = time.perf_counter_ns()
        layerwise = op.transfer_type == TransferType.LAYERWISE
        # a range on the profiler's timeline per op, as the reference annotates (worker.py:556-587)
        pushed = _lib.load().fkv_range_push(
            (f"launch {op.transfer_type.name} op_id: {op.transfer_op_id}, graph_id: "
             f"{op.transfer_graph_id}, num_blocks: "
             f"{len(op.src_block_ids_h2d) if layerwise else op.valid_block_num}").encode())
        try:
            ok = self.launch_transfer(op)
        except Exception as e:  # noqa: BLE001 - a failed op is reported, not fatal
            logger.error(
                "[FlexKV-IO] operation=transfer act=complete status=failed direction=%s "
                "blocks=%d op_id=%d graph_id=%d mode=%s transfer_time=%.4fs error=%r",
                "H2D" if layerwise else op.transfer_type.value,
                len(op.src_block_ids_h2d) if layerwise else op.valid_block_num,
                op.transfer_op_id, op.transfer_graph_id,
                "layerwise" if layerwise else "no-layerwise",
                (time.perf_counter_ns() - t_launch) / 1e9, str(e), exc_info=True)
        finally:
            if pushed:
                _lib.load().fkv_range_pop()
        t_done = time.perf_counter_ns()
        metrics = trace.build_worker_metrics(
            op, getattr(op, "prof_submitted_ns", 0), getattr(op, "_received_ns", t_done), t_launch,
            t_done, self.worker_id, getattr(self, "_bytes_per_block", 0),
            getattr(self, "kv_dim", 2),
            op.transfer_type in (TransferType.H2D, TransferType.LAYERWISE))
        if isinstance(ok, WorkerTransferResult):
            self.finished_ops_queue.put((ok, True, metrics))
        elif ok:
            self.finished_ops_queue.put((op.transfer_op_id, True, metrics))
        else:
            # dropping it would leave the op's graph unfinished for ever
            self.finished_ops_queue.put((op.transfer_op_id, False, None))

    def _dispatch(self, op) -> None:
        """Runs the op on this thread.  A worker with side lanes overrides this."""
        self._run_one(op)

    def run(self) -> None:
        """Receive, drain what else is already queued, run the batch in order.  Ends
        on the ``None`` sentinel or when the pipe closes; cleaning up is the process
        wrapper's job."""
        while True:
            try:
                if not self.transfer_conn.poll(timeout=0.0001):
                    continue
                batch: List[Any] = []
                stop = False
                while True:
                    msg = self.transfer_conn.recv()
                    if msg is None:
                        stop = True
                        break
                    if not isinstance(msg, dict):
                        msg._received_ns = time.perf_counter_ns()
                    batch.append(msg)
                    if not self.transfer_conn.poll(timeout=0):
                        break
                for msg in batch:
                    if isinstance(msg, dict):
                        if msg.get("type") == "control":
                            self._reply_control(msg)
                        continue
                    self._dispatch(msg)
                if stop:
                    for lane in self._lanes.values():
                        lane.drain()
                    return
            except EOFError:
                logger.warning("[worker %s] transfer pipe EOF; exiting run loop", self.worker_id)
                return
            except Exception as e:  # noqa: BLE001 - keep serving
                logger.error("Error in worker run loop: %s", e)


class WorkerHandle:
    """The engine's end of one worker process (worker.py:635-707)."""

    def __init__(self, worker_id: int, transfer_conn: Connection, process, ready_event) -> None:
        self.worker_id = worker_id
        self.transfer_conn = transfer_conn
        self.process = process
        self.ready_event = ready_event

    def wait_ready(self, timeout: float = 180.0) -> None:
        """Block until the worker's constructor has finished; raise if it died."""
        end = time.time() + timeout
        while not self.ready_event.wait(0.05):
            if not self.process.is_alive():
                raise RuntimeError(f"worker {self.worker_id} exited with code "
                                   f"{self.process.exitcode} before it became ready")
            if time.time() > end:
                raise TimeoutError(f"worker {self.worker_id} not ready after {timeout:.0f}s")

    def submit_transfer(self, op: Union[TransferOp, LayerwiseTransferOp]) -> None:
        wop = (WorkerLayerwiseTransferOp(op) if isinstance(op, LayerwiseTransferOp)
               else WorkerTransferOp(op))
        if trace.is_enabled():
            wop.prof_submitted_ns = time.perf_counter_ns()
            trace.record_submit(op.op_id, wop.prof_submitted_ns)
        self.transfer_conn.send(wop)

    def control(self, command: str, payload: Any = None, timeout: float = 120.0) -> Any:
        request_id = f"{self.worker_id}:{time.monotonic_ns()}"
        self.transfer_conn.send({"type": "control", "command": command, "payload": payload,
                                 "request_id": request_id})
        if not self.transfer_conn.poll(timeout):
            raise TimeoutError(f"Worker {self.worker_id} timed out handling {command}")
        reply = self.transfer_conn.recv()
        if reply.get("request_id") != request_id:
            raise RuntimeError(f"Unexpected worker control reply: {reply}")
        if "error" in reply:
            raise RuntimeError(f"Worker {self.worker_id} {command} failed: {reply['error']}")
        return reply.get("result")

    def shutdown(self) -> None:
        """Sentinel, then a bounded join; terminate, then kill, if the worker does not
        leave by itself."""
        try:
            self.transfer_conn.send(None)
        except (BrokenPipeError, OSError, EOFError):
            pass
        self.process.join(timeout=global_env().worker_shutdown_timeout_s)
        if self.process.is_alive():
            logger.warning("[WorkerHandle] worker %s still alive after graceful shutdown; "
                           "terminating", self.worker_id)
            self.process.terminate()
            self.process.join(timeout=30)
            if self.process.is_alive():
                self.process.kill()
                self.process.join()
        try:
            self.transfer_conn.close()
        except Exception:  # noqa: BLE001
            pass
        # tensors this process shared with the worker through torch: the worker has let go
        # of them, reclaim what torch kept on their behalf
        try:
            if torch.cuda.is_initialized():
                torch.cuda.ipc_collect()
        except Exception:  # noqa: BLE001
            pass

    def __del__(self) -> None:
        try:
            if getattr(self, "process", None) is not None and self.process.is_alive():
                self.shutdown()
        except Exception:  # noqa: BLE001
            pass


def _layer_ptrs(tensors: Sequence[torch.Tensor]) -> torch.Tensor:
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64)


def _measured_gpu_strides(tensors: Sequence[torch.Tensor], layout: KVCacheLayout, tpb: int,
                          itemsize: int, kv_dim: int) -> TransferStrides:
    """Strides of an engine's per-layer tensor as it really lies in memory, falling
    back to the layout's closed forms (worker.py:786-801)."""
    probed = None
    if len(tensors) > 1:
        t = tensors[0]
        probed = gpu_strides_from_tensor(tuple(t.shape), tuple(t.stride()), tpb, itemsize, kv_dim)
    s = TransferStrides.from_layout(layout, itemsize)
    if probed is None:
        return s
    return TransferStrides(kv=probed[0], block=probed[1], layer=probed[2], chunk=s.chunk)


def _release_imported(handles, tensors) -> int:
    """Gives back what importing ``handles`` mapped into this process: the tensors
    are dropped by the caller, mappings opened through the runtime's IPC calls are
    closed here.  Returns how many tensors were let go."""
    n = len(tensors)
    for h in handles:
        if isinstance(h, TensorSharedHandle):
            h.release()
    return n


def _direction(transfer_type: TransferType, src: torch.Tensor, dst: torch.Tensor, who: str):
    """(gpu ids, host ids, is_h2d) of a D2H / H2D op."""
    if transfer_type == TransferType.H2D:
        return dst, src, True
    if transfer_type == TransferType.D2H:
        return src, dst, False
    raise ValueError(f"Invalid transfer type: {transfer_type} for {who}")


class GPUCPUTransferWorker(TransferWorkerBase):
    """One GPU, whole-model D2H / H2D ops on a private stream (worker.py:709-1097)."""

    def __init__(self, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                 op_buffer_tensor: torch.Tensor, gpu_blocks: List[Any],
                 cpu_blocks: Union[torch.Tensor, PinnedPoolHandle], gpu_kv_layout: KVCacheLayout,
                 cpu_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout], dtype: torch.dtype,
                 gpu_device_id: int, use_ce_transfer_h2d: Any = False,
                 use_ce_transfer_d2h: Any = False, transfer_num_cta_h2d: int = 4,
                 transfer_num_cta_d2h: int = 4,
                 layer_groups: Optional[List[LayerGroupSpec]] = None,
                 gpu_blocks_per_group: Optional[List[List[Any]]] = None,
                 gpu_layouts_per_group: Optional[List[KVCacheLayout]] = None,
                 allow_pageable_host: Optional[bool] = None,
                 ssd_files: Optional[Dict[int, List[str]]] = None,
                 ssd_kv_layout: Optional[Union[KVCacheLayout, MultiGroupBlockLayout]] = None,
                 num_blocks_per_file: int = 0, overlap_directions: Optional[bool] = None) -> None:
        super().__init__(worker_id, transfer_conn, finished_ops_queue, op_buffer_tensor)
        # the device first: everything below creates state on the current device
        torch.cuda.set_device(gpu_device_id)
        self.gpu_device_id = gpu_device_id
        self.cpu_tensor = self._adopt_host_pool(cpu_blocks, "cpu_kv_pool", allow_pageable_host)
        self._gpu_handles = list(gpu_blocks)
        self._gpu_block_count = len(gpu_blocks)
        self.gpu_blocks = import_tensor_handles(gpu_blocks)
        self.gpu_blocks_ptrs = _layer_ptrs(self.gpu_blocks)
        self.dtype = dtype
        self.kv_dim = gpu_kv_layout.kv_dim
        self.num_kv_heads = gpu_kv_layout.num_kv_heads
        self.num_layers = gpu_kv_layout.num_layer
        self.layer_groups = layer_groups
        self.group_transfer_params: Optional[List[dict]] = None
        if layer_groups is not None and gpu_blocks_per_group is not None \
                and gpu_layouts_per_group is not None:
            self.cpu_is_blockfirst = True
            self._init_multi_group(gpu_blocks_per_group, gpu_layouts_per_group, cpu_kv_layout,
                                   layer_groups)
            ref_tensors, ref_layers = len(self._group_tensors[0]), layer_groups[0].num_layers
        else:
            self.cpu_is_blockfirst = cpu_kv_layout.type == KVCacheLayoutType.BLOCKFIRST
            g = _measured_gpu_strides(self.gpu_blocks, gpu_kv_layout,
                                      gpu_kv_layout.tokens_per_block, dtype.itemsize, self.kv_dim)
            c = TransferStrides.from_layout(cpu_kv_layout, dtype.itemsize)
            self.gpu_kv_stride_in_bytes = g.kv
            self.gpu_block_stride_in_bytes = g.block
            self.gpu_layer_stride_in_bytes = g.layer
            self.chunk_size_in_bytes = g.chunk
            self.cpu_kv_stride_in_bytes = c.kv
            self.cpu_layer_stride_in_bytes = c.layer
            self.cpu_block_stride_in_bytes = c.block
            self._bytes_per_block = g.chunk * self.num_layers * self.kv_dim
            ref_tensors, ref_layers = len(self.gpu_blocks), self.num_layers
        self.gpu_block_type_ = gpu_block_type_from_tensor_count(ref_tensors, ref_layers)
        self.transfer_stream = torch.cuda.Stream()
        # Gets next to puts.  The link carries both directions at once (93 GB/s in
        # sum against 57 one after the other), so with `overlap_directions` D2H and
        # H2D ops each run on a thread and stream of their own while this thread only
        # hands them out.  Ops of one direction still run in arrival order; an op
        # that shares a block with an unfinished op of the other direction waits for
        # it.  Completions of different directions may therefore overtake each
        # other, which the reference's one-at-a-time worker never does: opt-in
        # (FKV_WORKER_OVERLAP_DIRECTIONS=1 sets the default).
        if overlap_directions is None:
            overlap_directions = os.environ.get("FKV_WORKER_OVERLAP_DIRECTIONS", "0") == "1"
        self.h2d_stream: Optional[torch.cuda.Stream] = None
        if overlap_directions:
            self.h2d_stream = self._stream_on_another_queue(self.transfer_stream)
            self._lanes["h2d"] = _SideLane("h2d", self._run_one, gpu_device_id)
            self._lanes["d2h"] = _SideLane("d2h", self._run_one, gpu_device_id)
        self.transfer_num_cta_h2d = transfer_num_cta_h2d
        self.transfer_num_cta_d2h = transfer_num_cta_d2h
        self.use_ce_transfer_h2d = use_ce_transfer_h2d
        self.use_ce_transfer_d2h = use_ce_transfer_d2h
        env = global_env()
        self.ce_path_opt = env.ce_path_opt
        self.ce_segment_threshold = env.ce_segment_threshold
        self.ce_enable_memcpy2d = env.enable_ce_memcpy2d
        # A pinned pool lives in the process that allocated it (existing memory cannot
        # be registered on every platform), so the worker that owns the pool can also
        # serve its H2DISK / DISK2H ops: given SSD files it is both workers in one.
        self.ssd: Optional[SSDPoolMover] = None
        if ssd_files:
            self.ssd = SSDPoolMover(self.cpu_tensor, ssd_files, cpu_kv_layout, ssd_kv_layout, dtype,
                                    num_blocks_per_file,
                                    multi_group=self.group_transfer_params is not None)

    @staticmethod
    def _stream_on_another_queue(first: "torch.cuda.Stream") -> "torch.cuda.Stream":
        """A stream whose kernels can run next to those of `first`: streams that the
        runtime maps to one hardware queue take turns."""
        from ..c_ext import streams_run_concurrently
        spare: List[torch.cuda.Stream] = []   # kept alive so that the next one differs
        s = torch.cuda.Stream()
        while not streams_run_concurrently(first, s) and len(spare) < 8:
            spare.append(s)
            s = torch.cuda.Stream()
        return s

    def _dispatch(self, op) -> None:
        if not self._lanes:
            return self._run_one(op)
        kind = op.transfer_type
        if kind not in (TransferType.H2D, TransferType.D2H):
            # host<->SSD ops run on this thread once both lanes are empty
            for lane in self._lanes.values():
                lane.drain()
            return self._run_one(op)
        src, dst = self.get_transfer_block_ids(op)
        src_ids, dst_ids = src.numpy(), dst.numpy()
        if kind == TransferType.H2D:   # reads host blocks `src`, writes engine blocks `dst`
            cpu_ids, gpu_ids, mine, other = src_ids, dst_ids, "h2d", "d2h"
        else:                          # reads engine blocks `src`, writes host blocks `dst`
            cpu_ids, gpu_ids, mine, other = dst_ids, src_ids, "d2h", "h2d"
        # ops of one lane run in order; an unfinished op of the other lane that touches
        # the same host or engine blocks goes first (nothing else is handed out meanwhile)
        self._lanes[other].wait_until_clear_of(cpu_ids, gpu_ids)
        self._lanes[mine].submit(op, cpu_ids, gpu_ids)

    def _init_multi_group(self, gpu_blocks_per_group, gpu_layouts_per_group,
                          cpu_kv_layout: MultiGroupBlockLayout, layer_groups) -> None:
        """One set of strides and one byte range of the host block per layer group
        (worker.py:850-945)."""
        if not isinstance(cpu_kv_layout, MultiGroupBlockLayout):
            raise ValueError("layer groups need a MultiGroupBlockLayout host pool")
        self._group_tensors = [import_tensor_handles(h) for h in gpu_blocks_per_group]
        self.group_transfer_params = []
        block_bytes = cpu_kv_layout.get_block_stride()
        total = 0
        for gi, (g, st) in enumerate(zip(layer_groups, cpu_kv_layout.get_group_strides())):
            tensors = self._group_tensors[gi]
            tpb_g = cpu_kv_layout.tokens_per_block // g.compress_ratio
            s = _measured_gpu_strides(tensors, gpu_layouts_per_group[gi], tpb_g, g.itemsize,
                                      self.kv_dim)
            self.group_transfer_params.append({
                "gpu_ptrs": _layer_ptrs(tensors), "chunk_size": s.chunk, "gpu_kv_stride": s.kv,
                "gpu_block_stride": s.block, "gpu_layer_stride": s.layer,
                "cpu_layer_stride": st["layer_stride"], "cpu_kv_stride": st["kv_stride"],
                "cpu_block_stride": block_bytes, "cpu_offset_bytes": st["offset_bytes"],
                "num_layers": g.num_layers})
            total += s.chunk * g.num_layers * self.kv_dim
        self._bytes_per_block = total

    def _control_suspend_gpu(self, payload: Any) -> int:
        """The engine is about to free its KV tensors (worker.py:928-946): finish what
        runs, let go of the tensors and their mappings.  Ops that need them fail
        until ``resume_gpu`` brings new ones."""
        if self.group_transfer_params is not None:
            raise NotImplementedError("GPU hot remap does not support multi-group KV layouts")
        if not self.gpu_blocks:
            return 0
        for lane in self._lanes.values():
            lane.drain()
        with torch.cuda.device(self.gpu_device_id):
            torch.cuda.synchronize()
        old, self.gpu_blocks = self.gpu_blocks, []
        self.gpu_blocks_ptrs = torch.zeros_like(self.gpu_blocks_ptrs)
        handles, self._gpu_handles = self._gpu_handles, []
        released = _release_imported(handles, old)
        del old
        return released

    def _control_resume_gpu(self, gpu_blocks: List[Any]) -> int:
        """New KV tensors of the same count and shape (worker.py:948-962)."""
        if self.gpu_blocks:
            discard_tensor_handles(gpu_blocks)
            raise RuntimeError("GPU blocks are already registered")
        if len(gpu_blocks) != self._gpu_block_count:
            discard_tensor_handles(gpu_blocks)
            raise ValueError(f"Expected {self._gpu_block_count} GPU blocks, got {len(gpu_blocks)}")
        self._gpu_handles = list(gpu_blocks)
        self.gpu_blocks = import_tensor_handles(gpu_blocks)
        self.gpu_blocks_ptrs = _layer_ptrs(self.gpu_blocks)
        return len(self.gpu_blocks)

    def _transfer_impl(self, src_block_ids: torch.Tensor, dst_block_ids: torch.Tensor,
                       transfer_type: TransferType) -> None:
        from ..c_ext import transfer_kv_blocks, transfer_kv_blocks_multi
        assert src_block_ids.dtype == torch.int64 and dst_block_ids.dtype == torch.int64
        assert len(src_block_ids) == len(dst_block_ids)
        gpu_ids, cpu_ids, h2d = _direction(transfer_type, src_block_ids, dst_block_ids,
                                           "GPUCPUTransferWorker")
        if len(gpu_ids) == 0:
            return
        if not self.gpu_blocks:
            raise RuntimeError("GPU blocks are suspended: no transfer until resume_gpu")
        use_ce = self._engine(self.use_ce_transfer_h2d if h2d else self.use_ce_transfer_d2h)
        num_cta = self.transfer_num_cta_h2d if h2d else self.transfer_num_cta_d2h
        tail = dict(transfer_num_cta=num_cta, is_host_to_device=h2d, use_ce_transfer=use_ce,
                    kv_dim=self.kv_dim, num_kv_heads=self.num_kv_heads,
                    gpu_block_type=self.gpu_block_type_, sync=True, ce_path_opt=self.ce_path_opt,
                    ce_segment_threshold=self.ce_segment_threshold, ce_force_path=-1,
                    ce_enable_memcpy2d=self.ce_enable_memcpy2d,
                    is_blockfirst=self.cpu_is_blockfirst,
                    enable_transfer_trace=global_env().enable_transfer_trace)
        if self.group_transfer_params is not None:
            flat = self.cpu_tensor.view(torch.uint8).view(-1)
            # one descriptor per group, its slice of the block, in one call: the library
            # puts groups of like shape into one launch and waits once, after the last
            transfer_kv_blocks_multi(
                ((gpu_ids, gp["gpu_ptrs"], gp["gpu_kv_stride"], gp["gpu_block_stride"],
                  gp["gpu_layer_stride"], cpu_ids, flat[gp["cpu_offset_bytes"]:],
                  gp["cpu_kv_stride"], gp["cpu_layer_stride"], gp["cpu_block_stride"],
                  gp["chunk_size"], 0, gp["num_layers"]), tail)
                for gp in self.group_transfer_params)
            return
        transfer_kv_blocks(gpu_ids, self.gpu_blocks_ptrs, self.gpu_kv_stride_in_bytes,
                           self.gpu_block_stride_in_bytes, self.gpu_layer_stride_in_bytes,
                           cpu_ids, self.cpu_tensor, self.cpu_kv_stride_in_bytes,
                           self.cpu_layer_stride_in_bytes, self.cpu_block_stride_in_bytes,
                           self.chunk_size_in_bytes, 0, self.num_layers, **tail)

    def launch_transfer(self, transfer_op: WorkerTransferOp) -> bool:
        src, dst = self.get_transfer_block_ids(transfer_op)
        if transfer_op.transfer_type in (TransferType.H2DISK, TransferType.DISK2H):
            if self.ssd is None:
                raise ValueError(f"Invalid transfer type: {transfer_op.transfer_type} for "
                                 "GPUCPUTransferWorker without SSD files")
            t0 = time.time()
            self.ssd.move(src.contiguous(), dst.contiguous(), transfer_op.transfer_type,
                          "GPUCPUTransferWorker")
            self._log_transfer_performance(
                transfer_op, self.ssd.bytes_per_block * transfer_op.valid_block_num, t0,
                time.time())
            return True
        stream = self.transfer_stream
        if self.h2d_stream is not None and transfer_op.transfer_type == TransferType.H2D:
            stream = self.h2d_stream
        with torch.cuda.stream(stream):
            t0 = time.time()
            self._transfer_impl(src, dst, transfer_op.transfer_type)
            t1 = time.time()
        self._log_transfer_performance(
            transfer_op, self._bytes_per_block * transfer_op.valid_block_num, t0, t1)
        return True

    def shutdown(self) -> None:
        if getattr(self, "ssd", None) is not None:
            self.ssd.close()
        super().shutdown()


class tpGPUCPUTransferWorker(TransferWorkerBase):  # noqa: N801 - the reference's name
    """All GPUs of one tensor-parallel group behind one worker: one thread and
    stream per GPU inside the transfer library (worker.py:1098-1520)."""

    def __init__(self, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                 op_buffer_tensor: torch.Tensor, gpu_blocks: List[List[Any]],
                 cpu_blocks: Union[torch.Tensor, PinnedPoolHandle],
                 gpu_kv_layouts: List[KVCacheLayout],
                 cpu_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout],
                 dtype: torch.dtype, tp_group_size: int, use_ce_transfer_h2d: Any = False,
                 use_ce_transfer_d2h: Any = False, transfer_num_cta_h2d: int = 4,
                 transfer_num_cta_d2h: int = 4,
                 layer_groups: Optional[List[LayerGroupSpec]] = None,
                 gpu_blocks_per_group: Optional[List[List[List[Any]]]] = None,
                 gpu_layouts_per_group: Optional[List[List[KVCacheLayout]]] = None,
                 allow_pageable_host: Optional[bool] = None) -> None:
        from ..c_ext import TPTransferThreadGroup
        super().__init__(worker_id, transfer_conn, finished_ops_queue, op_buffer_tensor)
        assert len(gpu_blocks) == tp_group_size
        self._gpu_handles = [list(h) for h in gpu_blocks]
        self._gpu_block_counts = [len(h) for h in gpu_blocks]
        self.gpu_blocks = [import_tensor_handles(h) for h in gpu_blocks]
        torch.cuda.set_device(self.gpu_blocks[0][0].device)
        self.cpu_tensor = self._adopt_host_pool(cpu_blocks, "tp_cpu_kv_pool", allow_pageable_host)
        self.dtype = dtype
        self.kv_dim = gpu_kv_layouts[0].kv_dim
        self.num_kv_heads = gpu_kv_layouts[0].num_kv_heads
        self.num_layers = gpu_kv_layouts[0].num_layer
        self.num_gpus = len(self.gpu_blocks)
        self.tp_group_size = tp_group_size
        self.transfer_num_cta_h2d = transfer_num_cta_h2d
        self.transfer_num_cta_d2h = transfer_num_cta_d2h
        self.use_ce_transfer_h2d = use_ce_transfer_h2d
        self.use_ce_transfer_d2h = use_ce_transfer_d2h
        env = global_env()
        self.kv_shared_across_ranks_mode = env.kv_shared_across_ranks_mode
        self.layer_groups = layer_groups
        # the byte-flat pool of a multi-group model is block-first by construction
        self.cpu_is_blockfirst = isinstance(cpu_kv_layout, MultiGroupBlockLayout) \
            or cpu_kv_layout.type == KVCacheLayoutType.BLOCKFIRST
        self._ce = dict(ce_segment_threshold=env.ce_segment_threshold, ce_path_opt=env.ce_path_opt,
                        ce_enable_memcpy2d=env.enable_ce_memcpy2d,
                        is_blockfirst=self.cpu_is_blockfirst, num_kv_heads=self.num_kv_heads,
                        ce_gather_threads=env.ce_gather_threads, ce_gather_nt=env.ce_gather_nt)
        self.tp_group_transfer_groups: Optional[List[dict]] = None
        if layer_groups is not None and gpu_blocks_per_group is not None \
                and gpu_layouts_per_group is not None:
            self._init_tp_multi_group(gpu_blocks_per_group, gpu_layouts_per_group, cpu_kv_layout,
                                      layer_groups)
            return
        sz = dtype.itemsize
        per_gpu = [_measured_gpu_strides(self.gpu_blocks[i], lay, lay.tokens_per_block, sz,
                                         self.kv_dim) for i, lay in enumerate(gpu_kv_layouts)]
        self.cpu_block_stride_in_bytes = cpu_kv_layout.get_block_stride() * sz
        self.chunk_size_in_bytes = cpu_kv_layout.get_chunk_size() * sz
        self._bytes_per_block = self.chunk_size_in_bytes * self.num_layers * self.kv_dim
        # Heads are split over the ranks right below the block axis of the host pool:
        # with separate K/V heads the kv and layer strides shrink with the per-rank
        # head count, the block stride does not (worker.py:1199-1206).
        rank_layout = cpu_kv_layout
        if self.cpu_is_blockfirst and self.num_kv_heads > 1:
            rank_layout = cpu_kv_layout.div_head(tp_group_size)
        self.cpu_layer_stride_in_bytes = rank_layout.get_layer_stride() * sz
        self.cpu_kv_stride_in_bytes = rank_layout.get_kv_stride() * sz
        self.cpu_tp_stride_in_bytes = self.cpu_block_stride_in_bytes // tp_group_size
        self.tp_transfer_thread_group = TPTransferThreadGroup(
            self.num_gpus, [t.data_ptr() for ts in self.gpu_blocks for t in ts],
            len(self.gpu_blocks[0]), self.cpu_tensor.data_ptr(), self.num_layers,
            [s.kv for s in per_gpu], [s.block for s in per_gpu], [s.layer for s in per_gpu],
            [s.chunk for s in per_gpu], [ts[0].device.index for ts in self.gpu_blocks],
            **self._ce)

    def _init_tp_multi_group(self, gpu_blocks_per_group, gpu_layouts_per_group,
                             cpu_kv_layout: MultiGroupBlockLayout, layer_groups) -> None:
        """One thread group per layer group, each on its byte range of the host
        block (worker.py:1240-1383): the block holds the groups back to back, once
        per rank, so every group shares the block stride and the stride between
        the ranks' regions."""
        from ..c_ext import TPTransferThreadGroup
        if not isinstance(cpu_kv_layout, MultiGroupBlockLayout):
            raise ValueError("layer groups need a MultiGroupBlockLayout host pool")
        # the imported tensors stay referenced: the thread groups hold addresses only
        self._group_tensors = [[import_tensor_handles(h) for h in per_gpu]
                               for per_gpu in gpu_blocks_per_group]
        block_bytes = cpu_kv_layout.get_block_stride()
        flat = self.cpu_tensor.view(torch.uint8).view(-1)
        self.tp_group_transfer_groups = []
        total = 0
        for gi, (g, st) in enumerate(zip(layer_groups, cpu_kv_layout.get_group_strides())):
            per_rank = self._group_tensors[gi]
            if len(per_rank) != self.num_gpus:
                raise ValueError(f"layer group {gi}: tensors of {len(per_rank)} GPUs, "
                                 f"{self.num_gpus} expected")
            tpb_g = cpu_kv_layout.tokens_per_block // g.compress_ratio
            strides = [_measured_gpu_strides(per_rank[i], gpu_layouts_per_group[gi][i], tpb_g,
                                             g.itemsize, self.kv_dim)
                       for i in range(self.num_gpus)]
            group = TPTransferThreadGroup(
                self.num_gpus, [t.data_ptr() for ts in per_rank for t in ts], len(per_rank[0]),
                flat[st["offset_bytes"]:].data_ptr(), g.num_layers,
                [s.kv for s in strides], [s.block for s in strides], [s.layer for s in strides],
                [s.chunk for s in strides], [ts[0].device.index for ts in per_rank], **self._ce)
            self.tp_group_transfer_groups.append({
                "tp_thread_group": group, "cpu_kv_stride": st["kv_stride"],
                "cpu_layer_stride": st["layer_stride"], "cpu_block_stride": block_bytes,
                "cpu_tp_stride": block_bytes // self.tp_group_size,
                "cpu_offset_bytes": st["offset_bytes"], "num_layers": g.num_layers,
                "chunk_size": st["chunk_size"]})
            total += st["chunk_size"] * g.num_layers * self.kv_dim
        self._bytes_per_block = total

    def _control_suspend_gpu(self, payload: Any) -> int:
        """As for the one-GPU worker (worker.py:1385-1406): the thread group is left
        with null addresses and refuses transfers until ``resume_gpu``."""
        if self.tp_group_transfer_groups is not None:
            raise NotImplementedError("GPU hot remap does not support multi-group KV layouts")
        if not self.gpu_blocks:
            return 0
        self.tp_transfer_thread_group.update_gpu_block_ptrs([0] * sum(self._gpu_block_counts))
        old, self.gpu_blocks = self.gpu_blocks, []
        handles, self._gpu_handles = self._gpu_handles, []
        released = sum(_release_imported(h, ts) for h, ts in zip(handles, old))
        del old
        return released

    def _control_resume_gpu(self, gpu_blocks: List[List[Any]]) -> int:
        """New KV tensors for every rank, as many as before (worker.py:1408-1430)."""
        if self.gpu_blocks:
            discard_tensor_handles(gpu_blocks)
            raise RuntimeError("GPU blocks are already registered")
        counts = [len(h) for h in gpu_blocks]
        if counts != self._gpu_block_counts:
            discard_tensor_handles(gpu_blocks)
            raise ValueError(f"Expected GPU block counts {self._gpu_block_counts}, got {counts}")
        self._gpu_handles = [list(h) for h in gpu_blocks]
        imported = [import_tensor_handles(h) for h in gpu_blocks]
        flat = [t.data_ptr() for ts in imported for t in ts]
        self.tp_transfer_thread_group.update_gpu_block_ptrs(flat)
        self.gpu_blocks = imported
        return len(flat)

    def _transfer_impl(self, src_block_ids: torch.Tensor, dst_block_ids: torch.Tensor,
                       transfer_type: TransferType) -> None:
        gpu_ids, cpu_ids, h2d = _direction(transfer_type, src_block_ids, dst_block_ids,
                                           "tpGPUCPUTransferWorker")
        if len(gpu_ids) == 0:
            return
        if not self.gpu_blocks:
            raise RuntimeError("GPU blocks are suspended: no transfer until resume_gpu")
        num_cta = self.transfer_num_cta_h2d if h2d else self.transfer_num_cta_d2h
        use_ce = self._engine(self.use_ce_transfer_h2d if h2d else self.use_ce_transfer_d2h)
        if self.tp_group_transfer_groups is not None:
            # one call per layer group, all layers of the group (worker.py:1461-1482)
            for gp in self.tp_group_transfer_groups:
                gp["tp_thread_group"].tp_group_transfer(
                    gpu_ids, cpu_ids, gp["cpu_kv_stride"], gp["cpu_layer_stride"],
                    gp["cpu_block_stride"], gp["cpu_tp_stride"], num_cta, h2d, use_ce, 0,
                    gp["num_layers"], self.kv_dim, self.num_kv_heads,
                    self.kv_shared_across_ranks_mode)
            return
        self.tp_transfer_thread_group.tp_group_transfer(
            gpu_ids, cpu_ids, self.cpu_kv_stride_in_bytes, self.cpu_layer_stride_in_bytes,
            self.cpu_block_stride_in_bytes, self.cpu_tp_stride_in_bytes,
            self.transfer_num_cta_h2d if h2d else self.transfer_num_cta_d2h, h2d,
            self._engine(self.use_ce_transfer_h2d if h2d else self.use_ce_transfer_d2h), 0,
            self.num_layers, self.kv_dim, self.num_kv_heads, self.kv_shared_across_ranks_mode)

    def launch_transfer(self, transfer_op: WorkerTransferOp) -> bool:
        src, dst = self.get_transfer_block_ids(transfer_op)
        t0 = time.time()
        self._transfer_impl(src, dst, transfer_op.transfer_type)
        self._log_transfer_performance(
            transfer_op, self._bytes_per_block * transfer_op.valid_block_num, t0, time.time())
        return True


class SSDPoolMover:
    """Host pool <-> SSD files for one pool (the arithmetic and the calls of
    worker.py:1522-1722).  The files of ``ssd_files`` (device -> paths) together
    hold ``ssd_kv_layout.num_block`` blocks, striped over devices and files."""

    def __init__(self, cpu_blocks: torch.Tensor, ssd_files: Dict[int, List[str]],
                 cpu_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout],
                 ssd_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout], dtype: torch.dtype,
                 num_blocks_per_file: int, multi_group: bool = False,
                 num_threads_per_device: int = 32) -> None:
        from ..c_ext import SSDIOCTX
        self.cpu_blocks = cpu_blocks
        self.num_blocks_per_file = num_blocks_per_file
        self.num_files = sum(len(v) for v in ssd_files.values())
        self.round_robin = 1
        self.num_threads_per_device = num_threads_per_device
        self.multi_group = multi_group
        if multi_group:
            # identical byte-flat blocks on both sides: a block moves as one piece
            self.block_stride_in_bytes = cpu_kv_layout.get_block_stride()
            self.kv_dim, self.num_layers = 1, 1
            self.bytes_per_block = self.block_stride_in_bytes
        else:
            if cpu_kv_layout.type != ssd_kv_layout.type:
                raise ValueError("no support for different CPU and SSD KV cache layout type")
            self.kv_dim = cpu_kv_layout.kv_dim
            self.num_layers = cpu_kv_layout.num_layer
            per_file = ssd_kv_layout.div_block(self.num_files, padding=True)
            c = TransferStrides.from_layout(cpu_kv_layout, dtype.itemsize)
            f = TransferStrides.from_layout(per_file, dtype.itemsize)
            self.chunk_size_in_bytes = c.chunk
            self.block_stride_in_bytes = c.block
            self.cpu_kv_stride_in_bytes, self.cpu_layer_stride_in_bytes = c.kv, c.layer
            self.ssd_kv_stride_in_bytes, self.ssd_layer_stride_in_bytes = f.kv, f.layer
            self.bytes_per_block = c.chunk * self.num_layers * self.kv_dim
        env = global_env()
        try:
            self.ioctx = SSDIOCTX(ssd_files, len(ssd_files), env.iouring_entries, env.iouring_flags)
        except Exception as e:
            logger.error("Error setting ssd ioctx: %s", e)
            raise RuntimeError("SSD Worker init failed") from e

    def move(self, src_block_ids: torch.Tensor, dst_block_ids: torch.Tensor,
             transfer_type: TransferType, who: str) -> None:
        from ..c_ext import transfer_kv_blocks_ssd
        if transfer_type == TransferType.H2DISK:
            ssd_ids, cpu_ids, is_read = dst_block_ids, src_block_ids, False
        elif transfer_type == TransferType.DISK2H:
            ssd_ids, cpu_ids, is_read = src_block_ids, dst_block_ids, True
        else:
            raise ValueError(f"Invalid transfer type: {transfer_type} for {who}")
        opt = global_env().ssd_io_opt
        base = self.cpu_blocks.data_ptr()
        if self.multi_group:
            b = self.block_stride_in_bytes
            transfer_kv_blocks_ssd(self.ioctx, torch.zeros(1, dtype=torch.int32), base, ssd_ids,
                                   cpu_ids, b, 0, b, 0, b, b, is_read, self.num_blocks_per_file,
                                   self.round_robin, self.num_threads_per_device, 1, opt)
            return
        transfer_kv_blocks_ssd(
            self.ioctx, torch.arange(0, self.num_layers, dtype=torch.int32), base, ssd_ids,
            cpu_ids, self.cpu_layer_stride_in_bytes, self.cpu_kv_stride_in_bytes,
            self.ssd_layer_stride_in_bytes, self.ssd_kv_stride_in_bytes, self.chunk_size_in_bytes,
            self.block_stride_in_bytes, is_read, self.num_blocks_per_file, self.round_robin,
            self.num_threads_per_device, self.kv_dim, opt)

    def close(self) -> None:
        ctx = getattr(self, "ioctx", None)
        if ctx is not None:
            ctx.close()


class CPUSSDDiskTransferWorker(TransferWorkerBase):
    """Host pool <-> SSD files (worker.py:1522-1722): H2DISK and DISK2H ops, no GPU
    involved."""

    def __init__(self, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                 op_buffer_tensor: torch.Tensor, cpu_blocks: torch.Tensor,
                 ssd_files: Dict[int, List[str]],
                 cpu_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout],
                 ssd_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout], dtype: torch.dtype,
                 num_blocks_per_file: int, layer_groups: Optional[List[LayerGroupSpec]] = None,
                 num_threads_per_device: int = 32) -> None:
        super().__init__(worker_id, transfer_conn, finished_ops_queue, op_buffer_tensor)
        self.cpu_blocks = materialize_worker_tensor(cpu_blocks)
        self.ssd = SSDPoolMover(self.cpu_blocks, ssd_files, cpu_kv_layout, ssd_kv_layout, dtype,
                                num_blocks_per_file, multi_group=layer_groups is not None,
                                num_threads_per_device=num_threads_per_device)

    def launch_transfer(self, transfer_op: WorkerTransferOp) -> bool:
        src, dst = self.get_transfer_block_ids(transfer_op)
        t0 = time.time()
        self.ssd.move(src.contiguous(), dst.contiguous(), transfer_op.transfer_type,
                      "CPUSSDDiskTransferWorker")
        self._log_transfer_performance(
            transfer_op, self.ssd.bytes_per_block * transfer_op.valid_block_num, t0, time.time())
        return True

    def shutdown(self) -> None:
        ssd = getattr(self, "ssd", None)
        if ssd is not None:
            ssd.close()
        super().shutdown()


class LayerwiseTransferWorker(TransferWorkerBase):
    """Layer-by-layer restore for an engine that starts attention on layer L while
    layer L+1 is still on the link (layerwise.py:69-1059).  The engine's per-layer
    eventfds arrive over a unix socket before the transfer group is built."""

    def __init__(self, worker_id: int, transfer_conn: Connection, finished_ops_queue,
                 op_buffer_tensor: torch.Tensor, gpu_blocks: List[List[Any]],
                 cpu_blocks: Union[torch.Tensor, PinnedPoolHandle],
                 gpu_kv_layouts: List[KVCacheLayout],
                 cpu_kv_layout: Union[KVCacheLayout, MultiGroupBlockLayout], dtype: torch.dtype,
                 tp_group_size: int, layerwise_eventfd_socket: str = "",
                 use_ce_transfer_h2d: Any = False, h2d_cta_num: int = 4,
                 enable_eventfd: bool = True,
                 layer_groups: Optional[List[LayerGroupSpec]] = None,
                 gpu_blocks_per_group: Optional[List[List[List[Any]]]] = None,
                 gpu_layouts_per_group: Optional[List[List[KVCacheLayout]]] = None,
                 num_original_layers: Optional[int] = None,
                 swa_gpu_blocks: Optional[List[List[Any]]] = None,
                 swa_cpu_blocks: Optional[Union[torch.Tensor, PinnedPoolHandle]] = None,
                 swa_gpu_kv_layouts: Optional[List[KVCacheLayout]] = None,
                 swa_cpu_kv_layout: Optional[KVCacheLayout] = None,
                 swa_dtype: Optional[torch.dtype] = None,
                 eventfd_deadline_s: float = 180.0,
                 allow_pageable_host: Optional[bool] = None,
                 ssd_files: Optional[Dict[int, List[str]]] = None,
                 ssd_kv_layout: Optional[Union[KVCacheLayout, MultiGroupBlockLayout]] = None,
                 num_blocks_per_file: int = 0,
                 swa_ssd_files: Optional[Dict[int, List[str]]] = None,
                 swa_ssd_kv_layout: Optional[KVCacheLayout] = None,
                 swa_num_blocks_per_file: int = 0) -> None:
        from .eventfd_channel import receive_layer_eventfds
        super().__init__(worker_id, transfer_conn, finished_ops_queue, op_buffer_tensor)
        assert len(gpu_blocks) == tp_group_size, \
            f"len(gpu_blocks) = {len(gpu_blocks)}, tp_group_size = {tp_group_size}"
        self.has_multi_group = (layer_groups is not None and gpu_blocks_per_group is not None
                                and gpu_layouts_per_group is not None)
        first = (gpu_blocks_per_group[0][0][0] if self.has_multi_group else gpu_blocks[0][0])
        torch.cuda.set_device(first.device if isinstance(first.device, torch.device)
                              else torch.device(first.device))
        self.gpu_blocks = [import_tensor_handles(h) for h in gpu_blocks]
        self.dtype = dtype
        self.kv_dim = gpu_kv_layouts[0].kv_dim
        self.num_kv_heads = gpu_kv_layouts[0].num_kv_heads
        self.num_gpus = len(gpu_blocks)
        self.tp_group_size = tp_group_size
        # the engine's layer index space: the eventfd table is laid out over it
        self.num_layers = (num_original_layers if self.has_multi_group
                           else gpu_kv_layouts[0].num_layer)
        if self.has_multi_group and self.num_layers is None:
            raise ValueError("a multi-group worker needs num_original_layers")
        if enable_eventfd:
            fds = receive_layer_eventfds(layerwise_eventfd_socket, tp_group_size, self.num_layers,
                                         deadline_s=eventfd_deadline_s)
        else:
            fds = torch.empty(0, dtype=torch.int32)
        self.cpu_blocks = self._adopt_host_pool(cpu_blocks, "layerwise_cpu_kv_pool",
                                                allow_pageable_host)
        self.has_swa = swa_gpu_blocks is not None and swa_cpu_blocks is not None
        env = global_env()
        self.use_ce_transfer_h2d = use_ce_transfer_h2d
        self.h2d_cta_num = h2d_cta_num
        self.kv_shared_across_ranks_mode = env.kv_shared_across_ranks_mode
        self.layerwise_notify_mode = env.layerwise_notify_mode
        self.ssd_files = ssd_files or {}
        self.enable_ssd = len(self.ssd_files) > 0
        self.num_blocks_per_file = num_blocks_per_file if self.enable_ssd else 0
        self.round_robin = 1
        self.swa_ssd_files = swa_ssd_files or {}
        self._swa_num_blocks_per_file = swa_num_blocks_per_file
        self.ssd_layer_stride_in_bytes = self.ssd_kv_stride_in_bytes = 0
        self.swa_ssd = None
        swa_kwargs: Dict[str, Any] = {"has_swa": False}
        if self.has_swa:
            self.swa_gpu_blocks = [import_tensor_handles(h) for h in swa_gpu_blocks]
            self.swa_cpu_blocks = self._adopt_host_pool(swa_cpu_blocks, "layerwise_swa_cpu_pool",
                                                        allow_pageable_host)
            assert swa_cpu_kv_layout.num_layer == self.num_layers, (
                f"SWA num_layers ({swa_cpu_kv_layout.num_layer}) must equal main-KV num_layers "
                f"({self.num_layers}): the per-layer eventfd index space is shared")
            isz = (swa_dtype or dtype).itemsize
            per_gpu = [TransferStrides.from_layout(l, isz) for l in swa_gpu_kv_layouts]
            self.swa_cpu = TransferStrides.from_layout(swa_cpu_kv_layout, isz)
            i64 = lambda xs: torch.tensor(list(xs), dtype=torch.int64)  # noqa: E731
            if self.swa_ssd_files:
                files = sum(len(v) for v in self.swa_ssd_files.values())
                self.swa_ssd = TransferStrides.from_layout(
                    swa_ssd_kv_layout.div_block(files, padding=True), isz)
            swa_kwargs = dict(
                has_swa=True, swa_gpu_blocks=self.swa_gpu_blocks,
                swa_cpu_blocks=self.swa_cpu_blocks, swa_ssd_files=self.swa_ssd_files,
                swa_gpu_kv_strides_tensor=i64(s.kv for s in per_gpu),
                swa_gpu_block_strides_tensor=i64(s.block for s in per_gpu),
                swa_gpu_layer_strides_tensor=i64(s.layer for s in per_gpu),
                swa_gpu_chunk_sizes_tensor=i64(s.chunk for s in per_gpu))
        common = dict(iouring_entries=env.iouring_entries, iouring_flags=env.iouring_flags,
                      ssd_io_opt=env.ssd_io_opt, layer_eventfds_tensor=fds,
                      tp_size=tp_group_size, ce_segment_threshold=env.ce_segment_threshold,
                      ce_path_opt=env.ce_path_opt, ce_enable_memcpy2d=env.enable_ce_memcpy2d,
                      num_kv_heads=self.num_kv_heads, ce_gather_threads=env.ce_gather_threads,
                      ce_gather_nt=env.ce_gather_nt, **swa_kwargs)
        from ..c_ext import LayerwiseTransferGroup
        if self.has_multi_group:
            self._group_tensors = [[import_tensor_handles(h) for h in per_gpu]
                                   for per_gpu in gpu_blocks_per_group]
            tables = multi_group_tables(cpu_kv_layout, self.num_layers, gpu_layouts_per_group,
                                        tp_group_size)
            self.group_cpu_block_stride = tables["cpu_block_stride"]
            self.layerwise_transfer_group = LayerwiseTransferGroup(
                num_gpus=self.num_gpus, gpu_blocks_per_group=self._group_tensors,
                cpu_blocks=self.cpu_blocks, ssd_files=self.ssd_files,
                num_original_layers=self.num_layers,
                layer_members=tables["layer_members"], is_blockfirst=True,
                **{k: v for k, v in tables.items() if k.startswith("group_")}, **common)
            self._bytes_per_block = self.group_cpu_block_stride
            return
        sz = dtype.itemsize
        per_gpu = [TransferStrides.from_layout(l, sz) for l in gpu_kv_layouts]
        c = TransferStrides.from_layout(cpu_kv_layout, sz)
        self.cpu_chunk_size_in_bytes = c.chunk
        self.cpu_block_stride_in_bytes = c.block
        self.cpu_kv_stride_in_bytes = c.kv
        self.cpu_layer_stride_in_bytes = c.layer
        blockfirst = cpu_kv_layout.type == KVCacheLayoutType.BLOCKFIRST
        rank_layout = cpu_kv_layout.div_head(tp_group_size) \
            if blockfirst and self.num_kv_heads > 1 else cpu_kv_layout
        self.cpu_tp_stride_in_bytes = c.block // tp_group_size
        self.h2d_cpu_kv_stride_in_bytes = rank_layout.get_kv_stride() * sz
        self.h2d_cpu_layer_stride_in_bytes = rank_layout.get_layer_stride() * sz
        if self.enable_ssd:  # the files split the block axis, layerwise.py:630-638
            files = sum(len(v) for v in self.ssd_files.values())
            f = TransferStrides.from_layout(ssd_kv_layout.div_block(files, padding=True), sz)
            self.ssd_layer_stride_in_bytes, self.ssd_kv_stride_in_bytes = f.layer, f.kv
        i64 = lambda xs: torch.tensor(list(xs), dtype=torch.int64)  # noqa: E731
        self.layerwise_transfer_group = LayerwiseTransferGroup(
            num_gpus=self.num_gpus, gpu_blocks=self.gpu_blocks, cpu_blocks=self.cpu_blocks,
            ssd_files=self.ssd_files, num_layers=self.num_layers,
            gpu_kv_strides_tensor=i64(s.kv for s in per_gpu),
            gpu_block_strides_tensor=i64(s.block for s in per_gpu),
            gpu_layer_strides_tensor=i64(s.layer for s in per_gpu),
            gpu_chunk_sizes_tensor=i64(s.chunk for s in per_gpu), is_blockfirst=blockfirst,
            **common)
        self._bytes_per_block = c.chunk * self.num_layers * self.kv_dim

    def _swa_call_kwargs(self, src: Optional[torch.Tensor], dst: Optional[torch.Tensor],
                         disk_src: Optional[torch.Tensor] = None,
                         disk_dst: Optional[torch.Tensor] = None) -> dict:
        if not self.has_swa or ((src is None or src.numel() == 0) and disk_src is None):
            return {}
        c = self.swa_cpu
        empty = torch.empty(0, dtype=torch.int64)
        src = empty if src is None else src
        dst = empty if dst is None else dst
        extra = {}
        if disk_src is not None and self.swa_ssd is not None:
            extra = dict(swa_disk2h_src=disk_src, swa_disk2h_dst=disk_dst,
                         swa_ssd_layer_stride_in_bytes=self.swa_ssd.layer,
                         swa_ssd_kv_stride_in_bytes=self.swa_ssd.kv,
                         swa_num_blocks_per_file=self._swa_num_blocks_per_file)
        return dict(**extra, swa_h2d_src=src, swa_h2d_dst=dst, swa_cpu_kv_stride_in_bytes=c.kv,
                    swa_cpu_layer_stride_in_bytes=c.layer, swa_cpu_block_stride_in_bytes=c.block,
                    swa_cpu_chunk_size_in_bytes=c.chunk, swa_h2d_cpu_kv_stride_in_bytes=c.kv,
                    swa_h2d_cpu_layer_stride_in_bytes=c.layer,
                    swa_cpu_tp_stride_in_bytes=c.block // self.tp_group_size)

    def _transfer_impl(self, src_h2d: torch.Tensor, dst_h2d: torch.Tensor, counter_id: int,
                       swa_src: Optional[torch.Tensor], swa_dst: Optional[torch.Tensor],
                       disk_src: Optional[torch.Tensor] = None,
                       disk_dst: Optional[torch.Tensor] = None,
                       swa_disk_src: Optional[torch.Tensor] = None,
                       swa_disk_dst: Optional[torch.Tensor] = None) -> None:
        if swa_src is not None and swa_src.numel() > 0:
            assert self.has_swa, "SWA block ids given but the worker has no SWA pool"
            assert len(swa_src) == len(swa_dst)
        empty = torch.empty(0, dtype=torch.int64)
        if disk_src is not None and not self.enable_ssd:
            raise RuntimeError("disk2h block ids given but the worker has no SSD files")
        ssd_ids = disk_src if disk_src is not None else empty
        ssd_dst = disk_dst if disk_dst is not None else empty
        use_ce = self._engine(self.use_ce_transfer_h2d)
        tail = dict(counter_id=counter_id,
                    kv_shared_across_ranks_mode=self.kv_shared_across_ranks_mode,
                    notify_mode=self.layerwise_notify_mode,
                    enable_trace=global_env().enable_transfer_trace,
                    **self._swa_call_kwargs(swa_src, swa_dst, swa_disk_src, swa_disk_dst))
        if self.has_multi_group:
            self.layerwise_transfer_group.layerwise_transfer_multi_group(
                ssd_block_ids=ssd_ids, cpu_block_ids_d2h=ssd_dst,
                num_blocks_per_file=self.num_blocks_per_file,
                round_robin=self.round_robin, num_threads_per_device=32,
                gpu_block_id_tensor=dst_h2d,
                cpu_block_id_tensor=src_h2d, transfer_cta_num=self.h2d_cta_num,
                use_ce_transfer=use_ce, kv_dim=self.kv_dim, num_kv_heads=self.num_kv_heads, **tail)
            return
        # one layer per batch: the protocol posts one eventfd per layer
        self.layerwise_transfer_group.layerwise_transfer(
            ssd_ids, ssd_dst, self.ssd_layer_stride_in_bytes, self.ssd_kv_stride_in_bytes,
            self.num_blocks_per_file, self.round_robin, 32, dst_h2d, src_h2d,
            self.cpu_kv_stride_in_bytes,
            self.cpu_layer_stride_in_bytes, self.cpu_block_stride_in_bytes,
            self.cpu_chunk_size_in_bytes, self.h2d_cpu_kv_stride_in_bytes,
            self.h2d_cpu_layer_stride_in_bytes, self.cpu_tp_stride_in_bytes, self.h2d_cta_num,
            use_ce, self.num_layers, 1, self.kv_dim, self.num_kv_heads, **tail)

    def launch_transfer(self, transfer_op: WorkerLayerwiseTransferOp) -> bool:
        def ids(a: np.ndarray) -> Optional[torch.Tensor]:
            return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)) if a.size else None

        src = torch.from_numpy(np.ascontiguousarray(transfer_op.src_block_ids_h2d, dtype=np.int64))
        dst = torch.from_numpy(np.ascontiguousarray(transfer_op.dst_block_ids_h2d, dtype=np.int64))
        t0 = time.time()
        self._transfer_impl(src, dst, transfer_op.counter_id,
                            ids(transfer_op.swa_src_block_ids_h2d),
                            ids(transfer_op.swa_dst_block_ids_h2d),
                            ids(transfer_op.src_block_ids_disk2h),
                            ids(transfer_op.dst_block_ids_disk2h),
                            ids(transfer_op.swa_src_block_ids_disk2h),
                            ids(transfer_op.swa_dst_block_ids_disk2h))
        t1 = time.time()
        if self.has_multi_group:
            size = self.group_cpu_block_stride * len(src)
        else:
            size = self.cpu_chunk_size_in_bytes * self.num_layers * len(src) * self.kv_dim
            if self.num_kv_heads == 1:
                size *= self.tp_group_size
        self._log_transfer_performance(transfer_op, size, t0, t1)
        return True

    def shutdown(self) -> None:
        group = getattr(self, "layerwise_transfer_group", None)
        if group is not None:
            try:
                group.synchronize()  # the polling notifier must finish before unpinning
            except Exception as e:  # noqa: BLE001
                logger.warning("[worker %s] layerwise synchronize failed: %s", self.worker_id, e)
        super().shutdown()
