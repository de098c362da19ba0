"""Per-transfer trace lines.

Covers what ``flexkv/transfer/trace.py`` of the reference provides: with the one
switch on (FLEXKV_TRANSFER_TRACE), a worker attaches lifecycle timings to each
completion report and the engine side prints one ``[XFER]`` line per op and one
``[XFER-SUMMARY]`` line per ten-second window.  Field names and formats of both
lines are the reference's (trace.py:147-168, 186-198) so existing greps keep
working; numbers are raw, nothing is judged.

State lives in one ``TransferTrace`` object per process; the module-level
functions operate on the process-wide instance.
"""
from __future__ import annotations

import logging
import threading
import time
from collections import Counter
from typing import Dict, List, Optional

logger = logging.getLogger("flexkv")

SUMMARY_WINDOW_S = 10.0


def percentile(values: List[float], p: float = 50.0) -> float:
    """Nearest-rank percentile over the sorted values, 0.0 for no values."""
    if not values:
        return 0.0
    ordered = sorted(values)
    rank = int(round(p / 100.0 * (len(ordered) - 1)))
    return ordered[min(max(rank, 0), len(ordered) - 1)]


class _Window:
    """What one summary line is made from."""

    def __init__(self, inflight_now: int = 0) -> None:
        self.started = time.monotonic()
        self.wait_ms: List[float] = []
        self.xfer_ms: List[float] = []
        self.by_type: Counter = Counter()
        self.inflight_max = inflight_now

    def add(self, metrics: dict) -> None:
        self.wait_ms.append(metrics["wait_ms"])
        self.xfer_ms.append(metrics["xfer_ms"])
        self.by_type[metrics["type"]] += 1

    def line(self, now: float) -> str:
        kinds = " ".join(f"{name}={count}" for name, count in sorted(self.by_type.items()))
        return (f"[XFER-SUMMARY] window={now - self.started:.0f}s ops={len(self.wait_ms)} "
                f"inflight_max={self.inflight_max} "
                f"wait_p50={percentile(self.wait_ms):.3f}ms "
                f"wait_p99={percentile(self.wait_ms, 99):.3f}ms "
                f"xfer_p50={percentile(self.xfer_ms):.3f}ms "
                f"xfer_p99={percentile(self.xfer_ms, 99):.3f}ms type: {kinds}")


class TransferTrace:
    def __init__(self, enabled: bool = False, emit=None) -> None:
        self.enabled = bool(enabled)
        self._emit = emit or logger.info
        self._mu = threading.Lock()
        self._submitted: Dict[int, int] = {}   # op id -> perf_counter_ns at submit
        self._inflight = 0
        self._window = _Window()

    # ---- engine side ------------------------------------------------------------
    def op_submitted(self, op_id: int, submitted_ns: int) -> None:
        if not self.enabled:
            return
        with self._mu:
            self._submitted[op_id] = submitted_ns
            self._inflight += 1
            self._window.inflight_max = max(self._window.inflight_max, self._inflight)

    def op_finished(self, op_id: int, metrics: Optional[dict]) -> None:
        """Prints the op's [XFER] line (and the summary when its window is over)."""
        if not self.enabled:
            return
        with self._mu:
            t0 = self._submitted.pop(op_id, None)
            self._inflight = max(0, self._inflight - 1)
            backlog = self._inflight
        if metrics is None:
            return
        e2e_ms = 0.0 if t0 is None else (time.perf_counter_ns() - t0) / 1e6
        self._emit(xfer_line(op_id, metrics, e2e_ms, backlog))
        with self._mu:
            self._window.add(metrics)
            now = time.monotonic()
            if now - self._window.started >= SUMMARY_WINDOW_S:
                self._emit(self._window.line(now))
                self._window = _Window(self._inflight)

    def inflight(self) -> int:
        with self._mu:
            return self._inflight if self.enabled else 0

    def flush_summary(self) -> Optional[str]:
        """Ends the current window now; returns the line it printed."""
        if not self.enabled:
            return None
        with self._mu:
            line = self._window.line(time.monotonic())
            self._window = _Window(self._inflight)
        self._emit(line)
        return line


def xfer_line(op_id: int, m: dict, e2e_ms: float, backlog: int) -> str:
    nbytes, xfer_ms = m.get("bytes", 0), m.get("xfer_ms", 0.0)
    mbps = nbytes / (xfer_ms / 1000.0) / 1e6 if nbytes > 0 and xfer_ms > 0 else 0.0
    return (f"[XFER] op={op_id} type={m['type']} nb={m['nb']} bytes={nbytes} "
            f"h2d={int(m['is_h2d'])} kv_dim={int(m['kv_dim'])} ipc={m['ipc_ms']:.3f}ms "
            f"wait={m['wait_ms']:.3f}ms xfer={xfer_ms:.3f}ms e2e={e2e_ms:.3f}ms "
            f"bw={mbps:.0f}MB/s worker={m['worker_id']} graph={m['graph_id']} backlog={backlog}")


def worker_metrics(op, submitted_ns: int, received_ns: int, launch_ns: int, launched_ns: int,
                   worker_id: int, bytes_per_block: int, kv_dim: int, is_h2d: bool) -> dict:
    """Worker side: pipe latency (submit -> receive), queueing (receive -> launch) and
    transfer time (launch -> done) of one op plus what identifies it
    (trace.py:89-135).  ``bytes_per_block`` 0 means "unknown": bytes 0, no rate."""
    kind = getattr(op, "transfer_type", None)
    blocks = getattr(op, "valid_block_num", 0)
    if not blocks:
        h2d_ids = getattr(op, "src_block_ids_h2d", None)
        blocks = int(h2d_ids.size) if h2d_ids is not None else 0

    def ms(a: int, b: int) -> float:
        return max(0.0, (b - a) / 1e6)

    return {"type": kind.name if kind is not None else "UNKNOWN", "nb": int(blocks),
            "graph_id": getattr(op, "transfer_graph_id", -1), "worker_id": worker_id,
            "is_h2d": bool(is_h2d), "kv_dim": int(kv_dim),
            "bytes": int(bytes_per_block) * int(blocks), "ipc_ms": ms(submitted_ns, received_ns),
            "wait_ms": ms(received_ns, launch_ns), "xfer_ms": ms(launch_ns, launched_ns)}


# ---- the process-wide instance and the reference's function names ------------------------

_trace = TransferTrace(False)


def configure(enabled: bool) -> None:
    """Call once at start-up with the FLEXKV_TRANSFER_TRACE switch."""
    _trace.enabled = bool(enabled)


def is_enabled() -> bool:
    return _trace.enabled


def instance() -> TransferTrace:
    return _trace


def build_worker_metrics(op, submitted_ns, received_ns, launch_ns, launched_ns, worker_id,
                         bytes_per_block, kv_dim, is_h2d) -> Optional[dict]:
    if not _trace.enabled:
        return None
    return worker_metrics(op, submitted_ns, received_ns, launch_ns, launched_ns, worker_id,
                          bytes_per_block, kv_dim, is_h2d)


def record_submit(op_id: int, submitted_ns: int) -> None:
    _trace.op_submitted(op_id, submitted_ns)


def record_xfer(op_id: int, metrics: Optional[dict]) -> None:
    _trace.op_finished(op_id, metrics)
