"""Transfer-op records exchanged between the engine and the workers.

``TransferType`` / ``TransferOp`` / ``LayerwiseTransferOp`` follow
``flexkv/common/transfer.py:99-200`` (only the types a GPU<->CPU worker can be
handed are listed); the ``Worker*`` forms that actually cross the pipe follow
``flexkv/transfer/worker_op.py``.
"""
from __future__ import annotations

import threading
from dataclasses import dataclass, field
from enum import Enum
from typing import ClassVar, Optional, Tuple

import numpy as np


class TransferType(Enum):
    H2D = "H2D"
    D2H = "D2H"
    DISK2H = "DISK2H"
    H2DISK = "H2DISK"
    VIRTUAL = "Virtual"
    LAYERWISE = "LAYERWISE"


def _empty() -> np.ndarray:
    return np.array([], dtype=np.int64)


@dataclass
class TransferOp:
    _next_op_id: ClassVar[int] = 0
    _lock: ClassVar[threading.Lock] = threading.Lock()

    op_id: int = field(init=False)
    graph_id: int
    transfer_type: TransferType
    src_block_ids: np.ndarray
    dst_block_ids: np.ndarray
    # position of the id lists in the shared op buffer, -1 = ids travel with the op
    src_slot_id: int = -1
    dst_slot_id: int = -1
    valid_block_num: int = 0
    is_swa: bool = False

    def __post_init__(self) -> None:
        if self.transfer_type != TransferType.VIRTUAL and \
                self.src_block_ids.size != self.dst_block_ids.size:
            raise ValueError(
                "src_block_ids and dst_block_ids must have the same number of physical blocks, "
                f"but got src_block_ids.size={self.src_block_ids.size}, "
                f"dst_block_ids.size={self.dst_block_ids.size}")
        with TransferOp._lock:
            self.op_id = TransferOp._next_op_id
            TransferOp._next_op_id += 1
        assert self.src_block_ids.dtype == np.int64
        assert self.dst_block_ids.dtype == np.int64
        self.valid_block_num = self.src_block_ids.size


@dataclass
class LayerwiseTransferOp(TransferOp):
    src_block_ids_h2d: np.ndarray = field(default_factory=_empty)
    dst_block_ids_h2d: np.ndarray = field(default_factory=_empty)
    src_block_ids_disk2h: np.ndarray = field(default_factory=_empty)
    dst_block_ids_disk2h: np.ndarray = field(default_factory=_empty)
    swa_src_block_ids_h2d: np.ndarray = field(default_factory=_empty)
    swa_dst_block_ids_h2d: np.ndarray = field(default_factory=_empty)
    swa_src_block_ids_disk2h: np.ndarray = field(default_factory=_empty)
    swa_dst_block_ids_disk2h: np.ndarray = field(default_factory=_empty)
    counter_id: int = 0  # which of the eventfd sets (triple buffering) announces this op

    def __post_init__(self) -> None:
        super().__post_init__()
        assert self.transfer_type == TransferType.LAYERWISE
        for name in ("src_block_ids_h2d", "dst_block_ids_h2d", "swa_src_block_ids_h2d",
                     "swa_dst_block_ids_h2d"):
            assert getattr(self, name).dtype == np.int64, name
        if self.src_block_ids_h2d.size != self.dst_block_ids_h2d.size:
            raise ValueError("src_block_ids_h2d and dst_block_ids_h2d differ in length")
        if self.swa_src_block_ids_h2d.size != self.swa_dst_block_ids_h2d.size:
            raise ValueError("swa_src_block_ids_h2d and swa_dst_block_ids_h2d differ in length")


@dataclass(frozen=True)
class WorkerTransferResult:
    """Completion with per-block outcomes (worker_op.py:9-14)."""
    transfer_op_id: int
    block_results: Optional[Tuple[bool, ...]] = None


class WorkerTransferOp:
    """What crosses the pipe for a D2H / H2D op (worker_op.py:17-57): the id lists
    themselves only when they are not in the shared op buffer."""

    def __init__(self, transfer_op: TransferOp) -> None:
        self.transfer_op_id = transfer_op.op_id
        self.transfer_graph_id = transfer_op.graph_id
        self.transfer_type = transfer_op.transfer_type
        self.src_slot_id = transfer_op.src_slot_id
        self.dst_slot_id = transfer_op.dst_slot_id
        self.valid_block_num = transfer_op.valid_block_num
        self.prof_submitted_ns = 0
        if self.src_slot_id == -1 or self.dst_slot_id == -1:
            self.src_block_ids = transfer_op.src_block_ids
            self.dst_block_ids = transfer_op.dst_block_ids
        else:
            self.src_block_ids = np.empty(0)
            self.dst_block_ids = np.empty(0)


class WorkerLayerwiseTransferOp:
    """worker_op.py:60-93."""

    def __init__(self, transfer_op: LayerwiseTransferOp) -> None:
        assert transfer_op.transfer_type == TransferType.LAYERWISE
        self.transfer_op_id = transfer_op.op_id
        self.transfer_graph_id = transfer_op.graph_id
        self.transfer_type = transfer_op.transfer_type
        self.src_block_ids_h2d = transfer_op.src_block_ids_h2d
        self.dst_block_ids_h2d = transfer_op.dst_block_ids_h2d
        self.src_block_ids_disk2h = transfer_op.src_block_ids_disk2h
        self.dst_block_ids_disk2h = transfer_op.dst_block_ids_disk2h
        self.swa_src_block_ids_h2d = transfer_op.swa_src_block_ids_h2d
        self.swa_dst_block_ids_h2d = transfer_op.swa_dst_block_ids_h2d
        self.swa_src_block_ids_disk2h = transfer_op.swa_src_block_ids_disk2h
        self.swa_dst_block_ids_disk2h = transfer_op.swa_dst_block_ids_disk2h
        self.counter_id = transfer_op.counter_id
        self.prof_submitted_ns = 0
