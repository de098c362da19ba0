"""Block-id lists in shared memory.

An op that crosses the pipe to a worker carries two row numbers of this pool
instead of two id arrays; the worker pins the pool once and hands row slices
straight to the transfer call.  Same contract as ``SharedOpPool`` of the
reference (``flexkv/common/ring_buffer.py:13-97``): ``allocate_slot`` returns -1
for an empty or over-long list or when the pool is full, equal lists (per pool
kind) share a row, rows are reference counted, a double free raises.
"""
from __future__ import annotations

import threading
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

try:
    import xxhash

    def _content_key(ids: np.ndarray, kind: int) -> Tuple[int, int, int]:
        return (kind, ids.size, xxhash.xxh3_64_intdigest(ids.tobytes()))
except ImportError:  # pragma: no cover
    import hashlib

    def _content_key(ids: np.ndarray, kind: int) -> Tuple[int, int, int]:
        digest = hashlib.blake2b(ids.tobytes(), digest_size=8).digest()
        return (kind, ids.size, int.from_bytes(digest, "little"))


@dataclass
class _Row:
    key: Optional[Tuple[int, int, int]] = None
    refs: int = 0


class SharedOpPool:
    def __init__(self, max_op_num: int, max_block_num: int) -> None:
        self.max_op_num = int(max_op_num)
        self.max_block_num = int(max_block_num)
        self.buffer = torch.zeros((self.max_op_num, self.max_block_num),
                                  dtype=torch.int64).share_memory_()
        self._rows: List[_Row] = [_Row() for _ in range(self.max_op_num)]
        self._free: List[int] = list(range(self.max_op_num - 1, -1, -1))  # pop() -> lowest
        self._by_key: Dict[Tuple[int, int, int], int] = {}
        self._mu = threading.Lock()

    def allocate_slot(self, block_ids: np.ndarray, device_type_prefix: int = 0) -> int:
        """Row holding ``block_ids``.  ``device_type_prefix`` keeps equal id lists of
        different pools (GPU ids vs host ids) in different rows."""
        n = int(block_ids.size)
        if n == 0 or n > self.max_block_num:
            return -1
        ids = np.ascontiguousarray(block_ids, dtype=np.int64)
        key = _content_key(ids, int(device_type_prefix))
        with self._mu:
            slot = self._by_key.get(key)
            fresh = slot is None
            if fresh:
                if not self._free:
                    return -1
                slot = self._free.pop()
                self._by_key[key] = slot
                self._rows[slot].key = key
            self._rows[slot].refs += 1
            if fresh:
                # written under the lock: a second allocation of the same list may be
                # handed this row as soon as the key is visible
                self.buffer[slot, :n] = torch.from_numpy(ids)
        return slot

    def free_slot(self, slot_id: int) -> None:
        with self._mu:
            row = self._rows[slot_id]
            if row.key is None or row.refs <= 0:
                raise RuntimeError(f"Slot {slot_id} is not in use, double free detected!")
            row.refs -= 1
            if row.refs == 0:
                del self._by_key[row.key]
                row.key = None
                self._free.append(slot_id)

    def get_buffer(self) -> torch.Tensor:
        return self.buffer

    def get_buffer_size(self) -> Tuple[int, int]:
        return self.max_op_num, self.max_block_num

    def status(self) -> Dict[str, int]:
        with self._mu:
            used = len(self._by_key)
        return {"used_slots": used, "free_slots": self.max_op_num - used,
                "capacity": self.max_op_num}
