"""Worker subclasses without a device, for exercising the process harness."""
import time

import numpy as np

from flexkv_amd.transfer.ops import WorkerTransferResult
from flexkv_amd.transfer.worker import TransferWorkerBase


class RecordingWorker(TransferWorkerBase):
    """Adds the source ids into rows of a shared tensor.  Ops whose first source id
    is negative raise; graph id 77 returns False; graph id 88 returns a per-block
    result."""

    def __init__(self, worker_id, conn, queue, op_buffer, board, fail_init=False, delay_s=0.0):
        super().__init__(worker_id, conn, queue, op_buffer)
        if fail_init:
            raise RuntimeError("constructor failure requested")
        self.board = board
        self.delay_s = delay_s
        self._bytes_per_block = 4096
        self.kv_dim = 1

    def launch_transfer(self, op):
        src, dst = self.get_transfer_block_ids(op)
        if len(src) and int(src[0]) < 0:
            raise ValueError("negative id")
        if self.delay_s:
            time.sleep(self.delay_s)
        for s, d in zip(src.tolist(), dst.tolist()):
            self.board[d] += s + 1
        if op.transfer_graph_id == 77:
            return False
        if op.transfer_graph_id == 88:
            return WorkerTransferResult(op.transfer_op_id, tuple(i % 2 == 0 for i in range(len(src))))
        return True

    def _control_board_sum(self, payload):
        return int(self.board.sum())
