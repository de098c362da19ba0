"""Environment switches read by the transfer workers
(``flexkv/common/config.py:777-835``, same variable names and defaults)."""
from __future__ import annotations

import os
from dataclasses import dataclass


@dataclass(frozen=True)
class TransferEnv:
    use_ce_transfer_h2d: bool
    use_ce_transfer_d2h: bool
    transfer_num_cta_h2d: int
    transfer_num_cta_d2h: int
    ce_segment_threshold: int
    ce_path_opt: bool
    enable_ce_memcpy2d: bool
    ce_gather_threads: int
    ce_gather_nt: bool
    enable_transfer_trace: bool
    kv_shared_across_ranks_mode: str
    layerwise_notify_mode: str
    worker_shutdown_timeout_s: float
    ssd_io_opt: bool
    iouring_entries: int
    iouring_flags: int

    @classmethod
    def from_env(cls) -> "TransferEnv":
        g = os.getenv
        return cls(
            use_ce_transfer_h2d=bool(int(g("FLEXKV_USE_CE_TRANSFER_H2D", 0))),
            use_ce_transfer_d2h=bool(int(g("FLEXKV_USE_CE_TRANSFER_D2H", 0))),
            transfer_num_cta_h2d=int(g("FLEXKV_TRANSFER_NUM_CTA_H2D", 4)),
            transfer_num_cta_d2h=int(g("FLEXKV_TRANSFER_NUM_CTA_D2H", 4)),
            ce_segment_threshold=int(g("FLEXKV_CE_SEGMENT_THRESHOLD", 8)),
            ce_path_opt=bool(int(g("FLEXKV_CE_PATH_OPT", 1))),
            enable_ce_memcpy2d=bool(int(g("FLEXKV_ENABLE_CE_MEMCPY2D", 1))),
            ce_gather_threads=int(g("FLEXKV_CE_GATHER_THREADS", 4)),
            ce_gather_nt=bool(int(g("FLEXKV_CE_GATHER_NT", 1))),
            enable_transfer_trace=bool(int(g("FLEXKV_TRANSFER_TRACE", 0))),
            kv_shared_across_ranks_mode=g("FLEXKV_KV_SHARED_ACROSS_RANKS_MODE", "sharded"),
            layerwise_notify_mode=g("FLEXKV_LAYERWISE_NOTIFY_MODE", "hostfunc"),
            worker_shutdown_timeout_s=float(g("FLEXKV_WORKER_SHUTDOWN_TIMEOUT_S", 600)),
            ssd_io_opt=bool(int(g("FLEXKV_SSD_IO_OPT", 1))),
            iouring_entries=int(g("FLEXKV_IOURING_ENTRIES", 512)),
            iouring_flags=int(g("FLEXKV_IOURING_FLAGS", 0)),
        )


def global_env() -> TransferEnv:
    """Read once per process, like GLOBAL_CONFIG_FROM_ENV."""
    global _ENV
    if _ENV is None:
        _ENV = TransferEnv.from_env()
    return _ENV


_ENV = None
