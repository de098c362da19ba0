"""Operator module with the hot-path names of FlexKV's ``flexkv.c_ext``.

``transfer_kv_blocks``, ``TPTransferThreadGroup`` and ``LayerwiseTransferGroup``
take the same positional order, keyword names, defaults and error behaviour as
the pybind definitions in the reference (``csrc/bindings.cpp:439-459``,
``:761-830``, ``:471-545`` and ``:657-691``), so FlexKV's transfer workers
(``flexkv/transfer/worker.py:1002-1059, 1218-1236, 1484-1499``;
``flexkv/transfer/layerwise.py:647-664, 952-1001``) can import this module in
place of ``flexkv.c_ext`` for the GPU<->CPU path.

Everything here is a thin adapter: it pulls raw addresses and sizes out of
torch tensors, takes the current HIP stream from torch, and calls the C ABI of
``libfkv_hip.so``.  No copy is ever done in Python and there is no fallback
when the library is missing.
"""
from __future__ import annotations

import ctypes
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from ._lib import (CEConfig, LayerGroup, LayerMember, LayerwiseCall, LayerwiseMGParams,
                   LayerwiseParams, TPGroupParams, TransferDesc, check,
                   NOTIFY_HOSTFUNC, NOTIFY_POLLING)

_L = _lib.load()

__all__ = ["transfer_kv_blocks", "transfer_kv_blocks_multi", "transfer_kv_blocks_ssd", "SSDIOCTX", "TPTransferThreadGroup",
           "LayerwiseTransferGroup",
           "last_transfer_path", "get_stats", "reset_stats"]


def _ids(t: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.device.type != "cpu":
        raise ValueError(f"{name} must live in host memory")
    if t.dtype != torch.int64:
        raise TypeError(f"{name} must be int64, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


_gpu_seen = False
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream_handle() -> int:
    # Without a GPU the null stream is passed on: descriptor validation still runs
    # in the library, and the first device call there fails with a RuntimeError.
    # (torch.cuda.is_available() costs 7 us a call; once a GPU has been seen it stays.)
    global _gpu_seen
    if not _gpu_seen:
        if not torch.cuda.is_available():
            return 0
        _gpu_seen = True
    if _raw_stream is not None:
        return int(_raw_stream(torch.cuda.current_device()))
    return int(torch.cuda.current_stream().cuda_stream)


def _engine_code(use_ce_transfer) -> int:
    """False -> copy kernel, True -> copy engine, "auto" (or the integer 2) -> the
    library's per-transfer choice."""
    if use_ce_transfer == "auto" or (use_ce_transfer == 2 and not isinstance(use_ce_transfer, bool)):
        return 2
    return int(bool(use_ce_transfer))


def _ce_config(segment_threshold, path_opt, force_path, enable_memcpy2d, is_blockfirst,
               num_kv_heads, gather_threads, gather_nt) -> CEConfig:
    cfg = CEConfig()
    cfg.segment_threshold = int(segment_threshold)
    cfg.path_opt_enabled = int(bool(path_opt))
    cfg.force_path = int(force_path)
    cfg.enable_memcpy2d = int(bool(enable_memcpy2d))
    cfg.is_blockfirst = int(bool(is_blockfirst))
    cfg.num_kv_heads = int(num_kv_heads)
    cfg.gather_threads = int(gather_threads)
    cfg.gather_nt = int(bool(gather_nt))
    return cfg


def _transfer_desc(
        gpu_block_id_tensor: torch.Tensor, gpu_tensor_ptrs_tensor: torch.Tensor,
        gpu_kv_stride_in_bytes: int, gpu_block_stride_in_bytes: int,
        gpu_layer_stride_in_bytes: int, cpu_block_id_tensor: torch.Tensor,
        cpu_tensor: torch.Tensor, cpu_kv_stride_in_bytes: int,
        cpu_layer_stride_in_bytes: int, cpu_block_stride_in_bytes: int,
        chunk_size_in_bytes: int, start_layer_id: int, num_layers: int,
        transfer_num_cta: int = 4, is_host_to_device: bool = True,
        use_ce_transfer: bool = False, kv_dim: int = 2, num_kv_heads: int = 1,
        gpu_block_type: int = 0, sync: bool = True, ce_path_opt: bool = False,
        ce_segment_threshold: int = 8, ce_force_path: int = -1,
        ce_enable_memcpy2d: bool = False, is_blockfirst: bool = False,
        ce_gather_threads: int = 4, ce_gather_nt: bool = True,
        enable_transfer_trace: bool = False) -> Tuple[TransferDesc, tuple]:
    """The descriptor of one transfer and the tensors it points into (to be kept
    alive until the call has been made)."""
    gpu_ids = _ids(gpu_block_id_tensor, "gpu_block_id_tensor")
    cpu_ids = _ids(cpu_block_id_tensor, "cpu_block_id_tensor")
    if gpu_ids.numel() != cpu_ids.numel():
        raise ValueError("gpu_block_id_tensor and cpu_block_id_tensor differ in length")
    ptrs = _ids(gpu_tensor_ptrs_tensor, "gpu_tensor_ptrs_tensor")
    if cpu_tensor.device.type != "cpu":
        raise ValueError("cpu_tensor must live in host memory")

    d = TransferDesc()
    d.backend = int(gpu_block_type)
    # The reference builds its GTensorHandler with the num_layers of the call
    # (csrc/bindings.cpp:108-111), which indexes SGLang's K-then-V pointer table
    # correctly only for whole-model calls; take the true layer count from the
    # table itself so partial-layer calls address V tensors correctly too.
    d.num_layers_total = ptrs.numel() // 2 if int(gpu_block_type) == 2 else int(num_layers)
    d.gpu_tensor_ptrs = ptrs.data_ptr()
    d.num_gpu_tensor_ptrs = ptrs.numel()
    d.device = -1
    d.gpu_kv_stride = int(gpu_kv_stride_in_bytes)
    d.gpu_block_stride = int(gpu_block_stride_in_bytes)
    d.gpu_layer_stride = int(gpu_layer_stride_in_bytes)
    d.gpu_startoff_inside_chunks = 0
    d.cpu_ptr = cpu_tensor.data_ptr()
    d.cpu_kv_stride = int(cpu_kv_stride_in_bytes)
    d.cpu_layer_stride = int(cpu_layer_stride_in_bytes)
    d.cpu_block_stride = int(cpu_block_stride_in_bytes)
    d.cpu_startoff_inside_chunks = 0
    d.chunk_size = int(chunk_size_in_bytes)
    d.start_layer_id = int(start_layer_id)
    d.num_layers = int(num_layers)
    d.kv_dim = int(kv_dim)
    d.num_blocks = gpu_ids.numel()
    d.gpu_block_ids = gpu_ids.data_ptr()
    d.cpu_block_ids = cpu_ids.data_ptr()
    d.is_host_to_device = int(bool(is_host_to_device))
    d.use_ce_transfer = _engine_code(use_ce_transfer)
    d.transfer_num_cta = int(transfer_num_cta)
    d.sync = int(bool(sync))
    d.enable_trace = int(bool(enable_transfer_trace))
    d.ce = _ce_config(ce_segment_threshold, ce_path_opt, ce_force_path, ce_enable_memcpy2d,
                      is_blockfirst, num_kv_heads, ce_gather_threads, ce_gather_nt)
    return d, (gpu_ids, cpu_ids, ptrs, cpu_tensor)


def transfer_kv_blocks(
        gpu_block_id_tensor: torch.Tensor, gpu_tensor_ptrs_tensor: torch.Tensor,
        gpu_kv_stride_in_bytes: int, gpu_block_stride_in_bytes: int,
        gpu_layer_stride_in_bytes: int, cpu_block_id_tensor: torch.Tensor,
        cpu_tensor: torch.Tensor, cpu_kv_stride_in_bytes: int,
        cpu_layer_stride_in_bytes: int, cpu_block_stride_in_bytes: int,
        chunk_size_in_bytes: int, start_layer_id: int, num_layers: int,
        transfer_num_cta: int = 4, is_host_to_device: bool = True,
        use_ce_transfer: bool = False, kv_dim: int = 2, num_kv_heads: int = 1,
        gpu_block_type: int = 0, sync: bool = True, ce_path_opt: bool = False,
        ce_segment_threshold: int = 8, ce_force_path: int = -1,
        ce_enable_memcpy2d: bool = False, is_blockfirst: bool = False,
        ce_gather_threads: int = 4, ce_gather_nt: bool = True,
        enable_transfer_trace: bool = False) -> None:
    """Transfer multi-layer KV-cache between CPU and GPU on the current stream
    (``csrc/bindings.cpp:54-151``).

    ``gpu_tensor_ptrs_tensor`` is an int64 host tensor of device addresses: L
    entries for vLLM (``gpu_block_type`` 0), one for TRT-LLM (1), K₀..K_{L-1},
    V₀..V_{L-1} for SGLang (2).
    """
    d, _alive = _transfer_desc(
        gpu_block_id_tensor, gpu_tensor_ptrs_tensor, gpu_kv_stride_in_bytes,
        gpu_block_stride_in_bytes, gpu_layer_stride_in_bytes, cpu_block_id_tensor, cpu_tensor,
        cpu_kv_stride_in_bytes, cpu_layer_stride_in_bytes, cpu_block_stride_in_bytes,
        chunk_size_in_bytes, start_layer_id, num_layers, transfer_num_cta, is_host_to_device,
        use_ce_transfer, kv_dim, num_kv_heads, gpu_block_type, sync, ce_path_opt,
        ce_segment_threshold, ce_force_path, ce_enable_memcpy2d, is_blockfirst,
        ce_gather_threads, ce_gather_nt, enable_transfer_trace)
    check(_L.fkv_transfer_kv_blocks(ctypes.byref(d), _current_stream_handle()))


def transfer_kv_blocks_multi(calls) -> None:
    """Several transfers of one direction in one call: ``calls`` is a sequence of
    ``(args, kwargs)`` as ``transfer_kv_blocks`` takes them, e.g. one per layer group
    of a multi-group model (``flexkv/transfer/worker.py:998-1015`` issues them one
    after the other).  Equivalent to making the calls in order; ``sync`` of the last
    one applies to all.  On the kernel path up to four of them share one launch."""
    calls = list(calls)
    if not calls:
        return
    descs = (TransferDesc * len(calls))()
    alive = []
    for i, (args, kwargs) in enumerate(calls):
        d, keep = _transfer_desc(*args, **kwargs)
        descs[i] = d
        alive.append(keep)
    check(_L.fkv_transfer_kv_blocks_multi(descs, len(calls), _current_stream_handle()))


def layout_transform(
        buffer: torch.Tensor, buffer_layer_stride_in_bytes: int, buffer_kv_stride_in_bytes: int,
        buffer_block_stride_in_bytes: int, chunk_size_in_bytes: int,
        gpu_tensor_ptrs_tensor: torch.Tensor, gpu_kv_stride_in_bytes: int,
        gpu_block_stride_in_bytes: int, gpu_layer_stride_in_bytes: int,
        gpu_block_id_tensor: torch.Tensor, num_layers: int, kv_dim: int, buffer_to_target: bool,
        gpu_block_type: int = 0, start_layer_id: int = 0, sync: bool = False) -> None:
    """Engine KV blocks <-> a dense device buffer on the current stream
    (``launch_layout_transform_kernel``, ``csrc/gds/layout_transform.cu:26-108``;
    strides in bytes where the reference counts 8-byte words).

    Chunk (l, kv) of the i-th block id sits at ``buffer + i*block_stride +
    l*layer_stride + kv*kv_stride``.  ``buffer_to_target`` True writes the engine's
    tensors, False fills the buffer.  The block ids are a host tensor.
    """
    ids = _ids(gpu_block_id_tensor, "gpu_block_id_tensor")
    ptrs = _ids(gpu_tensor_ptrs_tensor, "gpu_tensor_ptrs_tensor")
    if buffer.device.type != "cuda":
        raise ValueError("buffer must live in device memory")
    d = _lib.LayoutTransformDesc()
    d.backend = int(gpu_block_type)
    d.num_layers_total = ptrs.numel() // 2 if int(gpu_block_type) == 2 else int(num_layers)
    d.gpu_tensor_ptrs = ptrs.data_ptr()
    d.num_gpu_tensor_ptrs = ptrs.numel()
    d.device = buffer.device.index if buffer.device.index is not None else -1
    d.gpu_kv_stride = int(gpu_kv_stride_in_bytes)
    d.gpu_block_stride = int(gpu_block_stride_in_bytes)
    d.gpu_layer_stride = int(gpu_layer_stride_in_bytes)
    d.buffer_ptr = buffer.data_ptr()
    d.buffer_layer_stride = int(buffer_layer_stride_in_bytes)
    d.buffer_kv_stride = int(buffer_kv_stride_in_bytes)
    d.buffer_block_stride = int(buffer_block_stride_in_bytes)
    d.chunk_size = int(chunk_size_in_bytes)
    d.start_layer_id = int(start_layer_id)
    d.num_layers = int(num_layers)
    d.kv_dim = int(kv_dim)
    d.num_blocks = ids.numel()
    d.gpu_block_ids = ids.data_ptr()
    d.buffer_to_target = int(bool(buffer_to_target))
    d.sync = int(bool(sync))
    need = ((d.num_blocks - 1) * d.buffer_block_stride + (d.num_layers - 1) * d.buffer_layer_stride
            + (d.kv_dim - 1) * d.buffer_kv_stride + d.chunk_size) if d.num_blocks and d.num_layers else 0
    if need > buffer.numel() * buffer.element_size():
        raise ValueError(f"buffer of {buffer.numel() * buffer.element_size()} bytes is shorter than "
                         f"the {need} bytes the strides address")
    check(_L.fkv_layout_transform(ctypes.byref(d), _current_stream_handle()))


def staging_transfer(
        comp_staging: torch.Tensor, staging_stride_in_bytes: int, comp_sizes: torch.Tensor,
        cpu_tensor: torch.Tensor, chunk_capacity_in_bytes: int, overflow: Optional[torch.Tensor],
        cpu_kv_stride_in_bytes: int, cpu_layer_stride_in_bytes: int, cpu_block_stride_in_bytes: int,
        cpu_block_id_tensor: torch.Tensor, cpu_size_table: torch.Tensor,
        cpu_size_table_block_stride: int, cpu_size_table_layer_stride: int, start_layer_id: int,
        kv_dim: int, batch_start: int, bsz: int, is_write_cpu: bool, transfer_num_cta: int = 0,
        sync: bool = False) -> None:
    """Payloads of different sizes between a dense device staging buffer and the host
    cache on the current stream, sizes kept in a host-side uint32 table
    (``staging_transfer_kernel<is_write_cpu>``,
    ``csrc/compression/common/staging_transfer.cuh:16-101``; same argument order).

    ``comp_staging`` (device, uint8) holds ``bsz`` slots of ``staging_stride`` bytes,
    ``comp_sizes`` (device, uint64-as-int64) their sizes, ``overflow`` a device int32
    counter of payloads that did not fit (may be None when reading).  ``cpu_tensor``
    and ``cpu_size_table`` are pinned host tensors, the block ids a host tensor."""
    ids = _ids(cpu_block_id_tensor, "cpu_block_id_tensor")
    if comp_staging.device.type != "cuda" or comp_sizes.device.type != "cuda":
        raise ValueError("comp_staging and comp_sizes must live in device memory")
    if comp_sizes.dtype not in (torch.int64, torch.uint64) or comp_sizes.numel() < bsz:
        raise ValueError("comp_sizes must hold bsz 64-bit sizes")
    if cpu_size_table.dtype not in (torch.int32, torch.uint32):
        raise ValueError("cpu_size_table must hold 32-bit entries")
    if comp_staging.numel() * comp_staging.element_size() < int(bsz) * int(staging_stride_in_bytes):
        raise ValueError("comp_staging is shorter than bsz slots of staging_stride bytes")
    if overflow is not None and (overflow.device.type != "cuda" or overflow.dtype != torch.int32):
        raise ValueError("overflow must be a device int32 tensor")
    d = _lib.StagingTransferDesc()
    d.staging = comp_staging.data_ptr()
    d.staging_stride = int(staging_stride_in_bytes)
    d.comp_sizes = comp_sizes.data_ptr()
    d.cpu_ptr = cpu_tensor.data_ptr()
    d.chunk_capacity = int(chunk_capacity_in_bytes)
    d.overflow = overflow.data_ptr() if overflow is not None else None
    d.cpu_kv_stride = int(cpu_kv_stride_in_bytes)
    d.cpu_layer_stride = int(cpu_layer_stride_in_bytes)
    d.cpu_block_stride = int(cpu_block_stride_in_bytes)
    d.cpu_block_ids = ids.data_ptr()
    d.size_table = cpu_size_table.data_ptr()
    d.size_table_block_stride = int(cpu_size_table_block_stride)
    d.size_table_layer_stride = int(cpu_size_table_layer_stride)
    d.start_layer_id, d.kv_dim, d.num_blocks = int(start_layer_id), int(kv_dim), ids.numel()
    d.batch_start, d.bsz = int(batch_start), int(bsz)
    d.is_write_cpu = int(bool(is_write_cpu))
    d.transfer_num_cta = int(transfer_num_cta)
    d.device = comp_staging.device.index if comp_staging.device.index is not None else -1
    d.sync = int(bool(sync))
    check(_L.fkv_staging_transfer(ctypes.byref(d), _current_stream_handle()))


def build_gpu_chunk_ptrs(
        out_ptrs: torch.Tensor, gpu_tensor_ptrs_tensor: torch.Tensor, gpu_kv_stride_in_bytes: int,
        gpu_block_stride_in_bytes: int, gpu_layer_stride_in_bytes: int,
        gpu_block_id_tensor: torch.Tensor, start_layer_id: int, kv_dim: int, batch_start: int,
        bsz: int, num_layers: int, gpu_block_type: int = 0, sync: bool = False) -> None:
    """``out_ptrs[i]`` (device, int64) = address of chunk ``batch_start + i`` of the call in
    the engine's tensors, chunks numbered layer-major, then K/V, then block position
    (``build_gpu_chunk_ptrs_kernel<Type>``,
    ``csrc/compression/common/staging_transfer.cuh:103-122``)."""
    ids = _ids(gpu_block_id_tensor, "gpu_block_id_tensor")
    ptrs = _ids(gpu_tensor_ptrs_tensor, "gpu_tensor_ptrs_tensor")
    if out_ptrs.device.type != "cuda" or out_ptrs.dtype not in (torch.int64, torch.uint64):
        raise ValueError("out_ptrs must be a 64-bit device tensor")
    if out_ptrs.numel() < bsz:
        raise ValueError("out_ptrs is shorter than bsz")
    d = _lib.ChunkPtrsDesc()
    d.out_ptrs = out_ptrs.data_ptr()
    d.backend = int(gpu_block_type)
    d.num_layers_total = ptrs.numel() // 2 if int(gpu_block_type) == 2 else int(num_layers)
    d.gpu_tensor_ptrs = ptrs.data_ptr()
    d.num_gpu_tensor_ptrs = ptrs.numel()
    d.device = out_ptrs.device.index if out_ptrs.device.index is not None else -1
    d.gpu_kv_stride = int(gpu_kv_stride_in_bytes)
    d.gpu_block_stride = int(gpu_block_stride_in_bytes)
    d.gpu_layer_stride = int(gpu_layer_stride_in_bytes)
    d.gpu_block_ids = ids.data_ptr()
    d.start_layer_id, d.kv_dim, d.num_blocks = int(start_layer_id), int(kv_dim), ids.numel()
    d.batch_start, d.bsz = int(batch_start), int(bsz)
    d.sync = int(bool(sync))
    check(_L.fkv_build_gpu_chunk_ptrs(ctypes.byref(d), _current_stream_handle()))


def streams_run_concurrently(stream_a, stream_b, device: int = -1) -> bool:
    """Whether kernels on the two torch streams can overlap, i.e. whether the
    streams sit on different hardware queues of this process.  Synchronises both."""
    out = ctypes.c_int32(0)
    check(_L.fkv_streams_run_concurrently(int(device), ctypes.c_void_p(stream_a.cuda_stream),
                                          ctypes.c_void_p(stream_b.cuda_stream),
                                          ctypes.byref(out)))
    return bool(out.value)


def streams_hand_over_us(stream_a, stream_b, device: int = -1) -> float:
    """Microseconds an event takes from one torch stream to the other and back on the
    device (a chain of waits enqueued ahead of time).  Synchronises both."""
    out = ctypes.c_double(0.0)
    check(_L.fkv_streams_hand_over_us(int(device), ctypes.c_void_p(stream_a.cuda_stream),
                                      ctypes.c_void_p(stream_b.cuda_stream), ctypes.byref(out)))
    return float(out.value)


def link_activity_post(is_host_to_device: bool, expected_us: int, device: int = -1) -> None:
    """Tell the other processes that use this GPU that this one keeps the host link
    busy in one direction for about `expected_us` more.  The library posts its own
    transfers; this is for bytes moved by other means."""
    check(_L.fkv_link_activity_post(int(device), int(bool(is_host_to_device)), int(expected_us)))


def link_activity_elsewhere(is_host_to_device: bool, window_ms: int = 20, device: int = -1) -> bool:
    """Whether another process has posted link activity of that direction on this
    GPU that has not ended more than `window_ms` ago."""
    out = ctypes.c_int32(0)
    check(_L.fkv_link_activity_elsewhere(int(device), int(bool(is_host_to_device)),
                                         int(window_ms), ctypes.byref(out)))
    return bool(out.value)


def last_transfer_path() -> str:
    """Name of the path the last transfer issued by this thread took: KERNEL or
    one of the copy-engine strategies."""
    return _lib.CE_PATH_NAMES.get(int(_L.fkv_last_path()), "UNKNOWN")


def get_stats() -> Dict[str, int]:
    s = _lib.Stats()
    _L.fkv_get_stats(ctypes.byref(s))
    return {name: int(getattr(s, name)) for name, _ in s._fields_ if name != "reserved"}


def reset_stats() -> None:
    _L.fkv_reset_stats()


def get_launch_policy(device: int = -1) -> Dict[str, int]:
    """The launch policy of ``device`` (-1: the current one) as a dict: XCD masks of
    the two directions, workgroup counts, windows, the staged restore's thresholds."""
    p = _lib.LaunchPolicy()
    check(_L.fkv_launch_policy_get(int(device), ctypes.byref(p)))
    return {name: int(getattr(p, name)) for name, _ in p._fields_ if name != "reserved"}


def set_launch_policy(device: int = -1, **fields: int) -> Dict[str, int]:
    """Change fields of the launch policy of ``device``; returns the table as it is
    afterwards (values are clamped, masks cut to the XCDs the device has)."""
    p = _lib.LaunchPolicy()
    check(_L.fkv_launch_policy_get(int(device), ctypes.byref(p)))
    known = {name for name, _ in p._fields_}
    for name, value in fields.items():
        if name not in known or name == "reserved":
            raise ValueError(f"unknown launch policy field {name!r}")
        setattr(p, name, int(value))
    check(_L.fkv_launch_policy_set(int(device), ctypes.byref(p)))
    return get_launch_policy(device)


def seed_launch_policy(device: int = -1) -> Dict[str, int]:
    """Re-base the link-dependent figures of the cost model on a measurement of ``device``
    (once per device; the library does it by itself before the first layerwise restore and
    the first transfer with ``use_ce_transfer=2``).  Returns the table."""
    check(_L.fkv_launch_policy_seed(int(device)))
    return get_launch_policy(device)


def reset_launch_policy(device: int = -1) -> None:
    check(_L.fkv_launch_policy_reset(int(device)))


class launch_policy:
    """``with launch_policy(arbiter=2): ...`` -- fields changed for the block only."""

    def __init__(self, device: int = -1, **fields: int) -> None:
        self.device, self.fields = device, fields

    def __enter__(self) -> Dict[str, int]:
        self.saved = get_launch_policy(self.device)
        return set_launch_policy(self.device, **self.fields)

    def __exit__(self, *exc) -> None:
        saved = {k: v for k, v in self.saved.items() if k not in ("xcd_count", "xcd_present_mask")}
        set_launch_policy(self.device, **saved)


class SSDIOCTX:
    """Open SSD cache files plus the I/O engine that serves them
    (``csrc/transfer_ssd.h:244-309``, ``csrc/bindings.cpp:785-787``).

    ``ssd_files`` maps device index -> list of file paths (every device the same
    number of files).  ``iouring_entries > 0`` asks for io_uring; when the kernel
    refuses it the context falls back to threads (``uses_iouring`` tells which).
    """

    def __init__(self, ssd_files: Dict[int, List[str]], num_devices: int, iouring_entries: int,
                 iouring_flags: int) -> None:
        self._h = ctypes.c_void_p()
        if num_devices < 1 or any(d not in ssd_files for d in range(num_devices)):
            raise RuntimeError("ssd_files must hold a path list for devices 0..num_devices-1")
        per_device = len(ssd_files[0])
        if per_device < 1 or any(len(ssd_files[d]) != per_device for d in range(num_devices)):
            raise RuntimeError("every SSD device must bring the same, non-zero number of files")
        flat = [str(p).encode() for d in range(num_devices) for p in ssd_files[d]]
        arr = (ctypes.c_char_p * len(flat))(*flat)
        self.num_devices, self.num_files_per_device = int(num_devices), per_device
        check(_L.fkv_ssd_open(arr, int(num_devices), per_device, int(iouring_entries),
                              int(iouring_flags), ctypes.byref(self._h)))

    @property
    def uses_iouring(self) -> bool:
        return bool(_L.fkv_ssd_uses_iouring(self._h))

    @property
    def last_transfer_was_direct(self) -> bool:
        """Whether the last transfer bypassed the page cache (O_DIRECT)."""
        return bool(_L.fkv_ssd_last_direct(self._h))

    def get_num_devices(self) -> int:
        return self.num_devices

    def get_num_files_per_device(self) -> int:
        return self.num_files_per_device

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            _L.fkv_ssd_close(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass


def transfer_kv_blocks_ssd(
        ioctx: SSDIOCTX, cpu_layer_id_list: torch.Tensor, cpu_tensor_ptr: int,
        ssd_block_ids: torch.Tensor, cpu_block_ids: torch.Tensor,
        cpu_layer_stride_in_bytes: int, cpu_kv_stride_in_bytes: int,
        ssd_layer_stride_in_bytes: int, ssd_kv_stride_in_bytes: int, chunk_size_in_bytes: int,
        block_stride_in_bytes: int, is_read: bool, num_blocks_per_file: int,
        round_robin: int = 1, num_threads_per_device: int = 16, kv_dim: int = 2,
        ssd_io_opt: bool = True) -> None:
    """Move KV blocks between the host pool and SSD files
    (``csrc/bindings.cpp:460-470``, ``csrc/transfer_ssd.cpp:327-512``).

    ``cpu_layer_id_list`` is an int32 tensor of consecutive layer ids; like the
    reference, the call covers ``[list[0], list[0] + len(list))``.  Blocks until
    the bytes have moved.  ``num_blocks_per_file`` is accepted for signature
    compatibility (the reference does not read it either).
    """
    ssd_ids = _ids(ssd_block_ids, "ssd_block_ids")
    cpu_ids = _ids(cpu_block_ids, "cpu_block_ids")
    if ssd_ids.numel() != cpu_ids.numel():
        raise ValueError("ssd_block_ids and cpu_block_ids differ in length")
    if cpu_layer_id_list.dtype != torch.int32:
        raise TypeError("cpu_layer_id_list must be int32")
    n_layers = int(cpu_layer_id_list.numel())
    start = int(cpu_layer_id_list[0]) if n_layers else 0
    check(_L.fkv_ssd_transfer(
        ioctx._h, start, n_layers, int(cpu_tensor_ptr), ssd_ids.data_ptr(), cpu_ids.data_ptr(),
        ssd_ids.numel(), int(cpu_layer_stride_in_bytes), int(cpu_kv_stride_in_bytes),
        int(ssd_layer_stride_in_bytes), int(ssd_kv_stride_in_bytes), int(chunk_size_in_bytes),
        int(block_stride_in_bytes), int(bool(is_read)), int(round_robin),
        int(num_threads_per_device), int(kv_dim), int(bool(ssd_io_opt))))


def _i64_array(values: Sequence[int], name: str, expect: Optional[int] = None) -> np.ndarray:
    arr = np.ascontiguousarray(np.asarray(list(values), dtype=np.int64))
    if expect is not None and arr.size != expect:
        raise ValueError(f"{name} must have {expect} entries, got {arr.size}")
    return arr


class TPTransferThreadGroup:
    """One transfer thread + stream per GPU of a tensor-parallel group
    (``csrc/bindings.cpp:761-830``, ``csrc/tp_transfer_thread_group.cpp``)."""

    def __init__(self, num_gpus: int, gpu_block_ptrs_flat: Sequence[int],
                 num_tensors_per_gpu: int, cpu_blocks_ptr: int, num_layers: int,
                 gpu_kv_strides_in_bytes: Sequence[int],
                 gpu_block_strides_in_bytes: Sequence[int],
                 gpu_layer_strides_in_bytes: Sequence[int],
                 gpu_chunk_sizes_in_bytes: Sequence[int],
                 gpu_device_ids: Sequence[int],
                 enable_nvcomp: bool = False, nvcomp_batch_size: int = 0,
                 nvcomp_data_type: int = 0, ce_segment_threshold: int = 8,
                 ce_path_opt: bool = True, ce_force_path: int = -1,
                 ce_enable_memcpy2d: bool = False, is_blockfirst: bool = False,
                 num_kv_heads: int = 1, ce_gather_threads: int = 4,
                 ce_gather_nt: bool = True) -> None:
        self._h = ctypes.c_void_p()
        # enable_nvcomp, nvcomp_batch_size and nvcomp_data_type are accepted and ignored, as
        # in a build of the reference without the codec (csrc/tp_transfer_thread_group.cpp:
        # 132-136).  The reference's own worker passes its copy-engine settings in these
        # positions (flexkv/transfer/worker.py:1218-1236), so a truthy value is no request.
        ptrs = np.ascontiguousarray(np.asarray(list(gpu_block_ptrs_flat), dtype=np.uint64))
        if ptrs.size != num_gpus * num_tensors_per_gpu:
            raise ValueError("gpu_block_ptrs_flat must hold num_gpus * num_tensors_per_gpu pointers")
        kvs = _i64_array(gpu_kv_strides_in_bytes, "gpu_kv_strides_in_bytes", num_gpus)
        bs = _i64_array(gpu_block_strides_in_bytes, "gpu_block_strides_in_bytes", num_gpus)
        ls = _i64_array(gpu_layer_strides_in_bytes, "gpu_layer_strides_in_bytes", num_gpus)
        cs = _i64_array(gpu_chunk_sizes_in_bytes, "gpu_chunk_sizes_in_bytes", num_gpus)
        dev = _i64_array(gpu_device_ids, "gpu_device_ids", num_gpus)
        p = TPGroupParams()
        p.num_gpus = int(num_gpus)
        p.num_tensors_per_gpu = int(num_tensors_per_gpu)
        p.gpu_block_ptrs_flat = ptrs.ctypes.data
        p.cpu_blocks_ptr = int(cpu_blocks_ptr)
        p.num_layers = int(num_layers)
        p.gpu_kv_strides = kvs.ctypes.data
        p.gpu_block_strides = bs.ctypes.data
        p.gpu_layer_strides = ls.ctypes.data
        p.gpu_chunk_sizes = cs.ctypes.data
        p.gpu_device_ids = dev.ctypes.data
        p.ce = _ce_config(ce_segment_threshold, ce_path_opt, ce_force_path, ce_enable_memcpy2d,
                          is_blockfirst, num_kv_heads, ce_gather_threads, ce_gather_nt)
        self._num_ptrs = int(ptrs.size)
        check(_L.fkv_tp_group_create(ctypes.byref(p), ctypes.byref(self._h)))

    def update_gpu_block_ptrs(self, gpu_block_ptrs_flat: Sequence[int]) -> None:
        ptrs = np.ascontiguousarray(np.asarray(list(gpu_block_ptrs_flat), dtype=np.uint64))
        check(_L.fkv_tp_group_update_gpu_block_ptrs(self._h, ptrs.ctypes.data, int(ptrs.size)))

    def tp_group_transfer(self, gpu_block_id_tensor: torch.Tensor,
                          cpu_block_id_tensor: torch.Tensor, cpu_kv_stride_in_bytes: int,
                          cpu_layer_stride_in_bytes: int, cpu_block_stride_in_bytes: int,
                          cpu_tp_stride_in_bytes: int, transfer_num_cta: int,
                          is_host_to_device: bool, use_ce_transfer: bool, layer_id: int,
                          layer_granularity: int, kv_dim: int, num_kv_heads: int,
                          kv_shared_across_ranks_mode: str = "sharded",
                          designated_rank: int = 0) -> None:
        gpu_ids = _ids(gpu_block_id_tensor, "gpu_block_id_tensor")
        cpu_ids = _ids(cpu_block_id_tensor, "cpu_block_id_tensor")
        if gpu_ids.numel() != cpu_ids.numel():
            raise ValueError("gpu_block_id_tensor and cpu_block_id_tensor differ in length")
        check(_L.fkv_tp_group_transfer(
            self._h, gpu_ids.data_ptr(), cpu_ids.data_ptr(), gpu_ids.numel(),
            int(cpu_kv_stride_in_bytes), int(cpu_layer_stride_in_bytes),
            int(cpu_block_stride_in_bytes), int(cpu_tp_stride_in_bytes),
            int(transfer_num_cta), int(bool(is_host_to_device)), int(bool(use_ce_transfer)),
            int(layer_id), int(layer_granularity), int(kv_dim), int(num_kv_heads),
            str(kv_shared_across_ranks_mode).encode(), int(designated_rank)))

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            _L.fkv_tp_group_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass


_NOTIFY = {"hostfunc": NOTIFY_HOSTFUNC, "polling": NOTIFY_POLLING}


def _numel(t) -> int:
    return int(t.numel()) if isinstance(t, torch.Tensor) else len(t)


class _GroupArrays:
    """C descriptions of layer groups plus the numpy buffers they point into."""

    def __init__(self, num_gpus: int, gpu_blocks_per_group, num_layers: Sequence[int],
                 cpu_offset_bytes, h2d_cpu_kv_strides, h2d_cpu_layer_strides,
                 cpu_block_strides, cpu_tp_strides, gpu_kv_strides, gpu_block_strides,
                 gpu_layer_strides, gpu_chunk_sizes, ctx: str) -> None:
        n = len(num_layers)
        if len(gpu_blocks_per_group) != n:  # csrc/layerwise.cpp:721-727, 398-404
            raise RuntimeError(f"{ctx} gpu_blocks_per_group size {len(gpu_blocks_per_group)} "
                               f"does not match num_groups {n}")
        self.count = n
        self.array = (LayerGroup * n)()
        self.devices: List[int] = []
        self._keep = []
        for gi in range(n):
            per_gpu = gpu_blocks_per_group[gi]
            if len(per_gpu) != num_gpus:  # :753-757
                raise RuntimeError(f"{ctx} gpu_blocks_per_group[{gi}].size() != num_gpus")
            tensors = len(per_gpu[0])
            ptrs = []
            for d in range(num_gpus):
                if len(per_gpu[d]) != tensors:  # :766-772
                    raise RuntimeError(f"{ctx} gpu_blocks_per_group[{gi}][{d}] tensor count "
                                       "mismatch")
                for t in per_gpu[d]:
                    if t.device.type != "cuda":
                        raise ValueError("gpu_blocks_per_group must hold device tensors")
                    ptrs.append(t.data_ptr())
            if gi == 0:
                self.devices = [per_gpu[d][0].device.index for d in range(num_gpus)]
            ptr_arr = np.ascontiguousarray(np.asarray(ptrs, dtype=np.uint64))
            per_dev = [np.ascontiguousarray(
                np.asarray(list(a)[gi * num_gpus:(gi + 1) * num_gpus], dtype=np.int64))
                for a in (gpu_kv_strides, gpu_block_strides, gpu_layer_strides, gpu_chunk_sizes)]
            for a in per_dev:
                if a.size != num_gpus:
                    raise ValueError(f"{ctx} per-GPU stride arrays must hold num_groups*num_gpus "
                                     "entries")
            g = self.array[gi]
            g.num_layers = int(num_layers[gi])
            g.num_tensors_per_gpu = tensors
            g.gpu_block_ptrs_flat = ptr_arr.ctypes.data
            g.cpu_offset_bytes = int(cpu_offset_bytes[gi])
            g.h2d_cpu_kv_stride = int(h2d_cpu_kv_strides[gi])
            g.h2d_cpu_layer_stride = int(h2d_cpu_layer_strides[gi])
            g.cpu_block_stride = int(cpu_block_strides[gi])
            g.cpu_tp_stride = int(cpu_tp_strides[gi])
            g.gpu_kv_strides = per_dev[0].ctypes.data
            g.gpu_block_strides = per_dev[1].ctypes.data
            g.gpu_layer_strides = per_dev[2].ctypes.data
            g.gpu_chunk_sizes = per_dev[3].ctypes.data
            self._keep.append((ptr_arr, per_dev))


def _member_csr(layer_members, num_original_layers: int, what: str):
    if len(layer_members) != num_original_layers:
        raise RuntimeError(f"{what} length {len(layer_members)} != num_original_layers "
                           f"{num_original_layers}")
    offsets = np.zeros(num_original_layers + 1, dtype=np.int32)
    flat = []
    for i, ms in enumerate(layer_members):
        for gi, local in ms:
            flat.append((int(gi), int(local)))
        offsets[i + 1] = len(flat)
    arr = (LayerMember * max(1, len(flat)))()
    for k, (gi, local) in enumerate(flat):
        arr[k].group, arr[k].local_layer = gi, local
    return offsets, arr


def _eventfd_array(layer_eventfds_tensor):
    if layer_eventfds_tensor is None or layer_eventfds_tensor.numel() == 0:
        return None
    if layer_eventfds_tensor.dtype != torch.int32:
        raise TypeError("layer_eventfds_tensor must be int32")
    return np.ascontiguousarray(layer_eventfds_tensor.cpu().numpy().reshape(-1))


class LayerwiseTransferGroup:
    """Per-layer host->GPU restore with completion signalling
    (``csrc/bindings.cpp:471-757``, ``csrc/layerwise.cpp``).

    Both constructors of the reference are provided and are told apart the way
    pybind does, by their argument names: the single-group form
    (``gpu_blocks``, ``num_layers``, ``gpu_*_strides_tensor``) and the
    multi-group form (``gpu_blocks_per_group``, ``num_original_layers``,
    ``layer_members``, ``group_*``).  With ``ssd_files`` / ``swa_ssd_files`` the
    group also performs the reference's step 0: blocks named by ``ssd_block_ids`` /
    ``swa_disk2h_src`` are read from the SSD files into the host pool, all layers
    at once, before the first layer goes to the GPU (``csrc/layerwise.cpp:1060-1110,
    1371-1432``).
    """

    _MULTI_NAMES = ("num_gpus", "gpu_blocks_per_group", "cpu_blocks", "ssd_files",
                    "num_original_layers", "layer_members", "group_num_layers",
                    "group_cpu_offset_bytes", "group_ssd_offset_bytes",
                    "group_cpu_layer_strides", "group_cpu_kv_strides",
                    "group_ssd_layer_strides", "group_ssd_kv_strides", "group_chunk_sizes",
                    "group_h2d_cpu_kv_strides", "group_h2d_cpu_layer_strides",
                    "group_cpu_block_strides", "group_cpu_tp_strides", "group_gpu_kv_strides",
                    "group_gpu_block_strides", "group_gpu_layer_strides",
                    "group_gpu_chunk_sizes", "iouring_entries", "iouring_flags",
                    "layer_eventfds_tensor", "tp_size")
    _SINGLE_NAMES = ("num_gpus", "gpu_blocks", "cpu_blocks", "ssd_files", "num_layers",
                     "gpu_kv_strides_tensor", "gpu_block_strides_tensor",
                     "gpu_layer_strides_tensor", "gpu_chunk_sizes_tensor", "iouring_entries",
                     "iouring_flags", "layer_eventfds_tensor", "tp_size")
    _COMMON_DEFAULTS = dict(has_swa=False, swa_gpu_blocks=(), swa_cpu_blocks=None,
                            swa_ssd_files=None, swa_gpu_kv_strides_tensor=None,
                            swa_gpu_block_strides_tensor=None,
                            swa_gpu_layer_strides_tensor=None, swa_gpu_chunk_sizes_tensor=None,
                            ce_segment_threshold=8, ce_path_opt=True, ce_force_path=-1,
                            ce_enable_memcpy2d=False, is_blockfirst=False, num_kv_heads=1,
                            ce_gather_threads=4, ce_gather_nt=True, ssd_io_opt=True)

    def __init__(self, *args, **kwargs) -> None:
        self._h = ctypes.c_void_p()
        multi = ("gpu_blocks_per_group" in kwargs or "layer_members" in kwargs or
                 (len(args) >= 6 and isinstance(args[5], (list, tuple))))
        required = self._MULTI_NAMES if multi else self._SINGLE_NAMES
        names = required + tuple(self._COMMON_DEFAULTS)
        if len(args) > len(names):
            raise TypeError(f"LayerwiseTransferGroup takes at most {len(names)} arguments")
        a = dict(self._COMMON_DEFAULTS)
        given = dict(zip(names, args))
        for k, v in kwargs.items():
            if k not in names:
                raise TypeError(f"LayerwiseTransferGroup got an unexpected argument {k!r}")
            if k in given:
                raise TypeError(f"LayerwiseTransferGroup got {k!r} twice")
            given[k] = v
        a.update(given)
        # tp_size is the one required name the reference's single-group form defaults
        if not multi:
            a.setdefault("tp_size", 1)
            a.setdefault("iouring_entries", 0)
            a.setdefault("iouring_flags", 0)
            a.setdefault("layer_eventfds_tensor", None)
            a.setdefault("ssd_files", None)
        missing = [k for k in required if k not in a]
        if missing:
            raise TypeError(f"LayerwiseTransferGroup missing arguments: {missing}")
        self._ssd_io_opt = bool(a["ssd_io_opt"])
        self._ioctx = self._swa_ioctx = None
        if a["ssd_files"]:
            self._ioctx = SSDIOCTX(a["ssd_files"], len(a["ssd_files"]), a["iouring_entries"],
                                   a["iouring_flags"])
        if a["swa_ssd_files"]:
            self._swa_ioctx = SSDIOCTX(a["swa_ssd_files"], len(a["swa_ssd_files"]),
                                       a["iouring_entries"], a["iouring_flags"])
        self._cpu_ptr = a["cpu_blocks"].data_ptr()
        self._swa_cpu_ptr = (a["swa_cpu_blocks"].data_ptr()
                             if a["swa_cpu_blocks"] is not None and a["swa_cpu_blocks"].numel()
                             else 0)
        self._opaque_block_stride = (int(a["group_cpu_block_strides"][0]) if multi else 0)
        self._swa_opaque_block_stride = 0
        ce = _ce_config(a["ce_segment_threshold"], a["ce_path_opt"], a["ce_force_path"],
                        a["ce_enable_memcpy2d"], a["is_blockfirst"], a["num_kv_heads"],
                        a["ce_gather_threads"], a["ce_gather_nt"])
        num_gpus = int(a["num_gpus"])
        fds = _eventfd_array(a["layer_eventfds_tensor"])
        self._num_gpus = num_gpus
        self._multi_group = multi
        self._keepalive = [a["cpu_blocks"]]
        if multi:
            self._init_multi(a, num_gpus, fds, ce)
        else:
            self._init_single(a, num_gpus, fds, ce)
        self._init_uniform_swa(a, num_gpus)

    def _init_single(self, a, num_gpus, fds, ce) -> None:
        gpu_blocks = a["gpu_blocks"]
        if gpu_blocks is None or len(gpu_blocks) != num_gpus:
            raise ValueError("gpu_blocks must hold one tensor list per GPU")
        per_gpu = len(gpu_blocks[0])
        ptrs, devs = [], []
        for tensors in gpu_blocks:
            if len(tensors) != per_gpu:
                raise ValueError("every GPU must bring the same number of KV tensors")
            for t in tensors:
                if t.device.type != "cuda":
                    raise ValueError("gpu_blocks must be device tensors")
                ptrs.append(t.data_ptr())
            devs.append(tensors[0].device.index)
        ptr_arr = np.ascontiguousarray(np.asarray(ptrs, dtype=np.uint64))
        kvs = _i64_array(a["gpu_kv_strides_tensor"].tolist(), "gpu_kv_strides_tensor", num_gpus)
        bs = _i64_array(a["gpu_block_strides_tensor"].tolist(), "gpu_block_strides_tensor",
                        num_gpus)
        ls = _i64_array(a["gpu_layer_strides_tensor"].tolist(), "gpu_layer_strides_tensor",
                        num_gpus)
        cs = _i64_array(a["gpu_chunk_sizes_tensor"].tolist(), "gpu_chunk_sizes_tensor", num_gpus)
        dev = _i64_array(devs, "gpu_device_ids", num_gpus)
        p = LayerwiseParams()
        p.num_gpus = num_gpus
        p.num_tensors_per_gpu = per_gpu
        p.gpu_block_ptrs_flat = ptr_arr.ctypes.data
        p.cpu_blocks_ptr = a["cpu_blocks"].data_ptr()
        p.num_layers = int(a["num_layers"])
        p.tp_size = int(a["tp_size"])
        p.gpu_kv_strides = kvs.ctypes.data
        p.gpu_block_strides = bs.ctypes.data
        p.gpu_layer_strides = ls.ctypes.data
        p.gpu_chunk_sizes = cs.ctypes.data
        p.gpu_device_ids = dev.ctypes.data
        p.layer_eventfds = fds.ctypes.data if fds is not None else None
        p.num_layer_eventfds = int(fds.size) if fds is not None else 0
        p.ce = ce
        # the library keeps raw addresses only: hold the tensors for its lifetime
        self._keepalive.append(gpu_blocks)
        self._num_layers = int(a["num_layers"])
        check(_L.fkv_layerwise_create(ctypes.byref(p), ctypes.byref(self._h)))

    def _init_multi(self, a, num_gpus, fds, ce) -> None:
        n_orig = int(a["num_original_layers"])
        ctx = "[LayerwiseTransferGroup multi-group]"
        if len(a["layer_members"]) != n_orig:  # csrc/layerwise.cpp:711-718
            raise RuntimeError(f"{ctx} layer_members must have length num_original_layers, got "
                               f"{len(a['layer_members'])} vs expected {n_orig}")
        groups = _GroupArrays(
            num_gpus, a["gpu_blocks_per_group"], a["group_num_layers"],
            a["group_cpu_offset_bytes"], a["group_h2d_cpu_kv_strides"],
            a["group_h2d_cpu_layer_strides"], a["group_cpu_block_strides"],
            a["group_cpu_tp_strides"], a["group_gpu_kv_strides"], a["group_gpu_block_strides"],
            a["group_gpu_layer_strides"], a["group_gpu_chunk_sizes"], ctx)
        offsets, members = _member_csr(a["layer_members"], n_orig, "layer_members")
        dev = _i64_array(groups.devices, "gpu_device_ids", num_gpus)
        p = LayerwiseMGParams()
        p.num_gpus = num_gpus
        p.num_original_layers = n_orig
        p.tp_size = int(a["tp_size"])
        p.num_groups = groups.count
        p.groups = groups.array
        p.member_offsets = offsets.ctypes.data
        p.members = members
        p.cpu_blocks_ptr = a["cpu_blocks"].data_ptr()
        p.gpu_device_ids = dev.ctypes.data
        p.layer_eventfds = fds.ctypes.data if fds is not None else None
        p.num_layer_eventfds = int(fds.size) if fds is not None else 0
        p.ce = ce
        self._keepalive.append(a["gpu_blocks_per_group"])
        self._num_layers = n_orig
        check(_L.fkv_layerwise_create_multi_group(ctypes.byref(p), ctypes.byref(self._h)))

    def _init_uniform_swa(self, a, num_gpus) -> None:
        # init_swa_sidecar_, csrc/layerwise.cpp:149-153: silently off unless all three hold
        swa_gpu_blocks = a["swa_gpu_blocks"] or ()
        swa_cpu = a["swa_cpu_blocks"]
        if not (a["has_swa"] and len(swa_gpu_blocks) > 0 and swa_cpu is not None
                and swa_cpu.numel() > 0):
            return
        zeros = [0]
        groups = _GroupArrays(
            num_gpus, [swa_gpu_blocks], [self._num_layers], zeros, zeros, zeros, zeros, zeros,
            a["swa_gpu_kv_strides_tensor"].tolist(), a["swa_gpu_block_strides_tensor"].tolist(),
            a["swa_gpu_layer_strides_tensor"].tolist(),
            a["swa_gpu_chunk_sizes_tensor"].tolist(), "[LayerwiseTransferGroup SWA]")
        self._keepalive.append((swa_gpu_blocks, swa_cpu))
        check(_L.fkv_layerwise_init_swa(self._h, groups.array, swa_cpu.data_ptr()))

    def init_swa_multi_group(
            self, swa_gpu_blocks_per_group, swa_cpu_blocks, swa_ssd_files, swa_layer_members,
            swa_group_num_layers, swa_group_cpu_offset_bytes, swa_group_ssd_offset_bytes,
            swa_group_cpu_layer_strides, swa_group_cpu_kv_strides, swa_group_ssd_layer_strides,
            swa_group_ssd_kv_strides, swa_group_chunk_sizes, swa_group_h2d_cpu_kv_strides,
            swa_group_h2d_cpu_layer_strides, swa_group_cpu_block_strides,
            swa_group_cpu_tp_strides, swa_group_gpu_kv_strides, swa_group_gpu_block_strides,
            swa_group_gpu_layer_strides, swa_group_gpu_chunk_sizes, iouring_entries: int = 512,
            iouring_flags: int = 0) -> None:
        """Attach a sidecar made of its own layer groups
        (``csrc/layerwise.cpp:355-429``, ``csrc/bindings.cpp:632-656``)."""
        if swa_cpu_blocks is None or swa_cpu_blocks.numel() == 0:
            raise RuntimeError("[LayerwiseTransferGroup] init_swa_multi_group() requires "
                               "non-empty swa_cpu_blocks")
        if len(swa_layer_members) != self._num_layers:  # :388-393
            raise RuntimeError(f"[LayerwiseTransferGroup] swa_layer_members length "
                               f"{len(swa_layer_members)} != num_original_layers "
                               f"{self._num_layers}")
        groups = _GroupArrays(
            self._num_gpus, swa_gpu_blocks_per_group, swa_group_num_layers,
            swa_group_cpu_offset_bytes, swa_group_h2d_cpu_kv_strides,
            swa_group_h2d_cpu_layer_strides, swa_group_cpu_block_strides,
            swa_group_cpu_tp_strides, swa_group_gpu_kv_strides, swa_group_gpu_block_strides,
            swa_group_gpu_layer_strides, swa_group_gpu_chunk_sizes,
            "[LayerwiseTransferGroup SWA multi-group]")
        offsets, members = _member_csr(swa_layer_members, self._num_layers, "swa_layer_members")
        check(_L.fkv_layerwise_init_swa_multi_group(
            self._h, groups.array, groups.count, offsets.ctypes.data, members,
            swa_cpu_blocks.data_ptr()))
        self._keepalive.append((swa_gpu_blocks_per_group, swa_cpu_blocks))
        self._swa_cpu_ptr = swa_cpu_blocks.data_ptr()
        self._swa_opaque_block_stride = int(swa_group_cpu_block_strides[0])
        if swa_ssd_files:
            self._swa_ioctx = SSDIOCTX(swa_ssd_files, len(swa_ssd_files), iouring_entries,
                                       iouring_flags)

    @staticmethod
    def _opaque_blocks_from_ssd(ioctx, cpu_ptr, ssd_ids, cpu_ids, block_stride, num_blocks_per_file,
                                round_robin, threads, kv_dim, opt) -> None:
        """Multi-group pools hold byte-flat blocks of identical layout in the host pool
        and on disk: a block moves as one piece (csrc/layerwise.cpp:1373-1397)."""
        transfer_kv_blocks_ssd(ioctx, torch.zeros(1, dtype=torch.int32), cpu_ptr, ssd_ids, cpu_ids,
                               block_stride, 0, block_stride, 0, block_stride, block_stride, True,
                               num_blocks_per_file, round_robin, threads, kv_dim, opt)

    def _run(self, call: LayerwiseCall, gpu_block_id_tensor, cpu_block_id_tensor, swa_h2d_src,
             swa_h2d_dst, notify_mode: str) -> None:
        gpu_ids = _ids(gpu_block_id_tensor, "gpu_block_id_tensor")
        cpu_ids = _ids(cpu_block_id_tensor, "cpu_block_id_tensor")
        if gpu_ids.numel() != cpu_ids.numel():
            raise ValueError("gpu_block_id_tensor and cpu_block_id_tensor differ in length")
        call.gpu_block_ids = gpu_ids.data_ptr()
        call.cpu_block_ids = cpu_ids.data_ptr()
        call.num_blocks = gpu_ids.numel()
        keep = None
        if swa_h2d_src is not None and _numel(swa_h2d_src) > 0:
            src = _ids(swa_h2d_src, "swa_h2d_src")
            dst = _ids(swa_h2d_dst, "swa_h2d_dst")
            if src.numel() != dst.numel():
                raise ValueError("swa_h2d_src and swa_h2d_dst differ in length")
            call.swa_cpu_block_ids = src.data_ptr()
            call.swa_gpu_block_ids = dst.data_ptr()
            call.swa_num_blocks = dst.numel()
            keep = (src, dst)
        # any string but "polling" selects the host-function mode, csrc/layerwise.cpp:987-988
        call.notify_mode = NOTIFY_POLLING if notify_mode == "polling" else NOTIFY_HOSTFUNC
        check(_L.fkv_layerwise_transfer_call(self._h, ctypes.byref(call)))
        del keep

    def layerwise_transfer_multi_group(
            self, ssd_block_ids, cpu_block_ids_d2h, num_blocks_per_file: int, round_robin: int,
            num_threads_per_device: int, gpu_block_id_tensor: torch.Tensor,
            cpu_block_id_tensor: torch.Tensor, transfer_cta_num: int, use_ce_transfer: bool,
            kv_dim: int, num_kv_heads: int, counter_id: int = 0,
            swa_h2d_src=None, swa_h2d_dst=None, swa_disk2h_src=None, swa_disk2h_dst=None,
            swa_cpu_kv_stride_in_bytes: int = 0, swa_cpu_layer_stride_in_bytes: int = 0,
            swa_cpu_block_stride_in_bytes: int = 0, swa_cpu_chunk_size_in_bytes: int = 0,
            swa_h2d_cpu_kv_stride_in_bytes: int = 0,
            swa_h2d_cpu_layer_stride_in_bytes: int = 0, swa_cpu_tp_stride_in_bytes: int = 0,
            swa_ssd_layer_stride_in_bytes: int = 0, swa_ssd_kv_stride_in_bytes: int = 0,
            swa_num_blocks_per_file: int = 0, kv_shared_across_ranks_mode: str = "sharded",
            notify_mode: str = "hostfunc", enable_trace: bool = False) -> None:
        """Restore every group member (and sidecar) of each original layer, one
        notification per original layer (``csrc/layerwise.cpp:1313-1682``)."""
        c = LayerwiseCall()
        c.multi_group = 1
        c.transfer_cta_num = int(transfer_cta_num)
        c.use_ce_transfer = _engine_code(use_ce_transfer)
        c.kv_dim = int(kv_dim)
        c.num_kv_heads = int(num_kv_heads)
        c.counter_id = int(counter_id)
        c.enable_trace = int(bool(enable_trace))
        c.kv_shared_across_ranks_mode = str(kv_shared_across_ranks_mode).encode()
        c.swa_h2d_cpu_kv_stride = int(swa_h2d_cpu_kv_stride_in_bytes)
        c.swa_h2d_cpu_layer_stride = int(swa_h2d_cpu_layer_stride_in_bytes)
        c.swa_cpu_block_stride = int(swa_cpu_block_stride_in_bytes)
        # step 0a / 0b: SSD -> host pool, csrc/layerwise.cpp:1371-1432
        if self._ioctx is not None and ssd_block_ids is not None and _numel(ssd_block_ids) > 0:
            self._opaque_blocks_from_ssd(self._ioctx, self._cpu_ptr, ssd_block_ids,
                                         cpu_block_ids_d2h, self._opaque_block_stride,
                                         num_blocks_per_file, round_robin, num_threads_per_device,
                                         int(kv_dim), self._ssd_io_opt)
        if self._swa_ioctx is not None and swa_disk2h_src is not None \
                and _numel(swa_disk2h_src) > 0:
            if self._swa_opaque_block_stride:
                self._opaque_blocks_from_ssd(self._swa_ioctx, self._swa_cpu_ptr, swa_disk2h_src,
                                             swa_disk2h_dst, self._swa_opaque_block_stride,
                                             swa_num_blocks_per_file, round_robin,
                                             num_threads_per_device, 1, self._ssd_io_opt)
            else:
                self._uniform_swa_from_ssd(
                    swa_disk2h_src, swa_disk2h_dst, swa_cpu_layer_stride_in_bytes,
                    swa_cpu_kv_stride_in_bytes, swa_ssd_layer_stride_in_bytes,
                    swa_ssd_kv_stride_in_bytes, swa_cpu_chunk_size_in_bytes,
                    swa_cpu_block_stride_in_bytes, swa_num_blocks_per_file, round_robin,
                    num_threads_per_device)
        self._run(c, gpu_block_id_tensor, cpu_block_id_tensor, swa_h2d_src, swa_h2d_dst,
                  notify_mode)

    def _uniform_swa_from_ssd(self, src, dst, cpu_layer_stride, cpu_kv_stride, ssd_layer_stride,
                              ssd_kv_stride, chunk, block_stride, num_blocks_per_file, round_robin,
                              threads) -> None:
        """All layers of the uniform sidecar in one call (csrc/layerwise.cpp:1098-1110,
        1412-1430)."""
        transfer_kv_blocks_ssd(
            self._swa_ioctx, torch.arange(0, self._num_layers, dtype=torch.int32),
            self._swa_cpu_ptr, src, dst, cpu_layer_stride, cpu_kv_stride, ssd_layer_stride,
            ssd_kv_stride, chunk, block_stride, True, num_blocks_per_file, round_robin, threads, 1,
            self._ssd_io_opt)

    def layerwise_transfer(
            self, ssd_block_ids, cpu_block_ids_d2h, ssd_layer_stride_in_bytes: int,
            ssd_kv_stride_in_bytes: int, num_blocks_per_file: int, round_robin: int,
            num_threads_per_device: int, gpu_block_id_tensor: torch.Tensor,
            cpu_block_id_tensor: torch.Tensor, cpu_kv_stride_in_bytes: int,
            cpu_layer_stride_in_bytes: int, cpu_block_stride_in_bytes: int,
            cpu_chunk_size_in_bytes: int, h2d_cpu_kv_stride_in_bytes: int,
            h2d_cpu_layer_stride_in_bytes: int, cpu_tp_stride_in_bytes: int,
            transfer_cta_num: int, use_ce_transfer: bool, num_layers: int,
            layer_granularity: int, kv_dim: int, num_kv_heads: int, counter_id: int = 0,
            swa_h2d_src=None, swa_h2d_dst=None, swa_disk2h_src=None, swa_disk2h_dst=None,
            swa_cpu_kv_stride_in_bytes: int = 0, swa_cpu_layer_stride_in_bytes: int = 0,
            swa_cpu_block_stride_in_bytes: int = 0, swa_cpu_chunk_size_in_bytes: int = 0,
            swa_h2d_cpu_kv_stride_in_bytes: int = 0,
            swa_h2d_cpu_layer_stride_in_bytes: int = 0, swa_cpu_tp_stride_in_bytes: int = 0,
            swa_ssd_layer_stride_in_bytes: int = 0, swa_ssd_kv_stride_in_bytes: int = 0,
            swa_num_blocks_per_file: int = 0, kv_shared_across_ranks_mode: str = "sharded",
            notify_mode: str = "hostfunc", enable_trace: bool = False) -> None:
        """Restore ``num_layers`` layers in batches of ``layer_granularity``
        (``csrc/layerwise.cpp:944-1311``)."""
        c = LayerwiseCall()
        c.multi_group = 0
        c.cpu_block_stride = int(cpu_block_stride_in_bytes)
        c.h2d_cpu_kv_stride = int(h2d_cpu_kv_stride_in_bytes)
        c.h2d_cpu_layer_stride = int(h2d_cpu_layer_stride_in_bytes)
        c.cpu_tp_stride = int(cpu_tp_stride_in_bytes)
        c.num_layers = int(num_layers)
        c.layer_granularity = int(layer_granularity)
        c.transfer_cta_num = int(transfer_cta_num)
        c.use_ce_transfer = _engine_code(use_ce_transfer)
        c.kv_dim = int(kv_dim)
        c.num_kv_heads = int(num_kv_heads)
        c.counter_id = int(counter_id)
        c.enable_trace = int(bool(enable_trace))
        c.kv_shared_across_ranks_mode = str(kv_shared_across_ranks_mode).encode()
        c.swa_h2d_cpu_kv_stride = int(swa_h2d_cpu_kv_stride_in_bytes)
        c.swa_h2d_cpu_layer_stride = int(swa_h2d_cpu_layer_stride_in_bytes)
        c.swa_cpu_block_stride = int(swa_cpu_block_stride_in_bytes)
        # step 0: SSD -> host pool for all layers at once, csrc/layerwise.cpp:1060-1110
        if self._ioctx is not None and ssd_block_ids is not None and _numel(ssd_block_ids) > 0:
            transfer_kv_blocks_ssd(
                self._ioctx, torch.arange(0, int(num_layers), dtype=torch.int32), self._cpu_ptr,
                ssd_block_ids, cpu_block_ids_d2h, cpu_layer_stride_in_bytes,
                cpu_kv_stride_in_bytes, ssd_layer_stride_in_bytes, ssd_kv_stride_in_bytes,
                cpu_chunk_size_in_bytes, cpu_block_stride_in_bytes, True, num_blocks_per_file,
                round_robin, num_threads_per_device, int(kv_dim), self._ssd_io_opt)
        if self._swa_ioctx is not None and swa_disk2h_src is not None \
                and _numel(swa_disk2h_src) > 0:
            self._uniform_swa_from_ssd(
                swa_disk2h_src, swa_disk2h_dst, swa_cpu_layer_stride_in_bytes,
                swa_cpu_kv_stride_in_bytes, swa_ssd_layer_stride_in_bytes,
                swa_ssd_kv_stride_in_bytes, swa_cpu_chunk_size_in_bytes,
                swa_cpu_block_stride_in_bytes, swa_num_blocks_per_file, round_robin,
                num_threads_per_device)
        self._run(c, gpu_block_id_tensor, cpu_block_id_tensor, swa_h2d_src, swa_h2d_dst,
                  notify_mode)

    # ---- additions for consumers in the same process -------------------------
    def wait_layer(self, layer: int, stream: Optional["torch.cuda.Stream"] = None,
                   gpu_index: int = 0) -> None:
        """Make ``stream`` (default: torch's current stream) wait until ``layer``
        of the last ``layerwise_transfer`` has landed."""
        handle = int((stream or torch.cuda.current_stream()).cuda_stream)
        check(_L.fkv_layerwise_wait_layer(self._h, int(gpu_index), int(layer), handle))

    def set_compute_stream(self, stream: Optional["torch.cuda.Stream"] = None,
                           gpu_index: int = 0) -> int:
        """Names the stream the engine's forward pass runs on (default: torch's current
        stream) next to this group's restores.  The group then keeps its own streams off
        that stream's hardware queue; on a shared queue a restore is added to the forward
        pass instead of hidden behind it.  Waits for ``stream``; call it at set-up.
        Returns how many of the group's streams still share the queue (normally 0)."""
        handle = int((stream or torch.cuda.current_stream()).cuda_stream)
        left = ctypes.c_int32(0)
        check(_L.fkv_layerwise_set_compute_stream(self._h, int(gpu_index), handle,
                                                  ctypes.byref(left)))
        return int(left.value)

    def synchronize(self) -> None:
        check(_L.fkv_layerwise_synchronize(self._h))

    def batch_times_ms(self) -> List[float]:
        n = ctypes.c_int32(0)
        cap = max(1, self._num_layers)
        buf = (ctypes.c_float * cap)()
        check(_L.fkv_layerwise_batch_times_ms(self._h, buf, cap, ctypes.byref(n)))
        return [float(buf[i]) for i in range(min(cap, n.value))]

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            _L.fkv_layerwise_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass
