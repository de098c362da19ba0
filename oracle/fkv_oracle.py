"""Python side of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.

Three things live here:

* a ctypes loader for ``libfkv_oracle.so`` (the C restatement in
  ``fkv_oracle.c``) with thin numpy wrappers;
* an independent *index* formulation of the same transfer,
  ``host.view(N, L, kv, chunk)[cpu_ids, l, kv] = gpu(l, kv)[gpu_ids]`` written
  with numpy strided views and fancy indexing.  It is the row gather/scatter
  the reference's own copy-engine path performs with ATen ``index_select`` /
  ``index_copy_`` (csrc/ce_transfer.cu:1051, 1135);
* ``torch_index_gather`` / ``torch_index_scatter``: the "reference CPU path"
  (torch index-gather of the selected blocks into the host cache layout) that
  the benchmark times as its CPU baseline.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfkv_oracle.so")
_lib: Optional[ctypes.CDLL] = None

BACKEND_VLLM, BACKEND_TRTLLM, BACKEND_SGLANG = 0, 1, 2
CE_NAMES = {-1: "PER_BLOCK", 0: "CONTIG_DIRECT", 1: "SEGMENT_DIRECT",
            2: "SEGMENT_SCATTER", 3: "GATHER_SCATTER", 4: "GATHER_DIRECT"}


def build(force: bool = False) -> str:
    """Compile fkv_oracle.c with gcc into libfkv_oracle.so next to it."""
    src = os.path.join(_HERE, "fkv_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(
            ["gcc", "-O2", "-std=c11", "-Wall", "-Wextra", "-fPIC", "-shared",
             "-o", _LIB_PATH, src])
    return _LIB_PATH


class Analysis(ctypes.Structure):
    _fields_ = [("gpu_log_contig", ctypes.c_int32),
                ("cpu_log_contig", ctypes.c_int32),
                ("cpu_phys_contig", ctypes.c_int32),
                ("gpu_phys_contig", ctypes.c_int32),
                ("num_segments", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


class Segment(ctypes.Structure):
    _fields_ = [("start_k", ctypes.c_int32), ("nr_blocks", ctypes.c_int32)]


class RankPlan(ctypes.Structure):
    _fields_ = [("active", ctypes.c_int32), ("start_layer", ctypes.c_int32),
                ("num_layers", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("cpu_startoff", ctypes.c_int64), ("gpu_startoff", ctypes.c_int64),
                ("chunk_size", ctypes.c_int64)]


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, u64, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_uint64, ctypes.c_void_p
        L.fkv_oracle_units_ok.argtypes = [i64] * 9
        L.fkv_oracle_units_ok.restype = i32
        L.fkv_oracle_chunk_addr.argtypes = [i32, vp, i64, i64, i64, i64, i64, i64, i64]
        L.fkv_oracle_chunk_addr.restype = u64
        L.fkv_oracle_transfer.argtypes = [
            i32, vp, i64, i64, i64, i64, i64, vp, i64, i64, i64, i64, i64,
            i32, i32, i32, i32, vp, vp, i32]
        L.fkv_oracle_transfer.restype = i32
        L.fkv_oracle_ce_analyze.argtypes = [vp, vp, i32, i64, i64, i64,
                                            ctypes.POINTER(Analysis), vp, i32]
        L.fkv_oracle_ce_analyze.restype = None
        L.fkv_oracle_ce_choose_path.argtypes = [ctypes.POINTER(Analysis), i32, i32,
                                                i64, i64, i32, i32]
        L.fkv_oracle_ce_choose_path.restype = i32
        L.fkv_oracle_is_full_block.argtypes = [i32, i32, i64, i64]
        L.fkv_oracle_is_full_block.restype = i32
        L.fkv_oracle_tp_rank_plan.argtypes = [
            i32, i32, i32, i32, ctypes.c_char_p, i32, i32, i32, i32, i32,
            i64, i64, i64, ctypes.POINTER(RankPlan)]
        L.fkv_oracle_tp_rank_plan.restype = i32
        L.fkv_oracle_layerwise_cpu_startoff.argtypes = [i32, i32, ctypes.c_char_p,
                                                        i32, i64, i64]
        L.fkv_oracle_layerwise_cpu_startoff.restype = i64
        L.fkv_oracle_host_scatter.argtypes = [vp, vp, vp, i32, i64, i64, i64, i32,
                                              i32, i64, i64, i32]
        L.fkv_oracle_host_scatter.restype = None
        L.fkv_oracle_ssd_locate.argtypes = [i64, i32, i32, i32, ctypes.POINTER(i32),
                                            ctypes.POINTER(i32), ctypes.POINTER(i64)]
        L.fkv_oracle_ssd_locate.restype = None
        L.fkv_oracle_ssd_transfer.argtypes = [vp, i64, i32, i32, i32, i32, vp, vp, vp, i32,
                                              i64, i64, i64, i64, i64, i64, i32, i32, i32]
        L.fkv_oracle_ssd_transfer.restype = i32
        L.fkv_oracle_layout_transform.argtypes = [vp, i64, i64, i64, i64, i32, vp, i64, i64, i64,
                                                  i64, vp, i32, i32, i32, i32, i32]
        L.fkv_oracle_layout_transform.restype = i32
        L.fkv_oracle_staging_transfer.argtypes = [vp, i64, vp, vp, i64, vp, i64, i64, i64, vp, vp,
                                                  i64, i64, i32, i32, i32, i32, i32, i32]
        L.fkv_oracle_staging_transfer.restype = None
        L.fkv_oracle_chunk_ptrs.argtypes = [vp, i32, vp, i64, i64, i64, i64, vp, i32, i32, i32,
                                            i32, i32]
        L.fkv_oracle_chunk_ptrs.restype = i32
        L.fkv_oracle_eventfd_index.argtypes = [i32] * 5
        L.fkv_oracle_eventfd_index.restype = i64
        L.fkv_oracle_host_chunk_bytes.argtypes = [ctypes.c_double]
        L.fkv_oracle_host_chunk_bytes.restype = u64
        _lib = L
    return _lib


def _i64(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int64))


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def transfer_c(backend: int, tensor_ptrs: Sequence[int], num_layers_total: int,
               gpu_kv_stride: int, gpu_block_stride: int, gpu_layer_stride: int,
               gpu_off: int, cpu_ptr: int, cpu_kv_stride: int, cpu_layer_stride: int,
               cpu_block_stride: int, cpu_off: int, chunk: int, start_layer: int,
               num_layers: int, kv_dim: int, gpu_ids, cpu_ids,
               is_host_to_device: bool) -> None:
    """Run the C restatement.  All pointers are HOST addresses (ints)."""
    ptrs = np.ascontiguousarray(np.asarray(tensor_ptrs, dtype=np.uint64))
    g = _i64(gpu_ids)
    c = _i64(cpu_ids)
    assert g.shape == c.shape
    rc = lib().fkv_oracle_transfer(
        backend, _ptr(ptrs), num_layers_total, gpu_kv_stride, gpu_block_stride,
        gpu_layer_stride, gpu_off, cpu_ptr, cpu_kv_stride, cpu_layer_stride,
        cpu_block_stride, cpu_off, chunk, start_layer, num_layers, kv_dim,
        int(g.size), _ptr(g), _ptr(c), int(bool(is_host_to_device)))
    if rc != 0:
        raise ValueError(f"oracle transfer rejected backend {backend}")


def layout_transform(buffer_ptr: int, buffer_layer_stride: int, buffer_kv_stride: int,
                     buffer_block_stride: int, chunk: int, backend: int,
                     tensor_ptrs: Sequence[int], num_layers_total: int, gpu_kv_stride: int,
                     gpu_block_stride: int, gpu_layer_stride: int, gpu_ids, num_layers: int,
                     kv_dim: int, buffer_to_target: bool, start_layer: int = 0) -> None:
    """Engine blocks <-> dense buffer; all pointers are HOST addresses (ints)."""
    ptrs = np.ascontiguousarray(np.asarray(tensor_ptrs, dtype=np.uint64))
    g = _i64(gpu_ids)
    rc = lib().fkv_oracle_layout_transform(
        buffer_ptr, buffer_layer_stride, buffer_kv_stride, buffer_block_stride, chunk, backend,
        _ptr(ptrs), num_layers_total, gpu_kv_stride, gpu_block_stride, gpu_layer_stride,
        _ptr(g), int(g.size), start_layer, num_layers, kv_dim, int(bool(buffer_to_target)))
    if rc != 0:
        raise ValueError(f"oracle layout transform rejected backend {backend}")


def staging_transfer(staging: np.ndarray, staging_stride: int, comp_sizes: np.ndarray,
                     cpu: np.ndarray, chunk_capacity: int, cpu_kv_stride: int,
                     cpu_layer_stride: int, cpu_block_stride: int, cpu_ids, size_table: np.ndarray,
                     table_block_stride: int, table_layer_stride: int, start_layer: int,
                     kv_dim: int, num_blocks: int, batch_start: int, bsz: int,
                     is_write_cpu: bool) -> int:
    """Payloads of different sizes between a dense staging buffer (uint8) and the
    host cache (uint8) with their sizes in ``size_table`` (uint32); ``comp_sizes`` is
    uint64.  All arrays are host memory, modified in place.  Returns the number of
    chunks that did not fit."""
    assert staging.dtype == np.uint8 and cpu.dtype == np.uint8
    assert comp_sizes.dtype == np.uint64 and size_table.dtype == np.uint32
    ids = _i64(cpu_ids)
    overflow = np.zeros(1, dtype=np.int32)
    lib().fkv_oracle_staging_transfer(
        _ptr(staging), staging_stride, _ptr(comp_sizes), _ptr(cpu), chunk_capacity, _ptr(overflow),
        cpu_kv_stride, cpu_layer_stride, cpu_block_stride, _ptr(ids), _ptr(size_table),
        table_block_stride, table_layer_stride, start_layer, kv_dim, num_blocks, batch_start, bsz,
        int(bool(is_write_cpu)))
    return int(overflow[0])


def chunk_ptrs(backend, tensor_ptrs, num_layers_total, kvs, bs, ls, gpu_ids, start_layer, kv_dim,
               batch_start, bsz) -> np.ndarray:
    """Addresses of the chunks of a batch, numbered layer-major, then K/V, then block."""
    ptrs = np.ascontiguousarray(np.asarray(tensor_ptrs, dtype=np.uint64))
    ids = _i64(gpu_ids)
    out = np.zeros(bsz, dtype=np.uint64)
    rc = lib().fkv_oracle_chunk_ptrs(_ptr(out), backend, _ptr(ptrs), num_layers_total, kvs, bs, ls,
                                     _ptr(ids), start_layer, kv_dim, int(ids.size), batch_start,
                                     bsz)
    if rc != 0:
        raise ValueError(f"oracle chunk_ptrs rejected backend {backend}")
    return out


def chunk_addr(backend, tensor_ptrs, num_layers_total, kvs, bs, ls, layer, kv, block) -> int:
    ptrs = np.ascontiguousarray(np.asarray(tensor_ptrs, dtype=np.uint64))
    return int(lib().fkv_oracle_chunk_addr(backend, _ptr(ptrs), num_layers_total,
                                           kvs, bs, ls, layer, kv, block))


def ce_analyze(gpu_ids, cpu_ids, cpu_block_stride, chunk, gpu_block_stride):
    g, c = _i64(gpu_ids), _i64(cpu_ids)
    n = int(g.size)
    out = Analysis()
    segs = (Segment * max(n, 1))()
    lib().fkv_oracle_ce_analyze(_ptr(g), _ptr(c), n, cpu_block_stride, chunk,
                                gpu_block_stride, ctypes.byref(out),
                                ctypes.cast(segs, ctypes.c_void_p), max(n, 1))
    seg_list = [(segs[i].start_k, segs[i].nr_blocks) for i in range(out.num_segments)]
    return out, seg_list


def ce_choose_path(analysis: Analysis, is_blockfirst: bool, num_kv_heads: int,
                   segment_threshold: int, chunk: int, is_host_to_device: bool,
                   is_full_block: bool) -> int:
    return int(lib().fkv_oracle_ce_choose_path(
        ctypes.byref(analysis), int(is_blockfirst), num_kv_heads, segment_threshold,
        chunk, int(is_host_to_device), int(is_full_block)))


def is_full_block(num_layers: int, kv_dim: int, chunk: int, cpu_block_stride: int) -> bool:
    return bool(lib().fkv_oracle_is_full_block(num_layers, kv_dim, chunk, cpu_block_stride))


def eventfd_index(counter: int, tp_rank: int, layer: int, tp_size: int, num_layers: int) -> int:
    return int(lib().fkv_oracle_eventfd_index(counter, tp_rank, layer, tp_size, num_layers))


def host_scatter(staging: np.ndarray, cpu: np.ndarray, cpu_ids, cpu_block_stride: int,
                 cpu_off: int, chunk: int, layer: int, kv: int, cpu_kv_stride: int,
                 cpu_layer_stride: int, to_cpu: bool) -> None:
    """Rows of one (layer, kv) between a dense staging array and the host cache,
    in place on the two uint8 arrays."""
    ids = _i64(cpu_ids)
    assert staging.dtype == np.uint8 and cpu.dtype == np.uint8
    assert staging.flags.c_contiguous and cpu.flags.c_contiguous
    assert staging.size >= ids.size * chunk
    lib().fkv_oracle_host_scatter(_ptr(staging), _ptr(cpu), _ptr(ids), ids.size, cpu_block_stride,
                                  cpu_off, chunk, layer, kv, cpu_kv_stride, cpu_layer_stride,
                                  int(to_cpu))


def tp_rank_plan(rank, num_gpus, num_kv_heads, is_h2d, mode, designated_rank,
                 rotate_counter, layer_id, layer_granularity, num_blocks,
                 gpu_chunk_size, cpu_block_stride, cpu_tp_stride):
    out = RankPlan()
    rc = lib().fkv_oracle_tp_rank_plan(
        rank, num_gpus, num_kv_heads, int(is_h2d), mode.encode(), designated_rank,
        rotate_counter, layer_id, layer_granularity, num_blocks, gpu_chunk_size,
        cpu_block_stride, cpu_tp_stride, ctypes.byref(out))
    if rc != 0:
        raise ValueError("sharded D2H needs gpu_chunk_size divisible by num_gpus")
    return out


# ---------------------------------------------------------------------------
# Independent index formulation (numpy strided views + fancy indexing)
# ---------------------------------------------------------------------------

def _view(base: np.ndarray, offset: int, shape, strides) -> np.ndarray:
    """uint8 strided view into ``base`` starting at byte ``offset``; bounds are
    checked so a wrong stride raises instead of reading outside ``base``."""
    last = offset + sum((s - 1) * st for s, st in zip(shape, strides) if s > 0)
    if offset < 0 or (all(s > 0 for s in shape) and last >= base.size):
        raise IndexError(f"strided view [{offset}, {last}] outside buffer of {base.size} B")
    return np.lib.stride_tricks.as_strided(base[offset:], shape=shape, strides=strides)


def transfer_index(backend: int, gpu_buffers: List[np.ndarray], num_layers_total: int,
                   gpu_kv_stride: int, gpu_block_stride: int, gpu_layer_stride: int,
                   gpu_off: int, host: np.ndarray, cpu_kv_stride: int,
                   cpu_layer_stride: int, cpu_block_stride: int, cpu_off: int,
                   chunk: int, start_layer: int, num_layers: int, kv_dim: int,
                   gpu_ids, cpu_ids, is_host_to_device: bool) -> None:
    """Row gather/scatter with numpy fancy indexing.

    ``gpu_buffers`` are flat uint8 arrays, one per engine tensor (1 for
    TRT-LLM, L for vLLM, 2L for SGLang); ``host`` is the flat uint8 host pool.
    """
    g, c = _i64(gpu_ids), _i64(cpu_ids)
    if g.size == 0:
        return
    for l in range(start_layer, start_layer + num_layers):
        for kv in range(kv_dim):
            if backend == BACKEND_VLLM:
                buf, off = gpu_buffers[l], kv * gpu_kv_stride
            elif backend == BACKEND_TRTLLM:
                buf, off = gpu_buffers[0], l * gpu_layer_stride + kv * gpu_kv_stride
            elif backend == BACKEND_SGLANG:
                buf, off = gpu_buffers[kv * num_layers_total + l], 0
            else:
                raise ValueError(backend)
            rows_g = _view(buf, off + gpu_off, (int(g.max()) + 1, chunk),
                           (gpu_block_stride, 1))
            rows_c = _view(host, l * cpu_layer_stride + kv * cpu_kv_stride + cpu_off,
                           (int(c.max()) + 1, chunk), (cpu_block_stride, 1))
            if is_host_to_device:
                rows_g[g] = rows_c[c]
            else:
                rows_c[c] = rows_g[g]


# ---------------------------------------------------------------------------
# "Reference CPU path": torch index-gather into the host cache layout.
# ---------------------------------------------------------------------------

def torch_index_gather(layers, host_cache, gpu_ids, cpu_ids) -> None:
    """vLLM-shaped tensors resident in host RAM -> BLOCKFIRST host cache.

    ``layers[l]`` is ``[kv, N, T, H, D]``; ``host_cache`` is
    ``[NH, L, kv, T, H, D]``.  host_cache[cpu_ids, l] = layers[l][:, gpu_ids]
    (block axis moved first)."""
    import torch
    for l, layer in enumerate(layers):
        picked = torch.index_select(layer, 1, gpu_ids)          # [kv, n, T, H, D]
        host_cache[:, l].index_copy_(0, cpu_ids, picked.transpose(0, 1))


def torch_index_scatter(layers, host_cache, gpu_ids, cpu_ids) -> None:
    """Inverse of torch_index_gather: layers[l][:, gpu_ids] = host_cache[cpu_ids, l]."""
    import torch
    for l, layer in enumerate(layers):
        picked = torch.index_select(host_cache[:, l], 0, cpu_ids)  # [n, kv, T, H, D]
        layer.index_copy_(1, gpu_ids, picked.transpose(0, 1))


def torch_index_gather_planes(planes, host_cache, gpu_ids, cpu_ids) -> None:
    """The same for engines that keep one tensor per (layer, K-or-V) with the block
    axis first (SGLang pages, MLA latent blocks): ``planes[l][kv]`` is
    ``[N, ...]``, ``host_cache`` is ``[NH, L, kv, ...]``;
    host_cache[cpu_ids, l, kv] = planes[l][kv][gpu_ids]."""
    import torch
    for l, kvs in enumerate(planes):
        for kv, plane in enumerate(kvs):
            host_cache[:, l, kv].index_copy_(0, cpu_ids, torch.index_select(plane, 0, gpu_ids))


def torch_index_scatter_planes(planes, host_cache, gpu_ids, cpu_ids) -> None:
    """Inverse of torch_index_gather_planes."""
    import torch
    for l, kvs in enumerate(planes):
        for kv, plane in enumerate(kvs):
            plane.index_copy_(0, gpu_ids, torch.index_select(host_cache[:, l, kv], 0, cpu_ids))


# ---- layerwise restore of heterogeneous layer groups ---------------------------

class GroupRef:
    """Host-memory stand-in of one layer group: ``tensors[d]`` are the numpy byte
    buffers that play the group's device tensors on GPU d (GroupParams,
    csrc/layerwise.h)."""

    def __init__(self, num_layers: int, tensors: List[List[np.ndarray]], gpu_kv_strides,
                 gpu_block_strides, gpu_layer_strides, gpu_chunk_sizes, cpu_offset_bytes=0,
                 h2d_cpu_kv_stride=0, h2d_cpu_layer_stride=0, cpu_block_stride=0,
                 cpu_tp_stride=0) -> None:
        self.num_layers = num_layers
        self.tensors = tensors
        n = len(tensors[0])
        # csrc/layerwise.cpp:792-806
        self.backend = (BACKEND_TRTLLM if n == 1 else BACKEND_VLLM if n == num_layers
                        else BACKEND_SGLANG if n == 2 * num_layers else None)
        if self.backend is None:
            raise RuntimeError(f"unsupported tensors_per_gpu={n} for num_layers={num_layers}")
        self.gpu_kv_strides = list(gpu_kv_strides)
        self.gpu_block_strides = list(gpu_block_strides)
        self.gpu_layer_strides = list(gpu_layer_strides)
        self.gpu_chunk_sizes = list(gpu_chunk_sizes)
        self.cpu_offset_bytes = cpu_offset_bytes
        self.h2d_cpu_kv_stride = h2d_cpu_kv_stride
        self.h2d_cpu_layer_stride = h2d_cpu_layer_stride
        self.cpu_block_stride = cpu_block_stride
        self.cpu_tp_stride = cpu_tp_stride


def _group_layer_h2d(g: GroupRef, d: int, host: np.ndarray, local_layer: int, num_layers: int,
                     gpu_ids, cpu_ids, kv_dim: int, cpu_kv_stride: int, cpu_layer_stride: int,
                     cpu_block_stride: int, cpu_off: int) -> None:
    transfer_c(g.backend, [t.ctypes.data for t in g.tensors[d]], g.num_layers,
               g.gpu_kv_strides[d], g.gpu_block_strides[d], g.gpu_layer_strides[d], 0,
               host.ctypes.data + g.cpu_offset_bytes, cpu_kv_stride, cpu_layer_stride,
               cpu_block_stride, cpu_off, g.gpu_chunk_sizes[d], local_layer, num_layers, kv_dim,
               gpu_ids, cpu_ids, True)


def _rank_off(d: int, num_kv_heads: int, mode: str, num_blocks: int, tp_stride: int,
              block_stride: int) -> int:
    # csrc/layerwise.cpp:1519-1526 (same rule at :448-453 and :1143-1166)
    if num_kv_heads == 1:
        return d * num_blocks * block_stride if mode == "all_write" else 0
    return d * tp_stride


def layerwise_multi_group(num_gpus: int, groups: List[GroupRef], layer_members, host: np.ndarray,
                          gpu_ids, cpu_ids, kv_dim: int, num_kv_heads: int,
                          mode: str = "sharded", swa: Optional[dict] = None):
    """layerwise_transfer_multi_group, csrc/layerwise.cpp:1313-1682, on host
    memory.  ``swa`` is None, ``{"kind": "uniform", "group", "host", "gpu_ids",
    "cpu_ids", "kv_stride", "layer_stride", "block_stride"}`` (launch_swa_h2d_layer_,
    :209-258) or ``{"kind": "multi", "groups", "members", "host", "gpu_ids",
    "cpu_ids"}`` (launch_swa_mg_h2d_layer_, :442-503).

    Returns ``(immediate, work)``: the original layers announced on entry because
    nothing is attached to them, and those announced once after their copies, in
    order."""
    if num_kv_heads == 1 and mode not in ("sharded", "all_write", "rank0_only"):
        mode = "sharded"  # :1349-1360
    swa_active = swa is not None and len(swa["cpu_ids"]) > 0
    immediate, work = [], []
    for orig, members in enumerate(layer_members):
        slots = 0
        if swa_active:
            slots = len(swa["members"][orig]) if swa["kind"] == "multi" else 1
        if not members and slots == 0:
            immediate.append(orig)  # :1437-1457
            continue
        work.append(orig)
        for gi, local in members:
            g = groups[gi]
            for d in range(num_gpus):
                off = _rank_off(d, num_kv_heads, mode, len(gpu_ids), g.cpu_tp_stride,
                                g.cpu_block_stride)
                _group_layer_h2d(g, d, host, local, 1, gpu_ids, cpu_ids, kv_dim,
                                 g.h2d_cpu_kv_stride, g.h2d_cpu_layer_stride,
                                 g.cpu_block_stride, off)
        if not swa_active:
            continue
        if swa["kind"] == "multi":
            for gi, local in swa["members"][orig]:
                g = swa["groups"][gi]
                for d in range(num_gpus):
                    off = _rank_off(d, 1, mode, len(swa["gpu_ids"]), g.cpu_tp_stride,
                                    g.cpu_block_stride)
                    _group_layer_h2d(g, d, swa["host"], local, 1, swa["gpu_ids"],
                                     swa["cpu_ids"], 1, g.h2d_cpu_kv_stride,
                                     g.h2d_cpu_layer_stride, g.cpu_block_stride, off)
        else:
            g = swa["group"]
            for d in range(num_gpus):
                _group_layer_h2d(g, d, swa["host"], orig, 1, swa["gpu_ids"], swa["cpu_ids"], 1,
                                 swa["kv_stride"], swa["layer_stride"], swa["block_stride"], 0)
    return immediate, work


# ---- host pool <-> SSD files -----------------------------------------------------

def ssd_locate(ssd_block_id: int, round_robin: int, num_devices: int, files_per_device: int):
    d, f, b = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64()
    lib().fkv_oracle_ssd_locate(ssd_block_id, round_robin, num_devices, files_per_device,
                                ctypes.byref(d), ctypes.byref(f), ctypes.byref(b))
    return d.value, f.value, b.value


def ssd_transfer(files: List[np.ndarray], num_devices: int, files_per_device: int,
                 start_layer: int, num_layers: int, host: np.ndarray, ssd_ids, cpu_ids,
                 cpu_layer_stride: int, cpu_kv_stride: int, ssd_layer_stride: int,
                 ssd_kv_stride: int, chunk: int, block_stride: int, is_read: bool,
                 round_robin: int = 1, kv_dim: int = 2) -> None:
    """``files[device * files_per_device + file]``: equally long uint8 arrays."""
    s, c = _i64(ssd_ids), _i64(cpu_ids)
    ptrs = (ctypes.c_void_p * len(files))(*[f.ctypes.data for f in files])
    rc = lib().fkv_oracle_ssd_transfer(
        ptrs, int(files[0].size), num_devices, files_per_device, start_layer, num_layers,
        host.ctypes.data, _ptr(s), _ptr(c), int(s.size), cpu_layer_stride, cpu_kv_stride,
        ssd_layer_stride, ssd_kv_stride, chunk, block_stride, int(bool(is_read)), round_robin,
        kv_dim)
    if rc != 0:
        raise ValueError("oracle ssd transfer: a chunk lies outside its file")
