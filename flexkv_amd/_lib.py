"""ctypes binding of libfkv_hip.so (the C ABI in include/fkv_transfer.h).

The library must have been built (``make -C flexkv_amd/csrc`` or
``python -c "import __graft_entry__ as g; g.build()"``).  There is no fallback:
if the shared object is missing or cannot be loaded the import of the package's
operator module fails.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_double, c_float, c_int32, c_int64,
                    c_size_t, c_uint32, c_uint64, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfkv_hip.so")

FKV_OK = 0
FKV_ERR_INVALID_ARG = 1
FKV_ERR_RUNTIME = 2
FKV_ERR_UNSUPPORTED = 3

FKV_PATH_KERNEL = 100
CE_PATH_NAMES = {-1: "PER_BLOCK", 0: "CONTIG_DIRECT", 1: "SEGMENT_DIRECT",
                 2: "SEGMENT_SCATTER", 3: "GATHER_SCATTER", 4: "GATHER_DIRECT",
                 FKV_PATH_KERNEL: "KERNEL"}

NOTIFY_HOSTFUNC = 0
NOTIFY_POLLING = 1


class CEConfig(Structure):
    _fields_ = [("segment_threshold", c_int64), ("path_opt_enabled", c_int32),
                ("force_path", c_int32), ("enable_memcpy2d", c_int32),
                ("is_blockfirst", c_int32), ("num_kv_heads", c_int32),
                ("gather_threads", c_int32), ("gather_nt", c_int32), ("reserved", c_int32)]


class TransferDesc(Structure):
    _fields_ = [("backend", c_int32), ("num_layers_total", c_int32),
                ("gpu_tensor_ptrs", c_void_p), ("num_gpu_tensor_ptrs", c_int32),
                ("device", c_int32),
                ("gpu_kv_stride", c_int64), ("gpu_block_stride", c_int64),
                ("gpu_layer_stride", c_int64), ("gpu_startoff_inside_chunks", c_int64),
                ("cpu_ptr", c_void_p),
                ("cpu_kv_stride", c_int64), ("cpu_layer_stride", c_int64),
                ("cpu_block_stride", c_int64), ("cpu_startoff_inside_chunks", c_int64),
                ("chunk_size", c_int64),
                ("start_layer_id", c_int32), ("num_layers", c_int32),
                ("kv_dim", c_int32), ("num_blocks", c_int32),
                ("gpu_block_ids", c_void_p), ("cpu_block_ids", c_void_p),
                ("is_host_to_device", c_int32), ("use_ce_transfer", c_int32),
                ("transfer_num_cta", c_int32), ("sync", c_int32),
                ("enable_trace", c_int32), ("reserved", c_int32),
                ("ce", CEConfig)]


class LayoutTransformDesc(Structure):
    _fields_ = [("backend", c_int32), ("num_layers_total", c_int32),
                ("gpu_tensor_ptrs", c_void_p), ("num_gpu_tensor_ptrs", c_int32),
                ("device", c_int32),
                ("gpu_kv_stride", c_int64), ("gpu_block_stride", c_int64),
                ("gpu_layer_stride", c_int64),
                ("buffer_ptr", c_void_p),
                ("buffer_layer_stride", c_int64), ("buffer_kv_stride", c_int64),
                ("buffer_block_stride", c_int64), ("chunk_size", c_int64),
                ("start_layer_id", c_int32), ("num_layers", c_int32),
                ("kv_dim", c_int32), ("num_blocks", c_int32),
                ("gpu_block_ids", c_void_p),
                ("buffer_to_target", c_int32), ("sync", c_int32)]


class CEAnalysis(Structure):
    _fields_ = [("gpu_log_contig", c_int32), ("cpu_log_contig", c_int32),
                ("cpu_phys_contig", c_int32), ("gpu_phys_contig", c_int32),
                ("num_segments", c_int32), ("reserved", c_int32)]


class CESegment(Structure):
    _fields_ = [("start_k", c_int32), ("nr_blocks", c_int32)]


class TPRankPlan(Structure):
    _fields_ = [("active", c_int32), ("start_layer", c_int32), ("num_layers", c_int32),
                ("reserved", c_int32), ("cpu_startoff", c_int64), ("gpu_startoff", c_int64),
                ("chunk_size", c_int64)]


class TPGroupParams(Structure):
    _fields_ = [("num_gpus", c_int32), ("num_tensors_per_gpu", c_int32),
                ("gpu_block_ptrs_flat", c_void_p), ("cpu_blocks_ptr", c_void_p),
                ("num_layers", c_int32), ("reserved", c_int32),
                ("gpu_kv_strides", c_void_p), ("gpu_block_strides", c_void_p),
                ("gpu_layer_strides", c_void_p), ("gpu_chunk_sizes", c_void_p),
                ("gpu_device_ids", c_void_p), ("ce", CEConfig)]


class LayerwiseParams(Structure):
    _fields_ = [("num_gpus", c_int32), ("num_tensors_per_gpu", c_int32),
                ("gpu_block_ptrs_flat", c_void_p), ("cpu_blocks_ptr", c_void_p),
                ("num_layers", c_int32), ("tp_size", c_int32),
                ("gpu_kv_strides", c_void_p), ("gpu_block_strides", c_void_p),
                ("gpu_layer_strides", c_void_p), ("gpu_chunk_sizes", c_void_p),
                ("gpu_device_ids", c_void_p), ("layer_eventfds", c_void_p),
                ("num_layer_eventfds", c_int32), ("reserved", c_int32), ("ce", CEConfig)]


class LayerGroup(Structure):
    _fields_ = [("num_layers", c_int32), ("num_tensors_per_gpu", c_int32),
                ("gpu_block_ptrs_flat", c_void_p), ("cpu_offset_bytes", c_int64),
                ("h2d_cpu_kv_stride", c_int64), ("h2d_cpu_layer_stride", c_int64),
                ("cpu_block_stride", c_int64), ("cpu_tp_stride", c_int64),
                ("gpu_kv_strides", c_void_p), ("gpu_block_strides", c_void_p),
                ("gpu_layer_strides", c_void_p), ("gpu_chunk_sizes", c_void_p)]


class LayerMember(Structure):
    _fields_ = [("group", c_int32), ("local_layer", c_int32)]


class LayerwiseMGParams(Structure):
    _fields_ = [("num_gpus", c_int32), ("num_original_layers", c_int32),
                ("tp_size", c_int32), ("num_groups", c_int32),
                ("groups", POINTER(LayerGroup)), ("member_offsets", c_void_p),
                ("members", POINTER(LayerMember)), ("cpu_blocks_ptr", c_void_p),
                ("gpu_device_ids", c_void_p), ("layer_eventfds", c_void_p),
                ("num_layer_eventfds", c_int32), ("reserved", c_int32), ("ce", CEConfig)]


class LayerwiseCall(Structure):
    _fields_ = [("gpu_block_ids", c_void_p), ("cpu_block_ids", c_void_p),
                ("num_blocks", c_int32), ("multi_group", c_int32),
                ("cpu_block_stride", c_int64), ("h2d_cpu_kv_stride", c_int64),
                ("h2d_cpu_layer_stride", c_int64), ("cpu_tp_stride", c_int64),
                ("num_layers", c_int32), ("layer_granularity", c_int32),
                ("transfer_cta_num", c_int32), ("use_ce_transfer", c_int32),
                ("kv_dim", c_int32), ("num_kv_heads", c_int32),
                ("counter_id", c_int32), ("notify_mode", c_int32),
                ("enable_trace", c_int32), ("swa_num_blocks", c_int32),
                ("kv_shared_across_ranks_mode", c_char_p),
                ("swa_gpu_block_ids", c_void_p), ("swa_cpu_block_ids", c_void_p),
                ("swa_h2d_cpu_kv_stride", c_int64), ("swa_h2d_cpu_layer_stride", c_int64),
                ("swa_cpu_block_stride", c_int64)]


class StagingTransferDesc(Structure):
    _fields_ = [("staging", c_void_p), ("staging_stride", c_int64), ("comp_sizes", c_void_p),
                ("cpu_ptr", c_void_p), ("chunk_capacity", c_int64), ("overflow", c_void_p),
                ("cpu_kv_stride", c_int64), ("cpu_layer_stride", c_int64),
                ("cpu_block_stride", c_int64), ("cpu_block_ids", c_void_p),
                ("size_table", c_void_p), ("size_table_block_stride", c_int64),
                ("size_table_layer_stride", c_int64),
                ("start_layer_id", c_int32), ("kv_dim", c_int32), ("num_blocks", c_int32),
                ("batch_start", c_int32), ("bsz", c_int32), ("is_write_cpu", c_int32),
                ("transfer_num_cta", c_int32), ("device", c_int32), ("sync", c_int32)]


class ChunkPtrsDesc(Structure):
    _fields_ = [("out_ptrs", c_void_p), ("backend", c_int32), ("num_layers_total", c_int32),
                ("gpu_tensor_ptrs", c_void_p), ("num_gpu_tensor_ptrs", c_int32),
                ("device", c_int32),
                ("gpu_kv_stride", c_int64), ("gpu_block_stride", c_int64),
                ("gpu_layer_stride", c_int64), ("gpu_block_ids", c_void_p),
                ("start_layer_id", c_int32), ("kv_dim", c_int32), ("num_blocks", c_int32),
                ("batch_start", c_int32), ("bsz", c_int32), ("sync", c_int32)]


class StagedRun(Structure):
    _fields_ = [("first_id", c_int64), ("rows", c_int32), ("row0", c_int32)]


class Stats(Structure):
    _fields_ = [("calls", c_uint64), ("bytes_h2d", c_uint64), ("bytes_d2h", c_uint64),
                ("kernel_launches", c_uint64), ("dma_copies", c_uint64),
                ("staging_bytes_device", c_uint64), ("staging_bytes_host", c_uint64),
                ("confined_launches", c_uint64), ("safety_net_ranges", c_uint64),
                ("staged_batches", c_uint64), ("gathered_batches", c_uint64),
                ("gather_busy_us", c_uint64), ("second_stream_batches", c_uint64),
                ("plan_slots", c_uint64), ("plan_slots_in_use", c_uint64),
                ("plan_slot_waits", c_uint64)]


class LaunchPolicy(Structure):
    """fkv_launch_policy: every tunable of the kernel path, per device."""
    _fields_ = [("xcd_count", c_int32), ("xcd_present_mask", c_uint32),
                ("arbiter", c_int32),
                ("d2h_busy_mask", c_uint32), ("h2d_busy_mask", c_uint32),
                ("d2h_home_mask", c_uint32), ("h2d_home_mask", c_uint32),
                ("busy_window_ms", c_int32), ("home_min_kb", c_int32),
                ("d2h_busy_pct", c_int32), ("h2d_busy_pct", c_int32),
                ("busy_claims_per_wg", c_int32), ("home_claims_per_wg", c_int32),
                ("all_claims_per_wg", c_int32), ("safety_net_wait_us", c_int32),
                ("link_gbps_estimate", c_int32),
                ("d2h_wg_per_cta", c_int32), ("h2d_wg_per_cta", c_int32),
                ("d2h_wg_threads", c_int32), ("h2d_wg_threads", c_int32),
                ("packed_grid_pct", c_int32), ("plan_mirror", c_int32),
                ("fuse_launches", c_int32), ("lane_streams", c_int32),
                ("staged_restore", c_int32), ("staged_ring", c_int32),
                ("staged_copy_overhead_us", c_int32), ("staged_overhead_pct", c_int32),
                ("staged_bridge_kb", c_int32), ("staged_max_mb", c_int32),
                ("hbm_workgroups", c_int32), ("hbm_wg_threads", c_int32), ("hbm_unroll", c_int32),
                ("ce_staging_mb", c_int32), ("ce_two_streams", c_int32),
                ("ce_rect_min_kb", c_int32),
                ("model_link_mbps", c_int32), ("model_kernel_d2h_mbps", c_int32),
                ("model_kernel_h2d_mbps", c_int32), ("model_dma_ns", c_int32),
                ("model_compaction_gbps", c_int32), ("model_host_pass_mbps", c_int32),
                ("model_launch_ns", c_int32), ("model_prefer_ce_pct", c_int32),
                ("d2h_lane_runs", c_int32),
                ("staged_gather", c_int32), ("gather_threads", c_int32), ("gather_ring", c_int32),
                ("gather_first_by_kernel", c_int32), ("model_gather_thread_mbps", c_int32),
                ("model_seed", c_int32), ("model_seeded", c_int32),
                ("staged_scatter_threads", c_int32), ("test_fail_restore_batch", c_int32),
                ("staged_dma_streams", c_int32), ("kernel_alt_stream_kb", c_int32),
                ("quiet_wait_us", c_int32)]


# name -> (restype, argtypes); the complete export list of include/fkv_transfer.h
SIGNATURES = {
    "fkv_abi_version": (c_int32, []),
    "fkv_last_error": (c_char_p, []),
    "fkv_last_path": (c_int32, []),
    "fkv_ce_config_default": (None, [POINTER(CEConfig)]),
    "fkv_transfer_kv_blocks": (c_int32, [POINTER(TransferDesc), c_void_p]),
    "fkv_transfer_kv_blocks_noalloc": (c_int32, [POINTER(TransferDesc), c_void_p]),
    "fkv_transfer_kv_blocks_multi": (c_int32, [POINTER(TransferDesc), c_int32, c_void_p]),
    "fkv_choose_engine": (c_int32, [POINTER(TransferDesc), POINTER(c_int32), POINTER(c_double),
                                    POINTER(c_double)]),
    "fkv_ce_analyze": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int64,
                                 POINTER(CEAnalysis), c_void_p, c_int32]),
    "fkv_ce_choose_path": (c_int32, [POINTER(CEAnalysis), POINTER(CEConfig), c_int64,
                                     c_int32, c_int32]),
    "fkv_tp_rank_plan_compute": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_char_p,
                                           c_int32, c_int32, c_int32, c_int32, c_int32,
                                           c_int64, c_int64, c_int64, POINTER(TPRankPlan)]),
    "fkv_tp_group_create": (c_int32, [POINTER(TPGroupParams), POINTER(c_void_p)]),
    "fkv_tp_group_update_gpu_block_ptrs": (c_int32, [c_void_p, c_void_p, c_int64]),
    "fkv_tp_group_transfer": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32,
                                        c_int64, c_int64, c_int64, c_int64,
                                        c_int32, c_int32, c_int32, c_int32, c_int32,
                                        c_int32, c_int32, c_char_p, c_int32]),
    "fkv_tp_group_destroy": (None, [c_void_p]),
    "fkv_launch_policy_seed": (c_int32, [c_int32]),
    "fkv_launch_policy_seeded": (c_int32, [POINTER(LaunchPolicy), c_double, c_double, c_double,
                                           POINTER(LaunchPolicy)]),
    "fkv_layerwise_create": (c_int32, [POINTER(LayerwiseParams), POINTER(c_void_p)]),
    "fkv_layerwise_create_multi_group": (c_int32, [POINTER(LayerwiseMGParams),
                                                   POINTER(c_void_p)]),
    "fkv_layerwise_init_swa": (c_int32, [c_void_p, POINTER(LayerGroup), c_void_p]),
    "fkv_layerwise_init_swa_multi_group": (c_int32, [c_void_p, POINTER(LayerGroup), c_int32,
                                                     c_void_p, POINTER(LayerMember),
                                                     c_void_p]),
    "fkv_layerwise_transfer_call": (c_int32, [c_void_p, POINTER(LayerwiseCall)]),
    "fkv_layerwise_transfer": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32,
                                         c_int64, c_int64, c_int64, c_int64,
                                         c_int32, c_int32, c_int32, c_int32, c_int32,
                                         c_int32, c_int32, c_char_p, c_int32, c_int32]),
    "fkv_layerwise_wait_layer": (c_int32, [c_void_p, c_int32, c_int32, c_void_p]),
    "fkv_layerwise_set_compute_stream": (c_int32, [c_void_p, c_int32, c_void_p, POINTER(c_int32)]),
    "fkv_layerwise_synchronize": (c_int32, [c_void_p]),
    "fkv_layerwise_batch_times_ms": (c_int32, [c_void_p, POINTER(c_float), c_int32,
                                               POINTER(c_int32)]),
    "fkv_layerwise_destroy": (None, [c_void_p]),
    "fkv_host_alloc": (c_int32, [c_size_t, POINTER(c_void_p)]),
    "fkv_host_free": (c_int32, [c_void_p]),
    "fkv_host_register": (c_int32, [c_void_p, c_size_t, c_size_t]),
    "fkv_host_unregister": (c_int32, [c_void_p, c_size_t, c_size_t]),
    "fkv_host_register_plan": (c_int64, [c_size_t, c_size_t, c_void_p, c_void_p, c_int64]),
    "fkv_host_chunk_bytes_from_gb": (c_size_t, [c_double]),
    "fkv_ssd_open": (c_int32, [POINTER(c_char_p), c_int32, c_int32, c_int32, c_int32,
                               POINTER(c_void_p)]),
    "fkv_ssd_close": (None, [c_void_p]),
    "fkv_layout_transform": (c_int32, [POINTER(LayoutTransformDesc), c_void_p]),
    "fkv_streams_run_concurrently": (c_int32, [c_int32, c_void_p, c_void_p, POINTER(c_int32)]),
    "fkv_streams_hand_over_us": (c_int32, [c_int32, c_void_p, c_void_p, POINTER(ctypes.c_double)]),
    "fkv_link_activity_post": (c_int32, [c_int32, c_int32, c_int64]),
    "fkv_link_activity_elsewhere": (c_int32, [c_int32, c_int32, c_int32, POINTER(c_int32)]),
    "fkv_range_push": (c_int32, [c_char_p]),
    "fkv_range_pop": (c_int32, []),
    "fkv_ssd_uses_iouring": (c_int32, [c_void_p]),
    "fkv_ssd_last_direct": (c_int32, [c_void_p]),
    "fkv_ssd_transfer": (c_int32, [c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
                                   c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_int32, c_int32, c_int32, c_int32, c_int32]),
    "fkv_ssd_locate": (c_int32, [c_int64, c_int32, c_int32, c_int32, POINTER(c_int32),
                                 POINTER(c_int32), POINTER(c_int64)]),
    "fkv_ssd_plan": (c_int64, [c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_int32,
                               c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int32,
                               c_int32, c_int32, c_void_p, c_int64]),
    "fkv_ipc_export": (c_int32, [c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64)]),
    "fkv_ipc_open": (c_int32, [c_void_p, c_int32, POINTER(c_void_p)]),
    "fkv_ipc_close": (c_int32, [c_void_p]),
    "fkv_get_stats": (None, [POINTER(Stats)]),
    "fkv_reset_stats": (None, []),
    "fkv_staging_transfer": (c_int32, [POINTER(StagingTransferDesc), c_void_p]),
    "fkv_build_gpu_chunk_ptrs": (c_int32, [POINTER(ChunkPtrsDesc), c_void_p]),
    "fkv_staged_restore_plan": (c_int32, [c_void_p, c_int32, c_int64, c_int32,
                                          POINTER(LaunchPolicy), POINTER(c_int32),
                                          POINTER(c_int32), POINTER(c_int64), c_void_p, c_int32,
                                          c_void_p]),
    "fkv_measure_hbm_rate": (c_int32, [c_int32, c_size_t, c_int32, c_int32,
                                       POINTER(c_double), POINTER(c_double)]),
    "fkv_launch_policy_get": (c_int32, [c_int32, POINTER(LaunchPolicy)]),
    "fkv_launch_policy_set": (c_int32, [c_int32, POINTER(LaunchPolicy)]),
    "fkv_launch_policy_reset": (c_int32, [c_int32]),
    "fkv_measure_link_peak": (c_int32, [c_int32, c_size_t, c_int32, c_int32,
                                        POINTER(c_double), POINTER(c_double)]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load libfkv_hip.so and attach the prototypes.  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build the HIP library first "
            "(make -C flexkv_amd/csrc); there is no CPU fallback for the transfer path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.fkv_abi_version() != 5:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.fkv_abi_version()} != 5")
    _lib = lib
    return lib


def last_error() -> str:
    return (load().fkv_last_error() or b"").decode(errors="replace")


def check(status: int) -> None:
    """Map a status code to the exception class the reference's pybind module
    would have raised (std::invalid_argument -> ValueError, everything else ->
    RuntimeError)."""
    if status == FKV_OK:
        return
    msg = last_error()
    if status == FKV_ERR_INVALID_ARG:
        raise ValueError(msg)
    raise RuntimeError(msg)


def default_ce_config() -> CEConfig:
    cfg = CEConfig()
    load().fkv_ce_config_default(ctypes.byref(cfg))
    return cfg
