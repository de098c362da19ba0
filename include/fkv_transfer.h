/*
 * fkv_transfer.h — C ABI of libfkv_hip.so: GPU<->CPU KV-cache block transfer for
 * AMD Instinct MI355X (gfx950).
 *
 * Every entry point is `extern "C"`, takes plain pointers / integers only and
 * returns an int status (FKV_OK == 0).  On failure the text of the error is kept
 * per calling thread and returned by fkv_last_error().  No C++ exception and no
 * torch type crosses this boundary.
 *
 * The functions replace, one for one, the hot-path part of FlexKV's pybind
 * module `flexkv.c_ext`.  Each declaration cites the reference interface it
 * stands in for (paths relative to the FlexKV source tree).
 *
 * Conventions
 *   - all strides, offsets and sizes are BYTES (the reference converts bytes to
 *     int64 units internally, csrc/transfer.cu:179-187; here bytes are kept);
 *   - a "chunk" is the contiguous byte run of one (layer, k-or-v, block);
 *   - `gpu_tensor_ptrs` is a HOST array of device addresses (the reference
 *     keeps the same table in pinned memory and lets the kernel dereference it,
 *     csrc/gtensor_handler.cuh:47; here the host resolves it per call);
 *   - block-id arrays are HOST arrays of int64 and need not be pinned: they are
 *     copied into library-owned, device-visible plan memory before the call
 *     returns, so the caller may free them immediately, also when sync == 0;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 */
#ifndef FKV_TRANSFER_H
#define FKV_TRANSFER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FKV_ABI_VERSION 5 /* 5: fkv_stats grew by plan_slots, plan_slots_in_use and plan_slot_waits, the last reserved slot of fkv_launch_policy became quiet_wait_us; 4: fkv_stats grew by second_stream_batches; 3: fkv_stats grew by gathered_batches and gather_busy_us, fkv_launch_policy by the host-gather and link-seeding fields; 2: fkv_stats grew by staged_batches; launch policy, no-alloc transfer, staging and HBM-rate entry points added */

/* status codes */
#define FKV_OK 0
#define FKV_ERR_INVALID_ARG 1 /* maps to ValueError / std::invalid_argument */
#define FKV_ERR_RUNTIME 2     /* HIP failure or internal error -> RuntimeError */
#define FKV_ERR_UNSUPPORTED 3 /* feature outside this library -> RuntimeError */

/* GPU tensor addressing, csrc/gtensor_handler.cuh:8 (enum BackendType) and
 * csrc/bindings.cpp:85-94 (gpu_block_type 0/1/2). */
#define FKV_BACKEND_VLLM 0   /* one tensor per layer:  ptrs[l] + kv*Ks + b*Bs          */
#define FKV_BACKEND_TRTLLM 1 /* one tensor in all:     ptrs[0] + b*Bs + l*Ls + kv*Ks   */
#define FKV_BACKEND_SGLANG 2 /* K then V per layer:    ptrs[kv*Ltot + l] + b*Bs        */

/* Copy-engine strategies, csrc/ce_transfer.h:42-49 (enum CEPath). */
#define FKV_CE_PER_BLOCK (-1)
#define FKV_CE_CONTIG_DIRECT 0
#define FKV_CE_SEGMENT_DIRECT 1
#define FKV_CE_SEGMENT_SCATTER 2
#define FKV_CE_GATHER_SCATTER 3
#define FKV_CE_GATHER_DIRECT 4
/* value reported by fkv_last_path() when the gather/scatter kernel ran */
#define FKV_PATH_KERNEL 100

/* csrc/ce_transfer.h:18-41 (struct CETransferConfig), same defaults when
 * zero-initialised fields are filled by fkv_ce_config_default(). */
typedef struct fkv_ce_config {
  int64_t segment_threshold; /* 8 */
  int32_t path_opt_enabled;  /* 1: adaptive strategies, 0: PER_BLOCK */
  int32_t force_path;        /* -1 auto, 0..4 force */
  int32_t enable_memcpy2d;   /* 0 */
  int32_t is_blockfirst;     /* host layout is [block, layer, kv, chunk] */
  int32_t num_kv_heads;      /* 1 = KV identical on all TP ranks (MLA) */
  int32_t gather_threads;    /* 4; host scatter/gather worker threads, 0 = caller only */
  int32_t gather_nt;         /* 1; streaming stores in the host scatter/gather */
  int32_t reserved;
} fkv_ce_config;

void fkv_ce_config_default(fkv_ce_config *cfg);

/* One transfer.  Replaces flexkv::transfer_kv_blocks<Type>()
 * (csrc/transfer.cuh:27-37, csrc/transfer.cu:164-313) together with the
 * GTensorHandler it receives (csrc/gtensor_handler.cuh:11-33). */
typedef struct fkv_transfer_desc {
  /* GPU side */
  int32_t backend;              /* FKV_BACKEND_* */
  int32_t num_layers_total;     /* GTensorHandler::num_layers (SGLang ptr index) */
  const uint64_t *gpu_tensor_ptrs; /* host array of device addresses */
  int32_t num_gpu_tensor_ptrs;  /* entries in gpu_tensor_ptrs (bounds check) */
  int32_t device;               /* HIP device ordinal of the GPU tensors, -1 = current */
  int64_t gpu_kv_stride;
  int64_t gpu_block_stride;
  int64_t gpu_layer_stride;
  int64_t gpu_startoff_inside_chunks;
  /* host side */
  void *cpu_ptr;
  int64_t cpu_kv_stride;
  int64_t cpu_layer_stride;
  int64_t cpu_block_stride;
  int64_t cpu_startoff_inside_chunks;
  /* what to move */
  int64_t chunk_size;
  int32_t start_layer_id;
  int32_t num_layers;
  int32_t kv_dim;
  int32_t num_blocks;
  const int64_t *gpu_block_ids; /* host, num_blocks entries */
  const int64_t *cpu_block_ids; /* host, num_blocks entries */
  /* how */
  int32_t is_host_to_device;
  int32_t use_ce_transfer;  /* 0 kernel, 1 copy engine, 2 pick per transfer (fkv_choose_engine) */
  int32_t transfer_num_cta; /* CTAs as the reference counts them; each becomes 4 (host->GPU)
                               or 12 (GPU->host) single-wavefront workgroups;
                               <= 0 = library default (4) */
  int32_t sync;             /* 1: return when the transfer (and what `stream` held before it)
                               has finished; where the reference calls cudaStreamSynchronize */
  int32_t enable_trace;     /* 1: print an "[XFER]" line per call to stderr */
  int32_t reserved;
  fkv_ce_config ce;
} fkv_transfer_desc;

/* csrc/bindings.cpp:54-151, 439-459 (`c_ext.transfer_kv_blocks`) and every
 * internal call of flexkv::transfer_kv_blocks<Type>.  The transfer is ordered
 * after the work `stream` holds at the call; with sync == 0, work queued on
 * `stream` afterwards is ordered after the transfer.  The kernels themselves may
 * run on a stream of the library when synchronous calls come in on more than two
 * streams (FKV_LANE_STREAMS=0: never, =1: always); the block-id arrays may be
 * reused as soon as the call returns. */
int fkv_transfer_kv_blocks(const fkv_transfer_desc *desc, void *stream);

/* The same for `count` descriptors of one direction and device at once, as the
 * reference's worker issues them one after the other for the layer groups of a
 * multi-group model (flexkv/transfer/worker.py:998-1015): one call per group with
 * the group's tensors, strides and chunk size.  Equivalent to `count` calls in
 * order; `sync` and `enable_trace` of the last descriptor apply to the whole.  On
 * the kernel path up to four of them share one launch. */
int fkv_transfer_kv_blocks_multi(const fkv_transfer_desc *descs, int32_t count, void *stream);

/* The kernel path of fkv_transfer_kv_blocks without any allocation.  No counterpart
 * in the reference; it is for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The plan
 * of the launch (base tables, block-id lists) and the claim counters live in a fixed
 * array in device memory that belongs to the library's code object (one copy per GPU,
 * held until the process ends) instead of memory allocated on demand; the call makes
 * no hipMalloc / hipHostMalloc / hipFree, creates no streams or events, copies nothing
 * with hipMemcpy and keeps no stream handle.  All it enqueues on `stream` is kernel
 * launches (the plan travels in the arguments of small fill kernels), so a stream
 * capture can record it; a replay moves the bytes that the tensors hold at that time.
 *   - same descriptor, same bytes moved as fkv_transfer_kv_blocks on the kernel path;
 *     use_ce_transfer must be 0 (FKV_ERR_UNSUPPORTED otherwise);
 *   - limit: 16 * num_blocks + 16 * num_layers * kv_dim <= FKV_NOALLOC_MAX_PLAN_BYTES and
 *     num_layers <= 1024 (FKV_ERR_INVALID_ARG beyond; split the call);
 *   - block-id arrays in pinned, registered or device memory are read in place by the
 *     kernel, as the reference's kernel reads its id tensors (csrc/transfer.cu:121-122):
 *     keep them unchanged until the transfer has run (a recorded graph reads them anew
 *     at every replay); id arrays in pageable memory are copied into the launches and
 *     may be reused as soon as the call returns;
 *   - all calls on one GPU share the array: calls on one stream are ordered by the
 *     stream; calls that are in flight at the same time on different streams of one GPU
 *     race for it and must be ordered by the caller; the call itself waits for nothing;
 *   - desc->sync waits with hipStreamSynchronize (leave it 0 under capture); the launches
 *     are not confined by the link arbiter of fkv_transfer_kv_blocks until that call has
 *     set up the device, and a recorded launch keeps the shape it was recorded with. */
#define FKV_NOALLOC_MAX_PLAN_BYTES (1u << 20)
int fkv_transfer_kv_blocks_noalloc(const fkv_transfer_desc *desc, void *stream);

/* Which path `use_ce_transfer == 2` would take for this descriptor, from a cost
 * model of both (DMA commands, staging passes, link time); pure host function.
 * The reference fixes the engine per direction by configuration
 * (FLEXKV_USE_CE_TRANSFER_{H2D,D2H}, flexkv/common/config.py:775-778) and has
 * no per-transfer choice.  Estimates are milliseconds; either may be NULL. */
int fkv_choose_engine(const fkv_transfer_desc *desc, int32_t *use_ce, double *est_kernel_ms,
                      double *est_ce_ms);

/* Thread-local text of the last failure on this thread ("" if none).
 * Stands in for the C++ exceptions of csrc/bindings.cpp:91-94, 147-150. */
const char *fkv_last_error(void);
int fkv_abi_version(void);

/* Path taken by the last fkv_transfer_kv_blocks on this thread:
 * FKV_PATH_KERNEL or one of FKV_CE_*.  The reference cannot report this
 * (tests/test_kv_transfer_correctness.py:1697-1705 wishes it could). */
int fkv_last_path(void);

/* ---- copy-engine analysis (pure host functions, usable without a GPU) ---- */

/* csrc/ce_transfer.h:53-65 */
typedef struct fkv_ce_segment {
  int32_t start_k;
  int32_t nr_blocks;
} fkv_ce_segment;

typedef struct fkv_ce_analysis {
  int32_t gpu_log_contig;
  int32_t cpu_log_contig;
  int32_t cpu_phys_contig;
  int32_t gpu_phys_contig;
  int32_t num_segments;
  int32_t reserved;
} fkv_ce_analysis;

/* csrc/ce_transfer.cu:37-66 (analyze_ce_transfer).  `segments` may be NULL;
 * otherwise at most `segment_capacity` entries are written.  */
int fkv_ce_analyze(const int64_t *gpu_block_ids, const int64_t *cpu_block_ids,
                   int32_t num_blocks, int64_t cpu_block_stride,
                   int64_t chunk_size, int64_t gpu_block_stride,
                   fkv_ce_analysis *out, fkv_ce_segment *segments,
                   int32_t segment_capacity);

/* csrc/ce_transfer.cu:71-104 (choose_path).  Returns an FKV_CE_* value. */
int fkv_ce_choose_path(const fkv_ce_analysis *analysis, const fkv_ce_config *cfg,
                       int64_t chunk_size, int32_t is_host_to_device,
                       int32_t is_full_block);

/* ---- per-rank placement for tensor-parallel groups (pure host function) ---- */

typedef struct fkv_tp_rank_plan {
  int32_t active;          /* 0: this rank moves nothing in this call */
  int32_t start_layer;
  int32_t num_layers;
  int32_t reserved;
  int64_t cpu_startoff;
  int64_t gpu_startoff;
  int64_t chunk_size;
} fkv_tp_rank_plan;

/* csrc/tp_transfer_thread_group.cpp:222-323 (offset / layer-range rules of
 * tp_group_transfer).  `mode` is the kv_shared_across_ranks_mode string;
 * `rotate_counter` is the value of the round-robin counter for rank_rotate.
 * Returns FKV_ERR_RUNTIME for the sharded/indivisible case (:237-247 throws
 * std::runtime_error). */
int fkv_tp_rank_plan_compute(int32_t rank, int32_t num_gpus, int32_t num_kv_heads,
                             int32_t is_host_to_device, const char *mode,
                             int32_t designated_rank, int32_t rotate_counter,
                             int32_t layer_id, int32_t layer_granularity,
                             int32_t num_blocks, int64_t gpu_chunk_size,
                             int64_t cpu_block_stride, int64_t cpu_tp_stride,
                             fkv_tp_rank_plan *out);

/* ---- TPTransferThreadGroup: csrc/tp_transfer_thread_group.h:42-133,
 *      csrc/bindings.cpp:761-830 ---- */

typedef struct fkv_tp_group fkv_tp_group;

typedef struct fkv_tp_group_params {
  int32_t num_gpus;
  int32_t num_tensors_per_gpu;
  const uint64_t *gpu_block_ptrs_flat; /* num_gpus * num_tensors_per_gpu */
  void *cpu_blocks_ptr;
  int32_t num_layers;
  int32_t reserved;
  const int64_t *gpu_kv_strides;    /* num_gpus entries each */
  const int64_t *gpu_block_strides;
  const int64_t *gpu_layer_strides;
  const int64_t *gpu_chunk_sizes;
  const int64_t *gpu_device_ids;
  fkv_ce_config ce;
} fkv_tp_group_params;

/* ctor, csrc/tp_transfer_thread_group.cpp:30-138 */
int fkv_tp_group_create(const fkv_tp_group_params *params, fkv_tp_group **out);
/* csrc/tp_transfer_thread_group.cpp:140-162 */
int fkv_tp_group_update_gpu_block_ptrs(fkv_tp_group *g, const uint64_t *ptrs_flat,
                                       int64_t count);
/* csrc/tp_transfer_thread_group.cpp:199-381 */
int fkv_tp_group_transfer(fkv_tp_group *g, const int64_t *gpu_block_ids,
                          const int64_t *cpu_block_ids, int32_t num_blocks,
                          int64_t cpu_kv_stride, int64_t cpu_layer_stride,
                          int64_t cpu_block_stride, int64_t cpu_tp_stride,
                          int32_t transfer_num_cta, int32_t is_host_to_device,
                          int32_t use_ce_transfer, int32_t layer_id,
                          int32_t layer_granularity, int32_t kv_dim,
                          int32_t num_kv_heads, const char *mode,
                          int32_t designated_rank);
/* dtor, csrc/tp_transfer_thread_group.cpp:164-185 */
void fkv_tp_group_destroy(fkv_tp_group *g);

/* ---- LayerwiseTransferGroup: csrc/layerwise.h:59-362,
 *      csrc/bindings.cpp:471-757 ---- */

typedef struct fkv_layerwise fkv_layerwise;

typedef struct fkv_layerwise_params {
  int32_t num_gpus;
  int32_t num_tensors_per_gpu;
  const uint64_t *gpu_block_ptrs_flat; /* num_gpus * num_tensors_per_gpu */
  void *cpu_blocks_ptr;
  int32_t num_layers;
  int32_t tp_size;
  const int64_t *gpu_kv_strides; /* num_gpus entries each */
  const int64_t *gpu_block_strides;
  const int64_t *gpu_layer_strides;
  const int64_t *gpu_chunk_sizes;
  const int64_t *gpu_device_ids;
  const int32_t *layer_eventfds; /* [num_counters, tp_size, num_layers] or NULL */
  int32_t num_layer_eventfds;    /* total entries, 0 = eventfd notification off */
  int32_t reserved;
  fkv_ce_config ce;
} fkv_layerwise_params;

#define FKV_NOTIFY_HOSTFUNC 0
#define FKV_NOTIFY_POLLING 1

/* Single-group ctor, csrc/layerwise.cpp:507-646.  The SSD files of the
 * reference's ctor are served by fkv_ssd_open / fkv_ssd_transfer, which the
 * caller runs before the restore (the Python operator does); a uniform SWA
 * sidecar is attached afterwards with fkv_layerwise_init_swa. */
int fkv_layerwise_create(const fkv_layerwise_params *params, fkv_layerwise **out);

/* One layer group: layers that share a KV shape, with their own device
 * tensors and their own byte range inside every host block -- GroupParams,
 * csrc/layerwise.h (filled by fill_group_params_from_arrays,
 * csrc/layerwise.cpp:264-353).  The backend follows from
 * num_tensors_per_gpu vs num_layers (1 -> TRT-LLM, L -> vLLM, 2L -> SGLang). */
typedef struct fkv_layer_group {
  int32_t num_layers;
  int32_t num_tensors_per_gpu;
  const uint64_t *gpu_block_ptrs_flat; /* num_gpus * num_tensors_per_gpu */
  int64_t cpu_offset_bytes;            /* of the group inside a host block */
  int64_t h2d_cpu_kv_stride;
  int64_t h2d_cpu_layer_stride;
  int64_t cpu_block_stride;
  int64_t cpu_tp_stride;
  const int64_t *gpu_kv_strides; /* num_gpus entries each */
  const int64_t *gpu_block_strides;
  const int64_t *gpu_layer_strides;
  const int64_t *gpu_chunk_sizes;
} fkv_layer_group;

/* (group, layer inside the group) attached to one original layer --
 * LayerMemberMap, flexkv/common/config.py:68-119. */
typedef struct fkv_layer_member {
  int32_t group;
  int32_t local_layer;
} fkv_layer_member;

typedef struct fkv_layerwise_mg_params {
  int32_t num_gpus;
  int32_t num_original_layers;
  int32_t tp_size;
  int32_t num_groups;
  const fkv_layer_group *groups;
  /* members of original layer i: members[member_offsets[i] .. member_offsets[i+1]) */
  const int32_t *member_offsets; /* num_original_layers + 1 entries */
  const fkv_layer_member *members;
  void *cpu_blocks_ptr;
  const int64_t *gpu_device_ids;
  const int32_t *layer_eventfds; /* [num_counters, tp_size, num_original_layers] */
  int32_t num_layer_eventfds;
  int32_t reserved;
  fkv_ce_config ce;
} fkv_layerwise_mg_params;

/* Multi-group ctor, csrc/layerwise.cpp:647-838. */
int fkv_layerwise_create_multi_group(const fkv_layerwise_mg_params *params,
                                     fkv_layerwise **out);

/* Uniform SWA sidecar (one ring of sliding-window blocks per layer with its own
 * host pool) -- init_swa_sidecar_, csrc/layerwise.cpp:139-207.  Of `swa` the
 * device fields and num_layers are read; the host strides come with each call.
 * Errors: "Unsupported SWA GPU block type: N". */
int fkv_layerwise_init_swa(fkv_layerwise *g, const fkv_layer_group *swa,
                           void *swa_cpu_blocks_ptr);
/* SWA / state sidecar made of its own layer groups --
 * init_swa_multi_group, csrc/layerwise.cpp:355-429. */
int fkv_layerwise_init_swa_multi_group(fkv_layerwise *g, const fkv_layer_group *groups,
                                       int32_t num_groups, const int32_t *member_offsets,
                                       const fkv_layer_member *members,
                                       void *swa_cpu_blocks_ptr);

/* Arguments of one restore: layerwise_transfer (csrc/layerwise.cpp:944-1311)
 * when multi_group == 0, layerwise_transfer_multi_group (:1313-1682) otherwise. */
typedef struct fkv_layerwise_call {
  const int64_t *gpu_block_ids; /* host arrays, num_blocks entries */
  const int64_t *cpu_block_ids;
  int32_t num_blocks;
  int32_t multi_group;
  /* single group only; a multi-group instance takes these from its groups */
  int64_t cpu_block_stride;
  int64_t h2d_cpu_kv_stride;
  int64_t h2d_cpu_layer_stride;
  int64_t cpu_tp_stride;
  int32_t num_layers;
  int32_t layer_granularity;
  int32_t transfer_cta_num;
  int32_t use_ce_transfer;
  int32_t kv_dim;
  int32_t num_kv_heads;
  int32_t counter_id;
  int32_t notify_mode;
  int32_t enable_trace;
  int32_t swa_num_blocks; /* 0 = no sidecar work in this call */
  const char *kv_shared_across_ranks_mode;
  /* sidecar: swa_h2d_dst (device block ids) / swa_h2d_src (host block ids) */
  const int64_t *swa_gpu_block_ids;
  const int64_t *swa_cpu_block_ids;
  /* uniform sidecar only */
  int64_t swa_h2d_cpu_kv_stride;
  int64_t swa_h2d_cpu_layer_stride;
  int64_t swa_cpu_block_stride;
} fkv_layerwise_call;

/* Host->GPU restore, one completion per layer batch (single group: batches of
 * `layer_granularity` layers; multi-group: one batch per original layer that
 * has members or sidecar work, original layers with neither get their eventfd
 * written on entry, csrc/layerwise.cpp:1437-1457).  HOSTFUNC returns after
 * every stream has drained (:1249-1256, 1634-1642), the eventfds of a batch
 * having been written as soon as the batch landed; POLLING returns right after
 * the launches and a library thread writes the eventfds. */
int fkv_layerwise_transfer_call(fkv_layerwise *g, const fkv_layerwise_call *call);

/* layerwise_transfer without sidecar work, positional form of the above. */
int fkv_layerwise_transfer(fkv_layerwise *g, const int64_t *gpu_block_ids,
                           const int64_t *cpu_block_ids, int32_t num_blocks,
                           int64_t cpu_block_stride, int64_t h2d_cpu_kv_stride,
                           int64_t h2d_cpu_layer_stride, int64_t cpu_tp_stride,
                           int32_t transfer_cta_num, int32_t use_ce_transfer,
                           int32_t num_layers, int32_t layer_granularity,
                           int32_t kv_dim, int32_t num_kv_heads, int32_t counter_id,
                           const char *mode, int32_t notify_mode,
                           int32_t enable_trace);

/* Make `consumer_stream` (a hipStream_t on GPU `gpu_index` of the group) wait
 * until `layer` (an original layer id for a multi-group instance) of the most
 * recent transfer has landed.  This is the in-process counterpart of the
 * eventfd a consumer in another process blocks on
 * (flexkv/integration/sglang/comm.py:705-744); the reference has no such call. */
int fkv_layerwise_wait_layer(fkv_layerwise *g, int32_t gpu_index, int32_t layer,
                             void *consumer_stream);
/* Names the stream on which the engine computes next to this group's restores on GPU
 * `gpu_index` (a hipStream_t, or NULL for the null stream).  A process has few hardware
 * queues (4 unless GPU_MAX_HW_QUEUES says otherwise) and the runtime spreads streams over
 * them; two streams on one queue run one after the other.  A restore whose scatter or copy
 * stream shares the queue of the engine's forward pass is therefore not hidden behind the
 * forward pass but added to it (61 layers of 36 MiB next to 0.6 ms of attention per layer:
 * 89 ms instead of 42).  The call swaps every stream the group uses on that GPU for one
 * that was seen to run next to `compute_stream` and to exchange events with it at the normal
 * latency (fkv_streams_run_concurrently and fkv_streams_hand_over_us per pair of streams
 * probed, up to 8 candidates per stream; 100 ms for the whole call on a device with four
 * queues) and, where the queues allow, puts the
 * scatter stream and the two copy streams on queues of their own; `streams_sharing` (may be NULL)
 * receives how many of the group's streams still share the queue afterwards, 0 in the
 * normal case.  It waits for the group's previous restore and for `compute_stream`: call
 * it when the group is set up, and again if the engine changes its stream.  No
 * counterpart in the reference, whose restore streams (csrc/layerwise.cpp:629, 822) land on a
 * queue by the order of creation. */
int fkv_layerwise_set_compute_stream(fkv_layerwise *g, int32_t gpu_index, void *compute_stream,
                                     int32_t *streams_sharing);
/* Block the host until the most recent transfer has finished on all GPUs and
 * every notification has been written. */
int fkv_layerwise_synchronize(fkv_layerwise *g);
/* Milliseconds between the start of the most recent transfer and the
 * completion of each layer batch, as seen by the transfer stream of GPU 0.
 * Writes min(capacity, num_batches) values and returns the count via
 * `num_batches`. Valid after fkv_layerwise_synchronize. */
int fkv_layerwise_batch_times_ms(fkv_layerwise *g, float *out_ms, int32_t capacity,
                                 int32_t *num_batches);
/* dtor, csrc/layerwise.cpp:840-905 */
void fkv_layerwise_destroy(fkv_layerwise *g);

/* ---- host memory: flexkv/transfer/host_buffer.py:66-118, 180-202 ---- */

/* hipHostMalloc(Portable|Mapped) — alloc_mapped_host_tensor (:180-202). */
int fkv_host_alloc(size_t bytes, void **out);
int fkv_host_free(void *ptr);
/* Chunked hipHostRegister(Portable|Mapped) with rollback on failure —
 * cudaHostRegister (:66-98).  chunk_bytes == 0 registers in one call. */
int fkv_host_register(void *ptr, size_t bytes, size_t chunk_bytes);
/* Reverse of fkv_host_register with the same chunking (:101-118). */
int fkv_host_unregister(void *ptr, size_t bytes, size_t chunk_bytes);
/* The (offset, size) pieces fkv_host_register would issue; pure arithmetic.
 * Returns the number of pieces (also when it exceeds `capacity`). */
int64_t fkv_host_register_plan(size_t bytes, size_t chunk_bytes, size_t *offsets,
                               size_t *sizes, int64_t capacity);
/* FLEXKV_CUDAHOST_CHUNK_SIZE_GB -> chunk bytes, host_buffer.py:57-63. */
size_t fkv_host_chunk_bytes_from_gb(double chunk_gb);

/* ---- host pool <-> SSD files: csrc/transfer_ssd.h:215-333,
 *      csrc/transfer_ssd.cpp:327-512 ---- */

typedef struct fkv_ssd_ctx fkv_ssd_ctx;

/* SSDIOCTX (csrc/transfer_ssd.h:244-309): opens every file buffered and, where
 * the file system allows, with O_DIRECT.  `paths` is device-major,
 * num_devices * files_per_device entries.  iouring_entries > 0 asks for the
 * io_uring engine (falls back to threads when the kernel refuses it). */
int fkv_ssd_open(const char *const *paths, int32_t num_devices, int32_t files_per_device,
                 int32_t iouring_entries, int32_t iouring_flags, fkv_ssd_ctx **out);
void fkv_ssd_close(fkv_ssd_ctx *ctx);
/* 1 when the context drives an io_uring, 0 when it uses threads. */
int fkv_ssd_uses_iouring(const fkv_ssd_ctx *ctx);
/* 1 when the context's last transfer went through O_DIRECT descriptors (aligned
 * call, file system with O_DIRECT, host memory the kernel can pin), 0 when it
 * went through the page cache.  A request refused with EFAULT/EINVAL on the
 * O_DIRECT descriptor is repeated buffered, and later calls on that host pool
 * start buffered.  No counterpart in the reference, which fails such a call. */
int fkv_ssd_last_direct(const fkv_ssd_ctx *ctx);
/* transfer_kv_blocks_ssd (csrc/transfer_ssd.cpp:327-512) for layers
 * [start_layer, start_layer + num_layers).  Blocks until all bytes have moved.
 * `block_stride` applies to the host pool and to the files alike. */
int fkv_ssd_transfer(fkv_ssd_ctx *ctx, int32_t start_layer, int32_t num_layers, void *cpu_ptr,
                     const int64_t *ssd_block_ids, const int64_t *cpu_block_ids,
                     int32_t num_blocks, int64_t cpu_layer_stride, int64_t cpu_kv_stride,
                     int64_t ssd_layer_stride, int64_t ssd_kv_stride, int64_t chunk_size,
                     int64_t block_stride, int32_t is_read, int32_t round_robin,
                     int32_t num_threads_per_device, int32_t kv_dim, int32_t ssd_io_opt);
/* (device, file, block inside the file) of an SSD block id --
 * partition_and_remap_blocks_by_device, csrc/transfer_ssd.cpp:22-44, and the
 * file split at :65-67. */
int fkv_ssd_locate(int64_t ssd_block_id, int32_t round_robin, int32_t num_devices,
                   int32_t files_per_device, int32_t *device, int32_t *file,
                   int64_t *block_in_file);
/* The requests fkv_ssd_transfer would issue, without touching any file: one row
 * of five int64 per iovec -- request number, device * files_per_device + file,
 * file offset of the request, host offset of the iovec, iovec length.  Returns
 * the number of rows (also when it exceeds `capacity`), -1 on bad arguments. */
int64_t fkv_ssd_plan(int32_t num_devices, int32_t files_per_device, int32_t start_layer,
                     int32_t num_layers, const int64_t *ssd_block_ids,
                     const int64_t *cpu_block_ids, int32_t num_blocks, int64_t cpu_layer_stride,
                     int64_t cpu_kv_stride, int64_t ssd_layer_stride, int64_t ssd_kv_stride,
                     int64_t chunk_size, int64_t block_stride, int32_t round_robin,
                     int32_t kv_dim, int32_t ssd_io_opt, int64_t *out, int64_t capacity);

/* ---- engine KV blocks <-> a dense device buffer: csrc/gds/layout_transform.{cu,cuh}
 *      (the re-layout step between the engine's tensors and the device staging
 *      buffer a direct-storage read or write works on) ---- */

typedef struct fkv_layout_transform_desc {
  /* engine side, as in fkv_transfer_desc */
  int32_t backend;
  int32_t num_layers_total;
  const uint64_t *gpu_tensor_ptrs; /* host array of device addresses */
  int32_t num_gpu_tensor_ptrs;
  int32_t device;                  /* -1 = current */
  int64_t gpu_kv_stride;
  int64_t gpu_block_stride;
  int64_t gpu_layer_stride;
  /* buffer side: chunk (l, kv) of the i-th block of the call lives at
   * buffer_ptr + i*buffer_block_stride + l*buffer_layer_stride + kv*buffer_kv_stride */
  void *buffer_ptr;                /* device memory */
  int64_t buffer_layer_stride;
  int64_t buffer_kv_stride;
  int64_t buffer_block_stride;
  int64_t chunk_size;              /* bytes */
  int32_t start_layer_id;          /* engine layer of buffer layer 0; the reference always uses 0 */
  int32_t num_layers;
  int32_t kv_dim;
  int32_t num_blocks;
  const int64_t *gpu_block_ids;    /* host, num_blocks entries (device memory in the reference) */
  int32_t buffer_to_target;        /* 1: buffer -> engine tensors, 0: engine tensors -> buffer */
  int32_t sync;
} fkv_layout_transform_desc;

/* launch_layout_transform_kernel<Type> (csrc/gds/layout_transform.cu:26-108), any
 * number of blocks per call. */
int fkv_layout_transform(const fkv_layout_transform_desc *desc, void *stream);

/* ---- engine tensors shared with a worker process:
 *      flexkv/common/memory_handle.py:1144-1250 (direct IPC branch of
 *      TensorSharedHandle) ---- */

#define FKV_IPC_HANDLE_BYTES 64

/* Owner side: handle of the device allocation `device_ptr` lives in
 * (hipIpcGetMemHandle of its base address), the offset of `device_ptr` inside
 * it and, optionally, the size of the allocation.  Allocations of 2 GiB or
 * more should not be shared this way. */
int fkv_ipc_export(const void *device_ptr, uint8_t *handle_out /* 64 bytes */,
                   int64_t *offset_out, int64_t *allocation_bytes_out);
/* Worker side: map the allocation on `device` (-1 = current) and return its
 * base address.  Repeated opens of one handle in a process return the same
 * mapping and are counted. */
int fkv_ipc_open(const uint8_t *handle /* 64 bytes */, int32_t device, void **base_out);
/* Drop one reference; the mapping goes with the last one. */
int fkv_ipc_close(void *base);

/* ---- counters (the reference's FLEXKV_GPU_CPU_TRANSFER metric hook is a
 *      no-op unless monitoring is compiled in, csrc/ce_transfer.cu:29-31) ---- */
typedef struct fkv_stats {
  uint64_t calls;
  uint64_t bytes_h2d;
  uint64_t bytes_d2h;
  uint64_t kernel_launches;
  uint64_t dma_copies;
  uint64_t staging_bytes_device;
  uint64_t staging_bytes_host;
  uint64_t confined_launches; /* kernel launches restricted to a subset of the XCDs */
  uint64_t safety_net_ranges; /* current device, since the process started (not reset): pieces of
                                 confined launches copied by the fallback workgroup because no
                                 workgroup on the chosen XCDs had claimed anything in time;
                                 expected to stay 0 */
  uint64_t staged_batches;    /* layer batches of a layerwise restore that went through the copy
                                 engines and a device staging buffer */
  uint64_t gathered_batches;  /* of those, the batches whose host rows were first gathered into a
                                 pinned buffer by host threads (one copy command per batch) */
  uint64_t gather_busy_us;    /* time host threads spent gathering such rows, summed over threads */
  uint64_t second_stream_batches; /* layer batches of a layerwise restore by kernel that were launched
                                 on the group's second stream (kernel_alt_stream_kb of the policy) */
  /* plan memory (the tables a launch reads: pinned slots with a device mirror, recycled behind
   * events): slots the pool holds and slots in use right now (not reset by fkv_reset_stats),
   * and how often a caller had to wait for the oldest user because the pool was at its limit */
  uint64_t plan_slots;
  uint64_t plan_slots_in_use;
  uint64_t plan_slot_waits;
} fkv_stats;
void fkv_get_stats(fkv_stats *out);
void fkv_reset_stats(void);

/* ---- compressed staging: the codec-independent device half -------------------
 *
 * A batched codec (nvcomp ANS in the reference, csrc/compression/ans/nvcomp_ans.cu:355-500)
 * works on a table of chunk addresses and leaves payloads of different sizes in a dense
 * staging buffer.  These two calls are what surrounds it: the address table, and the
 * movement of the payloads between staging and the host cache with their sizes recorded
 * in a host-side table.  Chunk i of a batch is chunk g = batch_start + i of the call:
 *   layer = g / (kv_dim * num_blocks), kv = (g % (kv_dim * num_blocks)) / num_blocks,
 *   b = g % num_blocks.
 * Block ids are host arrays here (the reference hands its kernels device-readable ones). */

/* Replaces staging_transfer_kernel<is_write_cpu>
 * (csrc/compression/common/staging_transfer.cuh:16-101).
 *   is_write_cpu != 0: payload i (comp_sizes[i] bytes at staging + i * staging_stride) goes
 *     to the host slot of its chunk and its size into the size table; a payload larger than
 *     chunk_capacity is not copied, its table entry becomes 0 and *overflow is incremented.
 *   is_write_cpu == 0: the table entry of chunk i says how many bytes to read from its host
 *     slot into staging slot i; the size is also stored into comp_sizes[i].  An entry larger
 *     than staging_stride (the reference would overrun the slot) is not copied:
 *     comp_sizes[i] = 0 and *overflow is incremented when a counter was given. */
typedef struct fkv_staging_transfer_desc {
  void *staging;            /* device memory, bsz slots of staging_stride bytes */
  int64_t staging_stride;
  uint64_t *comp_sizes;     /* device memory, [bsz] */
  void *cpu_ptr;            /* host cache, pinned / device-visible */
  int64_t chunk_capacity;   /* bytes of one host slot */
  int32_t *overflow;        /* device memory counter (the caller clears and reads it); may be
                               NULL when reading */
  int64_t cpu_kv_stride, cpu_layer_stride, cpu_block_stride; /* bytes */
  const int64_t *cpu_block_ids; /* host array, [num_blocks] */
  uint32_t *size_table;     /* host memory, pinned / device-visible */
  int64_t size_table_block_stride, size_table_layer_stride; /* in entries; K and V adjacent */
  int32_t start_layer_id, kv_dim, num_blocks, batch_start, bsz;
  int32_t is_write_cpu;
  int32_t transfer_num_cta; /* 0 = default */
  int32_t device;           /* -1 = current */
  int32_t sync;             /* wait for the stream before returning */
} fkv_staging_transfer_desc;
int fkv_staging_transfer(const fkv_staging_transfer_desc *desc, void *stream);

/* Replaces build_gpu_chunk_ptrs_kernel<Type>
 * (csrc/compression/common/staging_transfer.cuh:103-122): out_ptrs[i] = address of chunk
 * (start_layer_id + layer, kv, gpu_block_ids[b]) in the engine's tensors, ptr_at<> of
 * csrc/gtensor_handler.cuh:43-67. */
typedef struct fkv_chunk_ptrs_desc {
  void **out_ptrs;          /* device memory, [bsz] */
  int32_t backend;          /* FKV_BACKEND_* */
  int32_t num_layers_total;
  const uint64_t *gpu_tensor_ptrs; /* host array */
  int32_t num_gpu_tensor_ptrs;
  int32_t device;           /* -1 = current */
  int64_t gpu_kv_stride, gpu_block_stride, gpu_layer_stride; /* bytes */
  const int64_t *gpu_block_ids; /* host array, [num_blocks] */
  int32_t start_layer_id, kv_dim, num_blocks, batch_start, bsz;
  int32_t sync;
} fkv_chunk_ptrs_desc;
int fkv_build_gpu_chunk_ptrs(const fkv_chunk_ptrs_desc *desc, void *stream);

/* HBM reference rates for the launches whose both ends are device memory (device
 * staging, layout transform): `reps` launches of a streaming kernel over `bytes` of
 * contiguous device memory owned by the call, timed with hip events.  mode: 0 = read
 * only, 1 = write only, 2 = copy (result counts bytes read + bytes written).  GB/s
 * (1e9 B/s) of the best repetition.  No counterpart in the reference. */
int fkv_measure_hbm_rate(int32_t device, size_t bytes, int32_t reps, int32_t mode,
                         double *best_gbps, double *median_gbps);

/* ---- launch policy: every tunable of the kernel path, per device, in one table ----
 *
 * No counterpart in the reference, whose only launch parameter is transfer_num_cta.
 * The defaults are derived from the device (the XCDs it exposes are found by a probe
 * kernel on first use); a field can be preset through the environment variable named
 * beside it, read once when the device's table is first built, and changed at run
 * time with fkv_launch_policy_set.  XCD masks name physical XCD ids (bit k = XCD k);
 * a mask that covers every XCD of the device means "not confined". */
typedef struct fkv_launch_policy {
  /* read-only (ignored by _set) */
  int32_t xcd_count;          /* XCDs the device exposes */
  uint32_t xcd_present_mask;  /* their ids */
  /* both directions at once */
  int32_t arbiter;            /* FKV_LINK_ARBITER: 0 never confine; 1 confine a launch while the
                                 other direction is busy and keep large launches to home XCDs
                                 (default on devices with 4 XCDs or more); 2 confine every
                                 link-bound launch to its busy mask; 3 (tests) confine every
                                 link-bound launch to an XCD the device does not have, so that
                                 the safety-net workgroup alone does the work */
  uint32_t d2h_busy_mask;     /* XCDs of a GPU->host launch while gets are running */
  uint32_t h2d_busy_mask;     /* XCDs of a host->GPU launch while puts are running */
  uint32_t d2h_home_mask;     /* XCDs of a large GPU->host launch on an idle link */
  uint32_t h2d_home_mask;     /* the same, host->GPU */
  int32_t busy_window_ms;     /* a direction counts as busy this long after its last launch */
  int32_t home_min_kb;        /* launches of at least this size keep to home XCDs (-1: never) */
  int32_t d2h_busy_pct;       /* workgroups of a confined launch, percent of the unconfined count */
  int32_t h2d_busy_pct;
  int32_t busy_claims_per_wg; /* ranges a working workgroup claims, confined by a busy link */
  int32_t home_claims_per_wg; /* the same on home XCDs */
  int32_t all_claims_per_wg;  /* launches on all XCDs: 0 = fixed shares */
  int32_t safety_net_wait_us; /* how long workgroup 0 of a confined launch waits before it takes
                                 over a launch of which nothing landed on a selected XCD */
  int32_t link_gbps_estimate; /* what other processes are told a launch will take: bytes / this */
  /* launch shape of the link-bound kernel */
  int32_t d2h_wg_per_cta;     /* workgroups per requested CTA (transfer_num_cta) */
  int32_t h2d_wg_per_cta;
  int32_t d2h_wg_threads;     /* lanes per workgroup */
  int32_t h2d_wg_threads;
  int32_t packed_grid_pct;    /* packed short chunks: workgroups, percent of the normal count */
  int32_t plan_mirror;        /* -1 upload the plan unless the other direction is busy, 0 never, 1 always */
  int32_t fuse_launches;      /* members of one layer in one launch */
  int32_t lane_streams;       /* FKV_LANE_STREAMS: -1 auto, 0 never, 1 always */
  /* layerwise restore through the copy engines (see fkv_layerwise_transfer) */
  int32_t staged_restore;     /* FKV_STAGED_RESTORE: 0 never, 1 when the host blocks form few
                                 runs (default), 2 whenever the layout allows it */
  int32_t staged_ring;        /* staging buffers per layer group and GPU */
  int32_t staged_copy_overhead_us; /* cost of one more copy command, for the choice */
  int32_t staged_overhead_pct;     /* staged when copies x overhead stays below this share of
                                      the batch's time on the link */
  int32_t staged_bridge_kb;   /* holes between runs of host blocks up to this size are read along */
  int32_t staged_max_mb;      /* largest staging buffer (one of the ring) */
  /* HBM-bound launches: device compaction of the copy-engine strategies, layout transform,
   * the scatter of a staged restore */
  int32_t hbm_workgroups;
  int32_t hbm_wg_threads;
  int32_t hbm_unroll;         /* 16-byte vectors in flight per lane in these launches: 8 or 16 */
  int32_t ce_staging_mb;      /* FKV_CE_STAGING_MB: device staging of the copy-engine strategies */
  int32_t ce_two_streams;     /* 0: every copy of a copy-engine strategy on the caller's stream;
                                 2: runs of eight and more independent copies alternate between it
                                 and a second stream; 1 (default): that, and a GATHER_DIRECT that
                                 needs several staging groups of few, large copies alternates
                                 between two staging buffers, compaction launches on the caller's
                                 stream next to the copies on the second */
  int32_t ce_rect_min_kb;     /* copies of at least this size are issued as 2-D copies of one row,
                                 which the runtime hands to the copy engines (it is free to run a
                                 1-D hipMemcpyAsync between pinned host and device memory as a
                                 kernel on the compute units), except where a host thread waits
                                 for each copy (the staging ping-pong of SEGMENT_SCATTER and
                                 GATHER_SCATTER); 0 = all copies, -1 = none; default 32768 */
  /* cost model of fkv_choose_engine (use_ce_transfer = 2): what each engine is expected to take */
  int32_t model_link_mbps;          /* the link under plain copy-engine copies, MB/s */
  int32_t model_kernel_d2h_mbps;    /* the gather/scatter kernel GPU->host */
  int32_t model_kernel_h2d_mbps;    /* ... host->GPU */
  int32_t model_dma_ns;             /* cost of one more copy command over two streams */
  int32_t model_compaction_gbps;    /* device compaction pass, GB/s of bytes staged */
  int32_t model_host_pass_mbps;     /* host scatter/gather pass */
  int32_t model_launch_ns;          /* plan + launch of the kernel path */
  int32_t model_prefer_ce_pct;      /* the copy engine wins up to this percentage of the kernel's
                                       time: it leaves the CUs and their memory queues alone */
  int32_t d2h_lane_runs;      /* GPU->host launches with 16-byte vectors let every lane store 128
                                 adjacent bytes instead of every wavefront access 1 KiB: 0 never,
                                 1 (default) unless the other direction is busy, 2 always (about
                                 +1 % alone on the link, -2 % in sum next to traffic the other way) */
  /* layerwise restore of scattered host blocks: host threads gather a batch's rows into a
   * pinned buffer, one copy command moves it (see fkv_layerwise_transfer) */
  int32_t staged_gather;      /* FKV_STAGED_GATHER: 0 never; 1 (default) where the host blocks form
                                 too many runs for one copy command each and the gather threads
                                 keep up with the link; 2 whenever the copies-per-run route is
                                 not taken.  Both in groups of one GPU only: with several, the
                                 launching thread would gather for one GPU after the other (the
                                 same rows again where the ranks share their KV), and the route
                                 has run on one device only.  3 = like 2, groups of several GPUs
                                 included (host-side tests) */
  int32_t gather_threads;     /* FKV_GATHER_THREADS: host threads that gather (the launching thread
                                 of the restore is one of them); default 6, at most the cores of
                                 the machine less one */
  int32_t gather_ring;        /* pinned buffers per layer group and GPU */
  int32_t gather_first_by_kernel; /* 1 (default): the first batch of such a restore goes the kernel
                                 way, so that it lands one gather pass earlier while the rows of
                                 the second batch are being gathered */
  int32_t model_gather_thread_mbps; /* what one host thread gathers, MB/s, for the choice */
  /* where the rates of the cost model come from */
  int32_t model_seed;         /* FKV_MODEL_SEED: 1 (default) the first call that needs the model on a
                                 device measures the link once (two short pinned copies per direction)
                                 and scales the link-bound rates above by measured / compiled-in;
                                 0 keeps the compiled-in figures */
  int32_t model_seeded;       /* read-only: 1 once the rates of this table come from a measurement */
  int32_t staged_scatter_threads; /* lanes per workgroup of the launch that places a staged batch
                                 (staging buffer -> engine blocks); default 256: next to the
                                 engine's own kernels a workgroup of 256 lanes finds room on a
                                 CU where one of 1024 waits (36 MiB: 26 us against 146 us at the
                                 median next to fused attention, 17 us against 21 us alone) */
  int32_t test_fail_restore_batch; /* tests: n > 0 makes a layerwise restore give up before it
                                 enqueues its n-th batch, as a failed launch would (nothing faults:
                                 the batches before it run and are announced, the rest never lands) */
  int32_t staged_dma_streams; /* streams per GPU on which a layerwise restore issues its copy-engine
                                 copies, one per run of host blocks: 2 (default) consecutive batches
                                 alternate between two (batches of gathered rows keep to one), so
                                 that the event record and wait around a copy run next to the other
                                 stream's copy (4 MiB a batch: 84 us against 93 us per batch; the
                                 engine still takes the copies in the order of submission); 1 all
                                 on one */
  int32_t kernel_alt_stream_kb; /* a layerwise restore by kernel of twelve and more batches launches
                                 every other batch of at most this many KiB, from the third on, on a
                                 second stream, so that it starts while
                                 the last requests of its predecessor are in flight (two launches
                                 on one stream lie 8 us apart, next to 18 us of link time for
                                 1 MiB); events, notifications and wait_layer stay per batch and
                                 in order.  Default 4096; 0 = one stream */
  int32_t quiet_wait_us;        /* how a call waits for its transfer (sync = 1, the thread group, the
                                 layerwise restore in HOSTFUNC mode, fkv_layerwise_synchronize): the
                                 runtime's own waits keep a core busy for as long as they last (a
                                 synchronous 9 ms transfer costs 9 ms of CPU time, 64 waiting
                                 requests 13 of 16 cores, and the threads that still have to submit
                                 theirs wait for a core).  > 0 (default 100): while two threads of the
                                 process are already waiting the runtime's way, further ones poll
                                 their event instead: they sleep towards the moment the transfer
                                 would end alone on the link, spin for the 80 us around it, and
                                 after that sleep for spells that double from 20 us up to this many
                                 microseconds (2 % of a core each; such a wait ends up to that much
                                 later).  A caller that waits for one transfer at a time sees no
                                 difference, except that a transfer expected to take 20 ms or more
                                 (1.1 GB) is polled for as well, at a cost of a few parts in a
                                 thousand.  < 0: every waiting thread polls, with -value as the
                                 limit (a worker then costs 2 % of a core while it waits instead of a
                                 whole one, and its 9.4 ms op ends up to 0.1 ms later).  0 = always
                                 the runtime's wait */
} fkv_launch_policy;
/* The table of `device` (-1 = current).  The first call for a device runs the probe kernel. */
int fkv_launch_policy_get(int32_t device, fkv_launch_policy *out);
/* Replaces the table of `device`; read-only fields are ignored, masks are cut to the
 * XCDs the device has (except with arbiter == 3), counts are clamped to sane ranges. */
int fkv_launch_policy_set(int32_t device, const fkv_launch_policy *in);
/* Back to the defaults derived from the device and the environment. */
int fkv_launch_policy_reset(int32_t device);
/* Re-bases the figures of the table that depend on the host link of the box
 * (model_link_mbps, model_kernel_{d2h,h2d}_mbps, link_gbps_estimate, staged_copy_overhead_us)
 * on a measurement of `device`: three pinned copies of 64 MiB per direction and a burst of
 * small 2-D copies, once per device and process.  The library does this by itself before the
 * first layerwise restore and the first transfer with use_ce_transfer == 2 on a device
 * (model_seed = 0 / FKV_MODEL_SEED=0: never); fields that the caller or the environment has
 * changed from the compiled-in figure are left alone.  The reference fixes the engine per
 * direction by configuration (flexkv/common/config.py:770-786) and has no such model. */
int fkv_launch_policy_seed(int32_t device);
/* The arithmetic of the above without a device: `in` re-based on the given rates (GB/s) and
 * cost of a copy command (us; 0 = unknown). */
int fkv_launch_policy_seeded(const fkv_launch_policy *in, double d2h_gbps, double h2d_gbps,
                             double copy_overhead_us, fkv_launch_policy *out);

/* The arithmetic behind the staged layerwise restore, without a device (tests,
 * inspection): the runs of consecutive host block ids of a call, with the holes that are
 * read along, and which way a restore of these blocks goes under `policy` (brought into
 * its allowed ranges first): *staged = 0 the kernel path, 1 through the copy engines with
 * one copy command per run (runs, rows and row_of_position describe the staging buffer),
 * 2 through the copy engines after host threads have gathered the rows (no runs; the
 * staging row of position p is p).  `row_bytes` = bytes of one host block that one batch
 * of layers moves, `pieces` = copy commands per run and batch, which is also the number
 * of pieces a gathering thread copies per block (1 when a batch's chunks of a block are
 * adjacent on the host).  A layerwise call applies it whichever engine it was asked for
 * (use_ce_transfer only decides what the other batches fall back to), and with
 * staged_restore = 0 for a host pool that the device cannot read.  No counterpart in the
 * reference. */
typedef struct fkv_staged_run {
  int64_t first_id; /* first host block of the run */
  int32_t rows;     /* host blocks it spans, holes read along included */
  int32_t row0;     /* staging row of the first */
} fkv_staged_run;
int fkv_staged_restore_plan(const int64_t *cpu_block_ids, int32_t num_blocks, int64_t row_bytes,
                            int32_t pieces, const fkv_launch_policy *policy, int32_t *staged,
                            int32_t *num_runs, int64_t *total_rows, fkv_staged_run *runs,
                            int32_t run_capacity, int64_t *row_of_position);

/* Host-link reference rate: `reps` plain hipMemcpyAsync copies of `bytes`
 * between a pinned host buffer and a device buffer (both owned by the call),
 * timed with hip events.  direction: 0 = D2H, 1 = H2D.  Result in GB/s
 * (1e9 B/s) of the best repetition.  No counterpart in the reference. */
int fkv_measure_link_peak(int32_t device, size_t bytes, int32_t reps,
                          int32_t direction, double *best_gbps, double *median_gbps);

/* Named ranges for a profiler's timeline (rocprofv3 --marker-trace), where the
 * reference annotates with NVTX (csrc/layerwise.cpp:1073, 1380;
 * flexkv/transfer/worker.py:556-587, 1062-1095).  With FKV_ROCTX=1 in the
 * environment the two calls forward to roctxRangePushA / roctxRangePop of the
 * ROCm marker library, loaded on first use; otherwise, or when the library is
 * not installed, they do nothing.  The library brackets its own transfers the
 * same way.  Return 1 when the range was forwarded, 0 when not. */
int fkv_range_push(const char *label);
int fkv_range_pop(void);

/* Whether kernels on two streams of `device` can run at the same time.  A
 * process has few hardware queues (GPU_MAX_HW_QUEUES, 4 by default) and streams
 * that share one run their kernels one after the other: a stream of puts and a
 * stream of gets on the same queue move the one-way rate in sum.  The call times
 * a short wait kernel on `stream_a` alone and then on both streams at once (it
 * synchronises both streams) and sets *concurrent to 1 when the pair took less
 * than 1.5x the single one.  No counterpart in the reference. */
int fkv_streams_run_concurrently(int32_t device, void *stream_a, void *stream_b,
                                 int32_t *concurrent);
/* How long an event takes from one stream to another and back on the device: a chain of 16
 * round trips (tiny kernel, record, wait on the other stream, tiny kernel, record, wait) is
 * enqueued behind a 2 ms gate kernel and timed with events; *round_trip_us is the time per
 * round trip, the better of two runs.  A stream with itself takes 10 us, streams on different
 * hardware queues normally 22 us; with more than four queues some pairs take 107-118 us
 * although their kernels run at the same time (they share hardware further down), and a restore that hands an event to the
 * engine's stream per layer loses that time per layer.  Synchronises both streams.  No
 * counterpart in the reference. */
int fkv_streams_hand_over_us(int32_t device, void *stream_a, void *stream_b, double *round_trip_us);

/* Link activity across processes.  A put and a get that run at the same time are
 * kept on different XCDs; so that this also works when they come from different
 * processes (a worker for puts, another for layerwise restores), every process
 * posts its link-bound launches on a small board in /dev/shm (one per user and
 * GPU, keyed by the PCI address; FKV_LINK_BOARD=0 disables it,
 * FKV_LINK_BOARD_KEY replaces the PCI address).  The library posts its own
 * launches; a process that moves bytes over the link by other means can post
 * them with fkv_link_activity_post (`expected_us`: for how long from now, or from
 * the end of what it has already posted).  fkv_link_activity_elsewhere sets *busy
 * to 1 when another process has posted activity in that direction that has not
 * ended more than `window_ms` ago.  No counterpart in the reference. */
int fkv_link_activity_post(int32_t device, int32_t is_host_to_device, int64_t expected_us);
int fkv_link_activity_elsewhere(int32_t device, int32_t is_host_to_device, int32_t window_ms,
                                int32_t *busy);

#ifdef __cplusplus
}
#endif
#endif /* FKV_TRANSFER_H */
