/*
 * fkv_oracle.c — CPU restatement of FlexKV's GPU<->CPU KV-block transfer
 * arithmetic.  TEST INFRASTRUCTURE ONLY: the checker that the HIP path is
 * compared against, and the scalar CPU baseline that the benchmark times.
 * Nothing in the shipped library links, loads or calls this file.
 *
 * "GPU memory" here is ordinary host memory: the tensor-pointer table holds
 * host addresses, so every function runs without a GPU.
 *
 * Each function names the reference source it follows (paths relative to the
 * FlexKV tree).  The reference does its address arithmetic in int64 units
 * after dividing every byte quantity by 8 (csrc/transfer.cu:179-187,
 * csrc/gtensor_handler.cuh:30-32); this file keeps bytes.  The two agree
 * exactly whenever all strides, offsets and the chunk size are multiples of
 * 8, which the reference requires; fkv_oracle_units_ok() reports that
 * precondition.
 *
 * How each function is pinned (so a wrong sign, index or dropped term fails):
 *   fkv_oracle_chunk_addr     brute force against torch/numpy fancy indexing
 *                             on tensors of the engines' documented shapes
 *                             (tests/test_oracle.py), and the reference
 *                             tests' fill formula as a known answer
 *   fkv_oracle_transfer       same + round-trip identity + untouched-byte
 *                             guard pattern + agreement with the independent
 *                             numpy index formulation (oracle/fkv_oracle.py)
 *   fkv_oracle_ce_analyze     segment definition by brute force (maximal
 *                             runs where both id lists step by +1)
 *   fkv_oracle_ce_choose_path the strategy matrix of the reference's own
 *                             test predictor, restated by pattern/layout
 *                             names (tests/test_ce_analysis.py)
 *   fkv_oracle_tp_rank_plan   closed forms + partition properties (shards
 *                             tile the chunk, layer slices tile the range)
 *   fkv_oracle_host_scatter   numpy fancy indexing of shaped [N,L,kv,chunk] and
 *                             [L,kv,N,chunk] pools, both directions, untouched bytes,
 *                             in-chunk offsets (tests/test_oracle.py)
 *   fkv_oracle_is_full_block  the shapes the reference names: rank0_only / all_write
 *                             calls are full blocks, layer_parallel and sharded puts
 *                             are not (per-rank shapes from the rank plan, host block
 *                             from the layout's closed form; tests/test_oracle.py)
 *   fkv_oracle_eventfd_index  enumeration of a [3, tp, layers] table in Python loops
 *                             (tests/test_oracle.py); the GPU tests of the
 *                             notification contract index their eventfds with it
 *   fkv_oracle_layerwise_cpu_startoff  closed forms per mode (tests/test_tp_plan.py)
 *   fkv_oracle_host_chunk_bytes  the reference's constants (tests/test_abi.py)
 *   fkv_oracle_ssd_locate     the reference's second statement of the same
 *                             mapping (flexkv/transfer/nixlutil.py:351-385) as
 *                             closed forms, bijection onto a dense
 *                             (device, file, block) grid by brute force
 *   fkv_oracle_ssd_transfer   the reference tests' fixture (host pool filled
 *                             with arange % 9973, identity ids, one file of the
 *                             pool's own layout): the file image equals the
 *                             pool image; round trip; several files / devices
 *                             against numpy indexing of per-file arrays
 *   fkv_oracle_layout_transform  torch fancy indexing of shaped engine tensors
 *                             into a shaped [block, layer, kv, chunk] buffer,
 *                             for the three engine layouts; padded buffer
 *                             strides leave the padding untouched; round trip
 *   fkv_oracle_staging_transfer  a second, shaped statement in numpy (host cache
 *                             [N, L, kv, capacity] and size table [N, L, kv] indexed
 *                             by (layer, kv, id) in Python loops), oversize payloads,
 *                             batches that start and end inside a layer, write ->
 *                             read round trip (tests/test_staging.py)
 *   fkv_oracle_chunk_ptrs     equality with fkv_oracle_chunk_addr per (layer, kv,
 *                             block) enumerated in Python, all three engines
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FKV_BACKEND_VLLM 0
#define FKV_BACKEND_TRTLLM 1
#define FKV_BACKEND_SGLANG 2

/* csrc/transfer.cu:34-40 and :179-187 — every byte quantity is divided by 8
 * (and by 16 for the vector kernel); non-multiples are silently truncated in
 * the reference.  Returns 16, 8 or 0 (= outside the reference's domain). */
int fkv_oracle_units_ok(int64_t chunk, int64_t gpu_off, int64_t cpu_off,
                        int64_t gks, int64_t gbs, int64_t gls, int64_t cks,
                        int64_t cls, int64_t cbs) {
  if ((chunk | gpu_off | cpu_off | gks | gbs | gls | cks | cls | cbs) & 7)
    return 0;
  if ((chunk % 16 == 0) && (gpu_off % 16 == 0) && (cpu_off % 16 == 0))
    return 16; /* float4 kernel, csrc/transfer.cu:96-158 */
  return 8;    /* int64 kernel,  csrc/transfer.cu:45-92 */
}

/* csrc/gtensor_handler.cuh:43-67 (ptr_at<VLLM|TRTLLM|SGLANG>), in bytes. */
uint64_t fkv_oracle_chunk_addr(int backend, const uint64_t *tensor_ptrs,
                               int64_t num_layers_total, int64_t kv_stride,
                               int64_t block_stride, int64_t layer_stride,
                               int64_t layer, int64_t kv, int64_t block) {
  switch (backend) {
  case FKV_BACKEND_VLLM:
    return tensor_ptrs[layer] + (uint64_t)(kv * kv_stride) +
           (uint64_t)(block * block_stride);
  case FKV_BACKEND_TRTLLM:
    return tensor_ptrs[0] + (uint64_t)(block * block_stride) +
           (uint64_t)(layer * layer_stride) + (uint64_t)(kv * kv_stride);
  case FKV_BACKEND_SGLANG:
    return tensor_ptrs[kv * num_layers_total + layer] +
           (uint64_t)(block * block_stride);
  default:
    return 0;
  }
}

/* csrc/transfer.cu:96-158 (and :45-92, same byte effect): for every
 * (layer, block position, kv) copy one chunk between
 *   gpu = ptr_at(layer, kv, gpu_ids[pos]) + gpu_off
 *   cpu = cpu_ptr + layer*cLs + kv*cKs + cpu_ids[pos]*cBs + cpu_off
 * with `layer` the ABSOLUTE layer index on both sides (:119).
 * Returns 0, or -1 for an unknown backend. */
int fkv_oracle_transfer(int backend, const uint64_t *tensor_ptrs,
                        int64_t num_layers_total, int64_t gpu_kv_stride,
                        int64_t gpu_block_stride, int64_t gpu_layer_stride,
                        int64_t gpu_off, uint8_t *cpu_ptr, int64_t cpu_kv_stride,
                        int64_t cpu_layer_stride, int64_t cpu_block_stride,
                        int64_t cpu_off, int64_t chunk, int start_layer,
                        int num_layers, int kv_dim, int num_blocks,
                        const int64_t *gpu_ids, const int64_t *cpu_ids,
                        int is_host_to_device) {
  if (backend < 0 || backend > 2)
    return -1;
  for (int l = start_layer; l < start_layer + num_layers; ++l) {
    for (int pos = 0; pos < num_blocks; ++pos) {
      uint8_t *cpu_base = cpu_ptr + (int64_t)l * cpu_layer_stride +
                          cpu_ids[pos] * cpu_block_stride + cpu_off;
      for (int kv = 0; kv < kv_dim; ++kv) {
        uint8_t *c = cpu_base + (int64_t)kv * cpu_kv_stride;
        uint8_t *g = (uint8_t *)(uintptr_t)(fkv_oracle_chunk_addr(
                         backend, tensor_ptrs, num_layers_total, gpu_kv_stride,
                         gpu_block_stride, gpu_layer_stride, l, kv,
                         gpu_ids[pos])) +
                     gpu_off;
        if (is_host_to_device)
          memcpy(g, c, (size_t)chunk);
        else
          memcpy(c, g, (size_t)chunk);
      }
    }
  }
  return 0;
}

/* csrc/ce_transfer.h:53-65 */
typedef struct {
  int32_t start_k;
  int32_t nr_blocks;
} fkv_oracle_segment;

typedef struct {
  int32_t gpu_log_contig;
  int32_t cpu_log_contig;
  int32_t cpu_phys_contig;
  int32_t gpu_phys_contig;
  int32_t num_segments;
  int32_t reserved;
} fkv_oracle_analysis;

/* csrc/ce_transfer.cu:37-66 (analyze_ce_transfer). */
void fkv_oracle_ce_analyze(const int64_t *gpu_ids, const int64_t *cpu_ids,
                           int num_blocks, int64_t cpu_block_stride,
                           int64_t chunk, int64_t gpu_block_stride,
                           fkv_oracle_analysis *out, fkv_oracle_segment *segs,
                           int seg_cap) {
  out->gpu_log_contig = 1;
  out->cpu_log_contig = 1;
  out->cpu_phys_contig = (cpu_block_stride == chunk);
  out->gpu_phys_contig = (gpu_block_stride == 0 || gpu_block_stride == chunk);
  out->num_segments = 0;
  out->reserved = 0;
  if (num_blocks == 0)
    return;
  int n = 0, seg_start = 0;
  for (int k = 1; k < num_blocks; ++k) {
    int src_step = (gpu_ids[k] == gpu_ids[k - 1] + 1);
    int dst_step = (cpu_ids[k] == cpu_ids[k - 1] + 1);
    if (!src_step)
      out->gpu_log_contig = 0;
    if (!dst_step)
      out->cpu_log_contig = 0;
    if (!src_step || !dst_step) {
      if (segs && n < seg_cap) {
        segs[n].start_k = seg_start;
        segs[n].nr_blocks = k - seg_start;
      }
      ++n;
      seg_start = k;
    }
  }
  if (segs && n < seg_cap) {
    segs[n].start_k = seg_start;
    segs[n].nr_blocks = num_blocks - seg_start;
  }
  ++n;
  out->num_segments = n;
}

#define CE_CONTIG_DIRECT 0
#define CE_SEGMENT_DIRECT 1
#define CE_SEGMENT_SCATTER 2
#define CE_GATHER_SCATTER 3
#define CE_GATHER_DIRECT 4

/* csrc/ce_transfer.cu:71-104 (choose_path). */
int fkv_oracle_ce_choose_path(const fkv_oracle_analysis *a, int is_blockfirst,
                              int num_kv_heads, int64_t segment_threshold,
                              int64_t chunk, int is_host_to_device,
                              int is_full_block) {
  int odd_chunk = (chunk > 0 && chunk % 8 != 0);
  if (is_blockfirst && !a->cpu_phys_contig && a->gpu_phys_contig) {
    if (!is_host_to_device && num_kv_heads == 1) {
      if (a->num_segments > segment_threshold)
        return odd_chunk ? CE_SEGMENT_SCATTER : CE_GATHER_SCATTER;
      if (!is_full_block)
        return CE_SEGMENT_SCATTER;
    }
    return CE_GATHER_DIRECT;
  }
  if (a->gpu_log_contig && a->cpu_log_contig && a->cpu_phys_contig &&
      a->gpu_phys_contig)
    return CE_CONTIG_DIRECT;
  if (!a->gpu_phys_contig)
    return CE_GATHER_SCATTER;
  if (a->num_segments <= segment_threshold)
    return a->cpu_phys_contig ? CE_SEGMENT_DIRECT : CE_SEGMENT_SCATTER;
  return odd_chunk ? CE_SEGMENT_SCATTER : CE_GATHER_SCATTER;
}

/* csrc/transfer.cu:219-220 */
int fkv_oracle_is_full_block(int num_layers, int kv_dim, int64_t chunk,
                             int64_t cpu_block_stride) {
  return (int64_t)num_layers * kv_dim * chunk == cpu_block_stride;
}

typedef struct {
  int32_t active;
  int32_t start_layer;
  int32_t num_layers;
  int32_t reserved;
  int64_t cpu_startoff;
  int64_t gpu_startoff;
  int64_t chunk_size;
} fkv_oracle_rank_plan;

static int mode_is(const char *m, const char *s) { return strcmp(m, s) == 0; }

/* csrc/tp_transfer_thread_group.cpp:222-323: which rank moves what.
 * Returns 0, or -1 for the sharded D2H case whose chunk does not divide
 * (:237-247 throws). */
int fkv_oracle_tp_rank_plan(int rank, int num_gpus, int num_kv_heads,
                            int is_host_to_device, const char *mode_in,
                            int designated_rank, int rotate_counter, int layer_id,
                            int layer_granularity, int num_blocks,
                            int64_t gpu_chunk_size, int64_t cpu_block_stride,
                            int64_t cpu_tp_stride, fkv_oracle_rank_plan *out) {
  const char *mode = mode_in;
  /* :222-230 unknown mode (shared KV only) -> sharded */
  if (num_kv_heads == 1 && !mode_is(mode, "sharded") &&
      !mode_is(mode, "all_write") && !mode_is(mode, "rank0_only") &&
      !mode_is(mode, "layer_parallel") && !mode_is(mode, "rank_rotate"))
    mode = "sharded";
  int shared_d2h = (num_kv_heads == 1 && !is_host_to_device);
  if (shared_d2h && mode_is(mode, "sharded") && num_gpus > 1 &&
      gpu_chunk_size % num_gpus != 0)
    return -1;
  int eff_designated = designated_rank;
  if (shared_d2h && mode_is(mode, "rank_rotate"))
    eff_designated = rotate_counter; /* :249-254 */

  out->active = 1;
  out->start_layer = layer_id;
  out->num_layers = layer_granularity;
  out->reserved = 0;
  out->cpu_startoff = 0;
  out->gpu_startoff = 0;
  out->chunk_size = gpu_chunk_size;

  if (shared_d2h && (mode_is(mode, "rank0_only") || mode_is(mode, "rank_rotate")) &&
      rank != eff_designated) {
    out->active = 0; /* :257-265 */
    return 0;
  }
  if (shared_d2h && mode_is(mode, "layer_parallel")) {
    int per = layer_granularity / num_gpus, rem = layer_granularity % num_gpus;
    int mine = rank < rem ? per + 1 : per;
    if (mine == 0) {
      out->active = 0; /* :268-278 */
      return 0;
    }
    int start = rank < rem ? rank * (per + 1)
                           : rem * (per + 1) + (rank - rem) * per; /* :309-323 */
    out->start_layer = layer_id + start;
    out->num_layers = mine;
  }
  if (num_kv_heads > 1) {
    out->cpu_startoff = (int64_t)rank * cpu_tp_stride; /* :293-294 */
  } else if (mode_is(mode, "sharded") && !is_host_to_device) {
    int64_t shard = gpu_chunk_size / num_gpus; /* :295-300 */
    out->cpu_startoff = rank * shard;
    out->gpu_startoff = rank * shard;
    out->chunk_size = shard;
  } else if (mode_is(mode, "all_write")) {
    out->cpu_startoff = (int64_t)rank * num_blocks * cpu_block_stride; /* :301-304 */
  }
  return 0;
}

/* csrc/layerwise.cpp:1143-1166: host offset of rank `rank` for the
 * host->GPU restore (chunk is always full, gpu offset always 0). */
int64_t fkv_oracle_layerwise_cpu_startoff(int rank, int num_kv_heads,
                                          const char *mode_in, int num_blocks,
                                          int64_t cpu_block_stride,
                                          int64_t cpu_tp_stride) {
  if (num_kv_heads != 1)
    return (int64_t)rank * cpu_tp_stride;
  const char *mode = mode_in;
  if (!mode_is(mode, "sharded") && !mode_is(mode, "all_write") &&
      !mode_is(mode, "rank0_only"))
    mode = "sharded"; /* :1112-1121 */
  if (mode_is(mode, "all_write"))
    return (int64_t)rank * num_blocks * cpu_block_stride;
  return 0;
}

/* csrc/ce_transfer.cu:523-579 (scatter_to_cpu) / :585-641 (gather_from_cpu):
 * staging[k*chunk .. ] <-> cpu_base(layer,kv) + cpu_ids[k]*cBs. */
void fkv_oracle_host_scatter(uint8_t *staging, uint8_t *cpu_ptr,
                             const int64_t *cpu_ids, int num_blocks,
                             int64_t cpu_block_stride, int64_t cpu_off,
                             int64_t chunk, int layer, int kv,
                             int64_t cpu_kv_stride, int64_t cpu_layer_stride,
                             int to_cpu) {
  uint8_t *base =
      cpu_ptr + (int64_t)layer * cpu_layer_stride + (int64_t)kv * cpu_kv_stride + cpu_off;
  for (int k = 0; k < num_blocks; ++k) {
    uint8_t *c = base + cpu_ids[k] * cpu_block_stride;
    uint8_t *s = staging + (int64_t)k * chunk;
    if (to_cpu)
      memcpy(c, s, (size_t)chunk);
    else
      memcpy(s, c, (size_t)chunk);
  }
}

/* csrc/layerwise.cpp:15-34, 537-544: index of the eventfd that announces
 * (counter, tp_rank, layer) in the flat [counters, tp, layers] table. */
int64_t fkv_oracle_eventfd_index(int counter, int tp_rank, int layer, int tp_size,
                                 int num_layers) {
  return (int64_t)counter * tp_size * num_layers + (int64_t)tp_rank * num_layers +
         layer;
}

/* flexkv/transfer/host_buffer.py:57-63: FLEXKV_CUDAHOST_CHUNK_SIZE_GB ->
 * bytes (4 KiB safety margin, rounded down to a page). */
uint64_t fkv_oracle_host_chunk_bytes(double chunk_gb) {
  if (chunk_gb <= 0)
    return 0;
  int64_t c = (int64_t)(chunk_gb * (double)(1024LL * 1024 * 1024)) - 4096;
  return (uint64_t)(c & ~0xFFFLL);
}


/* ---- host pool <-> SSD files ------------------------------------------- */

/* partition_and_remap_blocks_by_device, csrc/transfer_ssd.cpp:22-44, and the
 * split of a device's blocks over its files, :65-67. */
void fkv_oracle_ssd_locate(int64_t ssd_block_id, int round_robin, int num_devices,
                           int files_per_device, int *device, int *file,
                           int64_t *block_in_file) {
  int64_t in_device;
  *device = (int)((ssd_block_id / round_robin) % num_devices);
  in_device = ((ssd_block_id / round_robin) / num_devices) * round_robin +
              (ssd_block_id % round_robin);
  *file = (int)(in_device % files_per_device);
  *block_in_file = in_device / files_per_device;
}

/* transfer_kv_blocks_ssd in its baseline form, csrc/transfer_ssd.cpp:187-255:
 * one chunk per (block, layer, kv).  `files[device * files_per_device + file]`
 * are byte arrays standing in for the files.  Returns -1 when a chunk would
 * fall outside its file (`file_bytes`). */
int fkv_oracle_ssd_transfer(uint8_t *const *files, int64_t file_bytes, int num_devices,
                            int files_per_device, int start_layer, int num_layers,
                            uint8_t *cpu_ptr, const int64_t *ssd_block_ids,
                            const int64_t *cpu_block_ids, int num_blocks,
                            int64_t cpu_layer_stride, int64_t cpu_kv_stride,
                            int64_t ssd_layer_stride, int64_t ssd_kv_stride,
                            int64_t chunk, int64_t block_stride, int is_read,
                            int round_robin, int kv_dim) {
  int b, l, kv;
  for (b = 0; b < num_blocks; ++b) {
    int device, file;
    int64_t in_file;
    fkv_oracle_ssd_locate(ssd_block_ids[b], round_robin, num_devices, files_per_device,
                          &device, &file, &in_file);
    for (l = start_layer; l < start_layer + num_layers; ++l)
      for (kv = 0; kv < kv_dim; ++kv) {
        const int64_t fo = in_file * block_stride + l * ssd_layer_stride + kv * ssd_kv_stride;
        uint8_t *h = cpu_ptr + cpu_block_ids[b] * block_stride + l * cpu_layer_stride +
                     kv * cpu_kv_stride;
        uint8_t *f = files[device * files_per_device + file] + fo;
        if (fo < 0 || fo + chunk > file_bytes)
          return -1;
        if (is_read)
          memcpy(h, f, (size_t)chunk);
        else
          memcpy(f, h, (size_t)chunk);
      }
  }
  return 0;
}

/* csrc/gds/layout_transform.cu:41-70: chunk index c in [0, L*K*N) names
 *   block position  c % N,  layer  c / (N*K),  kv  (c % (N*K)) / N;
 *   buffer = base + pos*bBs + layer*bLs + kv*bKs
 *   engine = ptr_at(start_layer + layer, kv, gpu_ids[pos])
 * (the reference passes layer itself, i.e. start_layer = 0).  Bytes here,
 * 8-byte words there.  Returns 0, or -1 for an unknown backend. */
int fkv_oracle_layout_transform(uint8_t *buffer, int64_t buffer_layer_stride,
                                int64_t buffer_kv_stride, int64_t buffer_block_stride,
                                int64_t chunk, int backend, const uint64_t *tensor_ptrs,
                                int64_t num_layers_total, int64_t gpu_kv_stride,
                                int64_t gpu_block_stride, int64_t gpu_layer_stride,
                                const int64_t *gpu_ids, int num_blocks, int start_layer,
                                int num_layers, int kv_dim, int buffer_to_target) {
  if (backend < 0 || backend > 2)
    return -1;
  const int64_t num_chunks = (int64_t)num_layers * kv_dim * num_blocks;
  for (int64_t c = 0; c < num_chunks; ++c) {
    const int64_t pos = c % num_blocks;
    const int64_t layer = c / ((int64_t)num_blocks * kv_dim);
    const int64_t kv = (c % ((int64_t)num_blocks * kv_dim)) / num_blocks;
    uint8_t *buf = buffer + pos * buffer_block_stride + layer * buffer_layer_stride +
                   kv * buffer_kv_stride;
    uint8_t *gpu = (uint8_t *)(uintptr_t)fkv_oracle_chunk_addr(
        backend, tensor_ptrs, num_layers_total, gpu_kv_stride, gpu_block_stride,
        gpu_layer_stride, start_layer + layer, kv, gpu_ids[pos]);
    if (buffer_to_target)
      memcpy(gpu, buf, (size_t)chunk);
    else
      memcpy(buf, gpu, (size_t)chunk);
  }
  return 0;
}

/* csrc/compression/common/staging_transfer.cuh:16-101 (staging_transfer_kernel):
 * chunk i of the batch is chunk g = batch_start + i of the call,
 *   layer = g / (kv_dim*num_blocks), kv = (g % (kv_dim*num_blocks)) / num_blocks,
 *   b = g % num_blocks;
 * host slot = cpu + (layer+start_layer)*cLs + kv*cKs + cpu_ids[b]*cBs,
 * table entry = table + cpu_ids[b]*tBs + (start_layer+layer)*tLs + kv.
 * Write: size > capacity -> ++overflow, entry = 0, no copy; else entry = size and
 * `size` bytes go staging -> host.  Read: size = entry, comp_sizes[i] = size, `size`
 * bytes go host -> staging.  The reference does not guard a read entry larger than
 * the staging slot (it would overrun it); here such an entry is counted in
 * *overflow, comp_sizes[i] = 0 and nothing is copied.  `overflow` may be NULL. */
void fkv_oracle_staging_transfer(uint8_t *staging, int64_t staging_stride, uint64_t *comp_sizes,
                                 uint8_t *cpu, int64_t chunk_capacity, int32_t *overflow,
                                 int64_t cpu_kv_stride, int64_t cpu_layer_stride,
                                 int64_t cpu_block_stride, const int64_t *cpu_ids,
                                 uint32_t *size_table, int64_t table_block_stride,
                                 int64_t table_layer_stride, int start_layer, int kv_dim,
                                 int num_blocks, int batch_start, int bsz, int is_write_cpu) {
  for (int64_t i = 0; i < bsz; ++i) {
    const int64_t g = (int64_t)batch_start + i;
    const int64_t layer = g / ((int64_t)kv_dim * num_blocks);
    const int64_t kv = (g % ((int64_t)kv_dim * num_blocks)) / num_blocks;
    const int64_t b = g % num_blocks;
    uint8_t *slot = cpu + (layer + start_layer) * cpu_layer_stride + kv * cpu_kv_stride +
                    cpu_ids[b] * cpu_block_stride;
    uint32_t *entry = size_table + cpu_ids[b] * table_block_stride +
                      (start_layer + layer) * table_layer_stride + kv;
    uint8_t *payload = staging + i * staging_stride;
    if (is_write_cpu) {
      const uint64_t sz = comp_sizes[i];
      if (sz > (uint64_t)chunk_capacity) {
        if (overflow)
          ++*overflow;
        *entry = 0;
        continue;
      }
      *entry = (uint32_t)sz;
      memcpy(slot, payload, (size_t)sz);
    } else {
      const uint64_t sz = *entry;
      if (sz > (uint64_t)staging_stride) {
        if (overflow)
          ++*overflow;
        comp_sizes[i] = 0;
        continue;
      }
      comp_sizes[i] = sz;
      memcpy(payload, slot, (size_t)sz);
    }
  }
}

/* csrc/compression/common/staging_transfer.cuh:103-122 (build_gpu_chunk_ptrs_kernel):
 * out[i] = ptr_at(start_layer + layer, kv, gpu_ids[b]) with the same numbering. */
int fkv_oracle_chunk_ptrs(uint64_t *out, int backend, const uint64_t *tensor_ptrs,
                          int64_t num_layers_total, int64_t gpu_kv_stride,
                          int64_t gpu_block_stride, int64_t gpu_layer_stride,
                          const int64_t *gpu_ids, int start_layer, int kv_dim, int num_blocks,
                          int batch_start, int bsz) {
  if (backend < 0 || backend > 2)
    return -1;
  for (int64_t i = 0; i < bsz; ++i) {
    const int64_t g = (int64_t)batch_start + i;
    const int64_t layer = g / ((int64_t)kv_dim * num_blocks);
    const int64_t kv = (g % ((int64_t)kv_dim * num_blocks)) / num_blocks;
    const int64_t b = g % num_blocks;
    out[i] = fkv_oracle_chunk_addr(backend, tensor_ptrs, num_layers_total, gpu_kv_stride,
                                   gpu_block_stride, gpu_layer_stride, start_layer + layer, kv,
                                   gpu_ids[b]);
  }
  return 0;
}
