// Variable-size chunks between a dense device staging buffer and the host cache,
// with a size table on the host side, and the table of chunk addresses a batched
// codec works on.  The codec-independent device half of a compressed transfer:
// replaces staging_transfer_kernel<is_write_cpu> and build_gpu_chunk_ptrs_kernel<Type>
// of the reference (csrc/compression/common/staging_transfer.cuh:16-122; callers
// csrc/compression/ans/nvcomp_ans.cu:355-409, 455-500).  The codec itself (nvcomp
// ANS) has no counterpart here.
//
// Chunk i of a batch is chunk g = batch_start + i of the call, numbered layer-major,
// then K/V, then block position:  layer = g / (kv_dim * num_blocks),
// kv = (g % (kv_dim * num_blocks)) / num_blocks, b = g % num_blocks.  Its payload
// sits at staging + i * staging_stride, its host slot at
// cpu + (start_layer + layer) * layer_stride + kv * kv_stride + cpu_ids[b] * block_stride,
// its size at size_table[cpu_ids[b] * table_block_stride +
// (start_layer + layer) * table_layer_stride + kv].
//
// One wavefront per chunk at a time (the reference: one 32-lane warp), 8 vectors of
// 16 bytes in flight per lane, sizes of any byte count (16-byte body + byte tail).
// The copy crosses the host link, so the launch has the shape of the link-bound
// gather/scatter kernel: single-wavefront workgroups, a few dozen of them.
#include "fkv_internal.h"

#include <algorithm>
#include <cstring>

namespace fkv {
namespace {

struct StagingKernelArgs {
  uint8_t *staging;
  int64_t staging_stride;
  uint64_t *comp_sizes;       // device, [bsz]
  uint8_t *cpu;               // device-visible alias of the host cache
  int64_t chunk_capacity;
  int32_t *overflow;          // device counter or nullptr
  int64_t cpu_kv_stride, cpu_layer_stride, cpu_block_stride;
  const int64_t *cpu_ids;     // device-visible, [num_blocks]
  uint32_t *size_table;       // device-visible alias of the host size table
  int64_t table_block_stride, table_layer_stride; // in entries
  int32_t start_layer, kv_dim, num_blocks, batch_start, bsz;
};

typedef unsigned int vec16 __attribute__((ext_vector_type(4)));

// Copies `bytes` from src to dst with one wavefront; VEC16: both are 16-byte aligned.
template <bool VEC16, bool NTS>
__device__ __forceinline__ void wave_copy(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                          int64_t bytes, int lane) {
  int64_t done = 0;
  if (VEC16) {
    const vec16 *s = reinterpret_cast<const vec16 *>(src);
    vec16 *d = reinterpret_cast<vec16 *>(dst);
    const int64_t nvec = bytes / 16;
    constexpr int U = kCopyUnroll;
    for (int64_t v0 = 0; v0 < nvec; v0 += 64 * U) {
      // all loads of a slice before the first store; lanes beyond the end re-read the
      // last vector rather than branch around the load
      vec16 r[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t v = v0 + u * 64 + lane;
        r[u] = __builtin_nontemporal_load(s + (v < nvec ? v : nvec - 1));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t v = v0 + u * 64 + lane;
        if (v < nvec) {
          if (NTS)
            __builtin_nontemporal_store(r[u], d + v);
          else
            d[v] = r[u];
        }
      }
    }
    done = nvec * 16;
  }
  for (int64_t j = done + lane; j < bytes; j += 64)
    dst[j] = src[j];
}

template <bool WRITE_CPU, bool VEC16>
__global__ __launch_bounds__(kCopyBlockThreads) void fkv_staging_transfer_kernel(StagingKernelArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x / 64);
  const int64_t per_layer = (int64_t)a.kv_dim * a.num_blocks;
  // Where chunk i lives on the host side.
  auto locate = [&](int64_t i, uint8_t **slot, uint32_t **entry) {
    const int64_t g = (int64_t)a.batch_start + i;
    const int64_t layer = g / per_layer;
    const int64_t kv = (g % per_layer) / a.num_blocks;
    const int64_t b = g % a.num_blocks;
    const int64_t id = a.cpu_ids[b];
    *slot = a.cpu + (layer + a.start_layer) * a.cpu_layer_stride + kv * a.cpu_kv_stride +
            id * a.cpu_block_stride;
    *entry = a.size_table + id * a.table_block_stride +
             (a.start_layer + layer) * a.table_layer_stride + kv;
  };
  // The size of a chunk that is read comes out of host memory, a round trip over the
  // link: the entry of the wavefront's next chunk is asked for before the current
  // chunk is copied, so that it has arrived when it is needed.
  uint8_t *slot = nullptr;
  uint32_t *entry = nullptr;
  int64_t sz_next = 0;
  if (wave < a.bsz) {
    locate(wave, &slot, &entry);
    if (!WRITE_CPU)
      sz_next = (int64_t)__builtin_nontemporal_load(entry);
  }
  for (int64_t i = wave; i < a.bsz; i += nwaves) {
    uint8_t *cur_slot = slot;
    uint32_t *cur_entry = entry;
    int64_t sz = sz_next;
    if (i + nwaves < a.bsz) {
      locate(i + nwaves, &slot, &entry);
      if (!WRITE_CPU)
        sz_next = (int64_t)__builtin_nontemporal_load(entry);
    }
    uint8_t *payload = a.staging + i * a.staging_stride;
    if (WRITE_CPU) {
      sz = (int64_t)a.comp_sizes[i];
      if (sz > a.chunk_capacity) { // does not fit its host slot: counted, size 0 recorded
        if (lane == 0) {
          if (a.overflow)
            atomicAdd(a.overflow, 1);
          *cur_entry = 0;
        }
        continue;
      }
      if (lane == 0)
        *cur_entry = (uint32_t)sz;
      wave_copy<VEC16, false>(payload, cur_slot, sz, lane);
    } else {
      if (sz > a.staging_stride) { // a stale or corrupt entry must not overrun the staging slot
        if (lane == 0) {
          if (a.overflow)
            atomicAdd(a.overflow, 1);
          a.comp_sizes[i] = 0;
        }
        continue;
      }
      if (lane == 0)
        a.comp_sizes[i] = (uint64_t)sz;
      wave_copy<VEC16, true>(cur_slot, payload, sz, lane);
    }
  }
}

__global__ void fkv_chunk_ptrs_kernel(void **__restrict__ out, const uint64_t *__restrict__ base,
                                      const int64_t *__restrict__ ids, int64_t block_stride,
                                      int32_t kv_dim, int32_t num_blocks, int32_t batch_start,
                                      int32_t bsz) {
  const int64_t per_layer = (int64_t)kv_dim * num_blocks;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < bsz;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t g = (int64_t)batch_start + i;
    const int64_t layer = g / per_layer;
    const int64_t kv = (g % per_layer) / num_blocks;
    const int64_t b = g % num_blocks;
    out[i] = reinterpret_cast<void *>(base[layer * kv_dim + kv] + (uint64_t)(ids[b] * block_stride));
  }
}

} // namespace
} // namespace fkv

extern "C" {

int fkv_staging_transfer(const fkv_staging_transfer_desc *dp, void *stream_v) try {
  using namespace fkv;
  clear_error();
  if (!dp)
    return fail(FKV_ERR_INVALID_ARG, "fkv_staging_transfer: null descriptor");
  const fkv_staging_transfer_desc &d = *dp;
  if (d.bsz < 0 || d.batch_start < 0 || d.num_blocks < 1 || d.kv_dim < 1 || d.start_layer_id < 0 ||
      d.staging_stride <= 0 || d.chunk_capacity <= 0)
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_staging_transfer: bsz=%d batch_start=%d num_blocks=%d kv_dim=%d start_layer=%d "
                "staging_stride=%lld chunk_capacity=%lld",
                d.bsz, d.batch_start, d.num_blocks, d.kv_dim, d.start_layer_id,
                (long long)d.staging_stride, (long long)d.chunk_capacity);
  if (d.bsz == 0)
    return FKV_OK;
  if (!d.staging || !d.comp_sizes || !d.cpu_ptr || !d.cpu_block_ids || !d.size_table)
    return fail(FKV_ERR_INVALID_ARG, "fkv_staging_transfer: null pointer");
  for (int i = 0; i < d.num_blocks; ++i)
    if (d.cpu_block_ids[i] < 0)
      return fail(FKV_ERR_INVALID_ARG, "negative block id at position %d", i);
  DeviceGuard guard(d.device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", d.device);
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  hipStream_t stream = static_cast<hipStream_t>(stream_v);
  void *cpu_dev = nullptr, *table_dev = nullptr;
  if (hipHostGetDevicePointer(&cpu_dev, d.cpu_ptr, 0) != hipSuccess || !cpu_dev ||
      hipHostGetDevicePointer(&table_dev, d.size_table, 0) != hipSuccess || !table_dev) {
    (void)hipGetLastError();
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_staging_transfer: the host cache and the size table must be device-visible "
                "(pinned or registered)");
  }
  const size_t ids_bytes = (size_t)d.num_blocks * 8;
  PlanSlot *slot = plan_acquire(device, ids_bytes);
  if (!slot)
    return FKV_ERR_RUNTIME;
  PlanSlotHold hold{slot, stream};
  std::memcpy(plan_host(slot), d.cpu_block_ids, ids_bytes);
  uint8_t *dv = nullptr;
  FKV_TRY(plan_publish(slot, ids_bytes, /*mirror=*/true, stream, &dv));
  StagingKernelArgs a{};
  a.staging = static_cast<uint8_t *>(d.staging);
  a.staging_stride = d.staging_stride;
  a.comp_sizes = d.comp_sizes;
  a.cpu = static_cast<uint8_t *>(cpu_dev);
  a.chunk_capacity = d.chunk_capacity;
  a.overflow = d.overflow;
  a.cpu_kv_stride = d.cpu_kv_stride;
  a.cpu_layer_stride = d.cpu_layer_stride;
  a.cpu_block_stride = d.cpu_block_stride;
  a.cpu_ids = reinterpret_cast<const int64_t *>(dv);
  a.size_table = static_cast<uint32_t *>(table_dev);
  a.table_block_stride = d.size_table_block_stride;
  a.table_layer_stride = d.size_table_layer_stride;
  a.start_layer = d.start_layer_id;
  a.kv_dim = d.kv_dim;
  a.num_blocks = d.num_blocks;
  a.batch_start = d.batch_start;
  a.bsz = d.bsz;
  const uint64_t align = (uint64_t)(uintptr_t)a.staging | (uint64_t)a.staging_stride |
                         (uint64_t)(uintptr_t)a.cpu | (uint64_t)a.cpu_kv_stride |
                         (uint64_t)a.cpu_layer_stride | (uint64_t)a.cpu_block_stride;
  const bool vec16 = (align & 15u) == 0;
  const bool write_cpu = d.is_write_cpu != 0;
  const fkv_launch_policy pol = policy_of(device);
  const int cta = d.transfer_num_cta > 0 ? d.transfer_num_cta : default_num_cta(!write_cpu);
  // Reading from the host, a wavefront has one payload in flight and drains between
  // payloads, whose last slice is short: twice the workgroups of the fixed-size
  // kernel make up for it (16-29 KiB payloads: 45 GB/s with 16 wavefronts, 55.0 with
  // 24, 55.7 with 32).
  int grid = cta * (write_cpu ? pol.d2h_wg_per_cta : 2 * pol.h2d_wg_per_cta);
  const int threads = write_cpu ? pol.d2h_wg_threads : pol.h2d_wg_threads;
  grid = std::max(1, std::min(grid, (d.bsz + threads / 64 - 1) / (threads / 64)));
#define FKV_LAUNCH_STAGING(W, V)                                                              \
  hipLaunchKernelGGL((fkv_staging_transfer_kernel<W, V>), dim3(grid), dim3(threads), 0, stream, a)
  if (write_cpu && vec16)
    FKV_LAUNCH_STAGING(true, true);
  else if (write_cpu)
    FKV_LAUNCH_STAGING(true, false);
  else if (vec16)
    FKV_LAUNCH_STAGING(false, true);
  else
    FKV_LAUNCH_STAGING(false, false);
#undef FKV_LAUNCH_STAGING
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(FKV_ERR_RUNTIME, "staging transfer launch failed: %s", hipGetErrorString(e));
  stats().kernel_launches.fetch_add(1, std::memory_order_relaxed);
  if (d.sync)
    FKV_HIP_TRY(hipStreamSynchronize(stream));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_build_gpu_chunk_ptrs(const fkv_chunk_ptrs_desc *dp, void *stream_v) try {
  using namespace fkv;
  clear_error();
  if (!dp)
    return fail(FKV_ERR_INVALID_ARG, "fkv_build_gpu_chunk_ptrs: null descriptor");
  const fkv_chunk_ptrs_desc &d = *dp;
  if (d.backend != FKV_BACKEND_VLLM && d.backend != FKV_BACKEND_TRTLLM &&
      d.backend != FKV_BACKEND_SGLANG)
    return fail(FKV_ERR_RUNTIME, "Unsupported gpu_block_type: %d", d.backend);
  if (d.bsz < 0 || d.batch_start < 0 || d.num_blocks < 1 || d.kv_dim < 1 || d.start_layer_id < 0)
    return fail(FKV_ERR_INVALID_ARG, "fkv_build_gpu_chunk_ptrs: bsz=%d batch_start=%d num_blocks=%d "
                "kv_dim=%d start_layer=%d", d.bsz, d.batch_start, d.num_blocks, d.kv_dim,
                d.start_layer_id);
  if (d.bsz == 0)
    return FKV_OK;
  if (!d.out_ptrs || !d.gpu_tensor_ptrs || !d.gpu_block_ids)
    return fail(FKV_ERR_INVALID_ARG, "fkv_build_gpu_chunk_ptrs: null pointer");
  const int64_t per_layer = (int64_t)d.kv_dim * d.num_blocks;
  const int64_t first_layer = d.batch_start / per_layer;
  const int64_t last_layer = ((int64_t)d.batch_start + d.bsz - 1) / per_layer;
  const int64_t last_abs = d.start_layer_id + last_layer;
  const int64_t need = d.backend == FKV_BACKEND_TRTLLM ? 1
                       : d.backend == FKV_BACKEND_VLLM
                           ? last_abs + 1
                           : (int64_t)(d.kv_dim - 1) * d.num_layers_total + last_abs + 1;
  if (d.num_gpu_tensor_ptrs < need)
    return fail(FKV_ERR_INVALID_ARG, "fkv_build_gpu_chunk_ptrs: %d tensor pointers, %lld needed",
                d.num_gpu_tensor_ptrs, (long long)need);
  for (int i = 0; i < d.num_blocks; ++i)
    if (d.gpu_block_ids[i] < 0)
      return fail(FKV_ERR_INVALID_ARG, "negative block id at position %d", i);
  DeviceGuard guard(d.device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", d.device);
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  hipStream_t stream = static_cast<hipStream_t>(stream_v);
  // base addresses of the (layer, kv) planes the batch touches, engine addressing resolved
  const int nplanes = (int)(last_layer + 1) * d.kv_dim;
  const size_t tab = (size_t)nplanes * 8, ids_bytes = (size_t)d.num_blocks * 8;
  PlanSlot *slot = plan_acquire(device, tab + ids_bytes);
  if (!slot)
    return FKV_ERR_RUNTIME;
  PlanSlotHold hold{slot, stream};
  uint8_t *h = plan_host(slot);
  uint64_t *base = reinterpret_cast<uint64_t *>(h);
  for (int64_t l = 0; l <= last_layer; ++l)
    for (int kv = 0; kv < d.kv_dim; ++kv)
      base[l * d.kv_dim + kv] =
          l < first_layer ? 0
                          : gpu_chunk_addr(d.backend, d.gpu_tensor_ptrs, d.num_layers_total,
                                           d.gpu_kv_stride, d.gpu_block_stride, d.gpu_layer_stride,
                                           d.start_layer_id + l, kv, 0);
  std::memcpy(h + tab, d.gpu_block_ids, ids_bytes);
  uint8_t *dv = nullptr;
  int rc = plan_publish(slot, tab + ids_bytes, /*mirror=*/true, stream, &dv);
  if (rc == FKV_OK) {
    const int threads = 256;
    const int grid = std::max(1, std::min((d.bsz + threads - 1) / threads, 1024));
    hipLaunchKernelGGL(fkv_chunk_ptrs_kernel, dim3(grid), dim3(threads), 0, stream, d.out_ptrs,
                       reinterpret_cast<const uint64_t *>(dv),
                       reinterpret_cast<const int64_t *>(dv + tab), d.gpu_block_stride, d.kv_dim,
                       d.num_blocks, d.batch_start, d.bsz);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
      rc = fail(FKV_ERR_RUNTIME, "chunk pointer launch failed: %s", hipGetErrorString(e));
  }
  if (rc != FKV_OK)
    return rc;
  stats().kernel_launches.fetch_add(1, std::memory_order_relaxed);
  if (d.sync)
    FKV_HIP_TRY(hipStreamSynchronize(stream));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
