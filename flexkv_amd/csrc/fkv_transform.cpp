// Engine KV blocks <-> a dense device buffer, both sides in HBM.
//
// Takes the place of launch_layout_transform_kernel<Type> of the reference
// (csrc/gds/layout_transform.cu:26-108): chunk (layer, kv) of the i-th block of
// the call sits at  buffer + i*buffer_block_stride + layer*buffer_layer_stride +
// kv*buffer_kv_stride  in the buffer and at the engine's address of block
// gpu_block_ids[i] on the other side.  The reference launches 128-lane
// workgroups, one chunk each in turn, four per multiprocessor, and is called
// once per block.  Here the call is one launch of the library's gather/scatter
// kernel over all blocks, with enough wavefronts to keep every HBM channel busy.
#include "fkv_internal.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>

using namespace fkv;

extern "C" int fkv_layout_transform(const fkv_layout_transform_desc *dp, void *stream_v) try {
  clear_error();
  if (!dp)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layout_transform: null descriptor");
  const fkv_layout_transform_desc &d = *dp;
  if (d.backend != FKV_BACKEND_VLLM && d.backend != FKV_BACKEND_TRTLLM &&
      d.backend != FKV_BACKEND_SGLANG)
    return fail(FKV_ERR_RUNTIME, "Unsupported gpu_block_type: %d", d.backend);
  if (d.num_blocks < 0 || d.num_layers < 0 || d.start_layer_id < 0 || d.kv_dim < 1 ||
      d.chunk_size <= 0)
    return fail(FKV_ERR_INVALID_ARG,
                "layout transform: num_blocks=%d layers=[%d,+%d) kv_dim=%d chunk=%lld",
                d.num_blocks, d.start_layer_id, d.num_layers, d.kv_dim, (long long)d.chunk_size);
  if (d.num_blocks == 0 || d.num_layers == 0) // csrc/gds/layout_transform.cu:86
    return FKV_OK;
  if (!d.gpu_tensor_ptrs || !d.buffer_ptr || !d.gpu_block_ids)
    return fail(FKV_ERR_INVALID_ARG, "layout transform: null pointer");
  const int64_t last_layer = (int64_t)d.start_layer_id + d.num_layers - 1;
  const int64_t need = d.backend == FKV_BACKEND_TRTLLM ? 1
                       : d.backend == FKV_BACKEND_VLLM
                           ? last_layer + 1
                           : (int64_t)(d.kv_dim - 1) * d.num_layers_total + last_layer + 1;
  if (d.num_gpu_tensor_ptrs < need)
    return fail(FKV_ERR_INVALID_ARG, "layout transform: %d tensor pointers, %lld needed",
                d.num_gpu_tensor_ptrs, (long long)need);
  for (int i = 0; i < d.num_blocks; ++i)
    if (d.gpu_block_ids[i] < 0)
      return fail(FKV_ERR_INVALID_ARG, "negative block id at position %d", i);
  DeviceGuard guard(d.device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "layout transform: cannot select device %d", d.device);
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  hipStream_t stream = static_cast<hipStream_t>(stream_v);
  const fkv_launch_policy pol = policy_of(device);
  const int workgroups = pol.hbm_workgroups, threads = pol.hbm_wg_threads;
  const bool to_buffer = d.buffer_to_target == 0;
  const int pairs = d.num_layers * d.kv_dim;
  for (int p0 = 0; p0 < pairs; p0 += kCopyMaxLK) {
    const int lk = std::min(kCopyMaxLK, pairs - p0);
    const size_t tab = (size_t)lk * 8, ids = (size_t)d.num_blocks * 8;
    PlanSlot *slot = plan_acquire(device, 2 * tab + ids);
    if (!slot)
      return FKV_ERR_RUNTIME;
    PlanSlotHold hold{slot, stream};
    uint8_t *h = plan_host(slot);
    uint64_t *gbase = reinterpret_cast<uint64_t *>(h);
    uint64_t *bbase = reinterpret_cast<uint64_t *>(h + tab);
    uint64_t acc = (uint64_t)d.chunk_size | (uint64_t)d.gpu_block_stride |
                   (uint64_t)d.buffer_block_stride;
    for (int i = 0; i < lk; ++i) {
      const int l = (p0 + i) / d.kv_dim, kv = (p0 + i) % d.kv_dim;
      gbase[i] = gpu_chunk_addr(d.backend, d.gpu_tensor_ptrs, d.num_layers_total, d.gpu_kv_stride,
                                d.gpu_block_stride, d.gpu_layer_stride,
                                (int64_t)d.start_layer_id + l, kv, 0);
      bbase[i] = (uint64_t)(uintptr_t)d.buffer_ptr + (uint64_t)(l * d.buffer_layer_stride) +
                 (uint64_t)(kv * d.buffer_kv_stride);
      acc |= gbase[i] | bbase[i];
    }
    std::memcpy(h + 2 * tab, d.gpu_block_ids, ids);
    uint8_t *dv = nullptr;
    int rc = plan_publish(slot, 2 * tab + ids, /*mirror=*/true, stream, &dv);
    if (rc == FKV_OK) {
      CopyKernelArgs a{};
      const uint64_t *dg = reinterpret_cast<const uint64_t *>(dv);
      const uint64_t *db = reinterpret_cast<const uint64_t *>(dv + tab);
      const int64_t *dids = reinterpret_cast<const int64_t *>(dv + 2 * tab);
      a.base_src = to_buffer ? dg : db;
      a.base_dst = to_buffer ? db : dg;
      a.ids_src = to_buffer ? dids : nullptr;
      a.ids_dst = to_buffer ? nullptr : dids;
      a.stride_src = to_buffer ? d.gpu_block_stride : d.buffer_block_stride;
      a.stride_dst = to_buffer ? d.buffer_block_stride : d.gpu_block_stride;
      a.chunk_bytes = d.chunk_size;
      a.num_blocks = d.num_blocks;
      a.lk = lk;
      a.vec = common_vector_width(&acc, 1);
      a.nt_store = 1;
      a.unroll = pol.hbm_unroll;
      a.xcd_mask = 0;
      rc = launch_copy_kernel(a, workgroups, threads, stream);
    }
    if (rc != FKV_OK)
      return rc;
  }
  stats().staging_bytes_device.fetch_add((uint64_t)pairs * (uint64_t)d.num_blocks *
                                         (uint64_t)d.chunk_size);
  if (d.sync)
    FKV_HIP_TRY(hipStreamSynchronize(stream));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}
