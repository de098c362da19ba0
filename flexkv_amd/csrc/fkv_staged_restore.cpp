// Layer-by-layer restore through the copy engines.
//
// The kernel path reads host memory from the compute units.  That reaches the
// link rate, but the requests it keeps in flight sit in the same memory queues
// as those of the engine's own kernels, which run measurably slower next to it
// (a fused-attention chain sized to the restore: 38 ms alone, 56 ms next to a
// 41 ms restore).  A copy-engine transfer costs the neighbours nothing (the same
// chain next to 2-D copies of the same bytes: 40.8 ms for both together), but the
// engines move contiguous runs or regular 2-D shapes only, one command each at
// about 10 us of overhead.  So where the host blocks of a restore form few runs
// of consecutive block ids, each batch of layers goes
//     host rows --(one 2-D copy per run: width = the batch's bytes of a block,
//                  pitch = host block stride)--> dense staging buffer in HBM
//     staging   --(one launch of the gather/scatter kernel, HBM-bound, ~20 us for
//                  36 MiB)--> the engine's blocks
// on two streams: the copies of batch b+1 run while batch b is scattered.  The
// staging buffers form a small ring per (layer group, GPU); a buffer is reused
// once the scatter that read it has finished (event).  Small holes between runs
// are read along (their bytes cost less link time than one more command).
//
//
// Where the host blocks are scattered (a host pool after some churn hands out ids
// in no order), a command per run is too many.  Then host threads gather the rows
// of a batch into a pinned buffer first and ONE copy command moves the batch:
//     host rows --(host threads, streaming stores)--> pinned buffer
//               --(one 2-D copy of one row)--> staging buffer in HBM --(scatter)--> blocks
// The thread that launches the restore gathers batch b+1 (with its helpers) while
// the engine copies batch b; four threads gather 36 MiB of 72 KiB rows in 0.3 ms
// against 0.67 ms on the link.  This is the host->GPU half of SEGMENT_SCATTER
// (gather_from_cpu + one DMA, csrc/ce_transfer.cu:585-641, 645-812) under the
// per-layer loop of csrc/layerwise.cpp:1129-1257, pipelined instead of
// synchronised per (layer, kv).
//
// Replaces, for restores with few runs, the per-layer kernel launches of
// csrc/layerwise.cpp:1129-1257; related to SEGMENT_SCATTER of
// csrc/ce_transfer.cu:645-812, which stages in host memory instead.
#include "fkv_host_copy.h"
#include "fkv_internal.h"

#include <algorithm>
#include <cstring>
#include <thread>

namespace fkv {

void StagedRing::release() {
  for (uint8_t *b : buf)
    if (b && hipFree(b) != hipSuccess)
      (void)hipGetLastError();
  for (auto *set : {&copied, &freed})
    for (hipEvent_t e : *set)
      if (e && hipEventDestroy(e) != hipSuccess)
        (void)hipGetLastError();
  buf.clear();
  copied.clear();
  freed.clear();
  used.clear();
  cap = 0;
  next = 0;
}

void GatherRing::release() {
  for (uint8_t *b : buf)
    if (b && hipHostFree(b) != hipSuccess)
      (void)hipGetLastError();
  for (hipEvent_t e : read)
    if (e && hipEventDestroy(e) != hipSuccess)
      (void)hipGetLastError();
  buf.clear();
  read.clear();
  used.clear();
  cap = 0;
  next = 0;
}

namespace {

int pinned_prepare(GatherRing &ring, int slots, size_t bytes) {
  if ((int)ring.buf.size() == slots && ring.cap >= bytes)
    return FKV_OK;
  // Only called while nothing of an earlier restore is in flight.
  ring.release();
  ring.buf.assign(slots, nullptr);
  ring.read.assign(slots, nullptr);
  ring.used.assign(slots, false);
  size_t cap = (bytes + (2u << 20) - 1) & ~(size_t)((2u << 20) - 1);
  for (int k = 0; k < slots; ++k) {
    hipError_t e = hipHostMalloc(reinterpret_cast<void **>(&ring.buf[k]), cap, hipHostMallocDefault);
    if (e == hipSuccess)
      e = hipEventCreateWithFlags(&ring.read[k], kBookkeepingEvent);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      ring.release();
      return fail(FKV_ERR_RUNTIME, "gathered restore: cannot allocate %d pinned buffers of %zu MiB: %s",
                  slots, cap >> 20, hipGetErrorString(e));
    }
  }
  ring.cap = cap;
  stats().staging_bytes_host.fetch_add((uint64_t)cap * slots, std::memory_order_relaxed);
  return FKV_OK;
}

int ring_prepare(StagedRing &ring, int slots, size_t bytes) {
  if ((int)ring.buf.size() == slots && ring.cap >= bytes)
    return FKV_OK;
  // Only called while nothing of an earlier restore is in flight.
  ring.release();
  ring.buf.assign(slots, nullptr);
  ring.copied.assign(slots, nullptr);
  ring.freed.assign(slots, nullptr);
  ring.used.assign(slots, false);
  size_t cap = (bytes + (2u << 20) - 1) & ~(size_t)((2u << 20) - 1);
  for (int k = 0; k < slots; ++k) {
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&ring.buf[k]), cap);
    // Both events only order work.  `copied` stands behind copy-engine writes, which
    // pass no cache that a fence at the event would have to flush; the scatter
    // kernel that waits on it invalidates its caches when it starts, like any kernel.
    if (e == hipSuccess)
      e = hipEventCreateWithFlags(&ring.copied[k], kBookkeepingEvent);
    if (e == hipSuccess)
      e = hipEventCreateWithFlags(&ring.freed[k], kBookkeepingEvent);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      ring.release();
      return fail(FKV_ERR_RUNTIME, "staged restore: cannot allocate %d staging buffers of %zu MiB: %s",
                  slots, cap >> 20, hipGetErrorString(e));
    }
  }
  ring.cap = cap;
  stats().staging_bytes_device.fetch_add((uint64_t)cap * slots, std::memory_order_relaxed);
  return FKV_OK;
}

} // namespace

// The arithmetic of the choice, without a device: runs of consecutive host block ids,
// which holes between them are read along, and whether the copy engines are worth it.
// `row_bytes` = bytes of one host block that a batch moves, `pieces` = copy commands
// per run and batch.  Returns false when the restore stays on the kernel path.
bool staged_layout(const int64_t *cpu_ids, int num_blocks, int64_t row_bytes, int pieces,
                   const fkv_launch_policy &pol, std::vector<StagedPlan::Seg> *segs,
                   int64_t *total_rows_out, int free_commands = 0) {
  segs->clear();
  *total_rows_out = 0;
  if (pol.staged_restore == 0 || num_blocks <= 0 || row_bytes <= 0 || pieces < 1)
    return false;
  std::vector<int64_t> ids(cpu_ids, cpu_ids + num_blocks);
  std::sort(ids.begin(), ids.end());
  ids.erase(std::unique(ids.begin(), ids.end()), ids.end());
  struct Hole {
    int64_t rows;
    size_t after; // index into ids of the last block before the hole
  };
  std::vector<Hole> holes;
  for (size_t k = 0; k + 1 < ids.size(); ++k)
    if (ids[k + 1] != ids[k] + 1)
      holes.push_back(Hole{ids[k + 1] - ids[k] - 1, k});
  // Holes are read along, smallest first, while each stays below the bridge size
  // and all together below the allowed share of the useful bytes.
  const double useful = (double)ids.size() * (double)row_bytes;
  const double max_waste = useful * pol.staged_overhead_pct / 100.0;
  std::vector<size_t> order(holes.size());
  for (size_t k = 0; k < order.size(); ++k)
    order[k] = k;
  std::stable_sort(order.begin(), order.end(),
                   [&](size_t x, size_t y) { return holes[x].rows < holes[y].rows; });
  std::vector<bool> bridged(holes.size(), false);
  double waste = 0;
  int64_t extra_rows = 0;
  for (size_t k : order) {
    const double bytes = (double)holes[k].rows * (double)row_bytes;
    if (bytes > (double)pol.staged_bridge_kb * 1024 || waste + bytes > max_waste)
      break;
    bridged[k] = true;
    waste += bytes;
    extra_rows += holes[k].rows;
  }
  int64_t nsegs = 1;
  for (size_t k = 0; k < holes.size(); ++k)
    nsegs += bridged[k] ? 0 : 1;
  const int64_t total_rows = (int64_t)ids.size() + extra_rows;
  if (total_rows * row_bytes > (int64_t)pol.staged_max_mb << 20)
    return false;
  if (pol.staged_restore == 1 && nsegs * pieces > free_commands) {
    // the copy commands of a batch against the batch's time on the link
    const double batch_us = useful / (std::max(1, pol.link_gbps_estimate) * 1e3);
    if ((double)(nsegs * pieces) * pol.staged_copy_overhead_us >
        batch_us * pol.staged_overhead_pct / 100.0)
      return false;
  }
  if (nsegs * pieces > 4096) // a batch of thousands of commands is never the better way
    return false;
  segs->reserve((size_t)nsegs);
  StagedPlan::Seg cur{ids[0], 1, 0};
  size_t h = 0;
  for (size_t k = 0; k + 1 < ids.size(); ++k) {
    if (ids[k + 1] == ids[k] + 1) {
      cur.rows += 1;
      continue;
    }
    if (bridged[h]) {
      cur.rows += (int32_t)(ids[k + 1] - ids[k]);
    } else {
      segs->push_back(cur);
      cur = StagedPlan::Seg{ids[k + 1], 1, cur.row0 + cur.rows};
    }
    ++h;
  }
  segs->push_back(cur);
  *total_rows_out = total_rows;
  return true;
}

int gather_threads_of(const fkv_launch_policy &pol) {
  const int cores = (int)std::thread::hardware_concurrency();
  const int most = cores > 1 ? cores - 1 : 1;
  return std::max(1, std::min(pol.gather_threads, most));
}

// Per piece a gathering thread pays a call, an alignment head and a fence on top of
// the bytes; only matters for rows cut into many small pieces.
constexpr double kGatherPieceNs = 50.0;

int staged_route(const int64_t *cpu_ids, int num_blocks, int64_t row_bytes, int pieces,
                 const fkv_launch_policy &pol, std::vector<StagedPlan::Seg> *segs,
                 int64_t *total_rows, int free_commands) {
  if (staged_layout(cpu_ids, num_blocks, row_bytes, pieces, pol, segs, total_rows, free_commands))
    return kRouteRuns;
  segs->clear();
  *total_rows = 0;
  if (pol.staged_gather == 0 || num_blocks <= 0 || row_bytes <= 0 || pieces < 1)
    return kRouteKernel;
  const double bytes = (double)num_blocks * (double)row_bytes;
  if (bytes > (double)((int64_t)pol.staged_max_mb << 20))
    return kRouteKernel;
  if (pol.staged_gather == 1) {
    const double link_us = bytes / (double)std::max(1, pol.model_link_mbps); // B / (MB/s) = us
    // the one copy command of a batch against the batch's time on the link
    if ((double)pol.staged_copy_overhead_us > link_us * pol.staged_overhead_pct / 100.0)
      return kRouteKernel;
    // the gather of batch b+1 has to fit, with room, into the copy of batch b
    const int threads = gather_threads_of(pol);
    const double gather_us =
        bytes / ((double)threads * (double)std::max(1, pol.model_gather_thread_mbps)) +
        (double)num_blocks * pieces * kGatherPieceNs / 1e3 / threads;
    if (gather_us > 0.8 * link_us)
      return kRouteKernel;
  }
  *total_rows = num_blocks;
  return kRouteGathered;
}

// Staging row of host block `id`: the last run whose first id is <= id.
int64_t staged_row_of(const std::vector<StagedPlan::Seg> &segs, int64_t id) {
  size_t lo = 0, hi = segs.size();
  while (hi - lo > 1) {
    const size_t mid = (lo + hi) / 2;
    if (segs[mid].first_id <= id)
      lo = mid;
    else
      hi = mid;
  }
  return segs[lo].row0 + (id - segs[lo].first_id);
}

int staged_plan_build(const fkv_transfer_desc &d, int batch_layers, StagedRing &ring,
                      GatherRing &pinned, hipStream_t scatter_stream, StagedPlan *out,
                      bool host_visible, bool kernel_allowed, bool several_gpus) {
  *out = StagedPlan{};
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  // the choice prices copy commands and gather passes against this device's link
  fkv_launch_policy pol = policy_of_seeded(device);
  if (!host_visible) // a pageable pool: the copy engines cannot take its rows, host threads can
    pol.staged_restore = 0;
  // Rows gathered by host threads are for groups of one GPU, unless the policy says 3: the
  // launching thread would gather for one GPU after the other (the same rows again where
  // the ranks share their KV), and the route has not run on several devices.
  if (pol.staged_gather == 3)
    pol.staged_gather = 2;
  else if (several_gpus)
    pol.staged_gather = 0;
  if ((pol.staged_restore == 0 && pol.staged_gather == 0) || d.num_blocks <= 0 ||
      d.num_layers <= 0 || batch_layers < 1)
    return FKV_OK;
  const int nl = std::min(batch_layers, d.num_layers);
  const int lk = nl * d.kv_dim;
  if (lk > kCopyMaxLK)
    return FKV_OK;
  // which chunks of one host block are adjacent
  const bool kv_adjacent = d.kv_dim == 1 || d.cpu_kv_stride == d.chunk_size;
  const bool layers_adjacent = kv_adjacent && d.cpu_layer_stride == d.kv_dim * d.chunk_size;
  out->kind = layers_adjacent ? 0 : kv_adjacent ? 1 : 2;
  const int64_t batch_row_bytes = (int64_t)lk * d.chunk_size; // of one block, all pieces
  const int pieces = out->kind == 0 ? 1 : out->kind == 1 ? nl : lk;
  int64_t total_rows = 0;
  // Asked for on the copy engine, the alternative to a staged batch is not a kernel launch but
  // a copy-engine strategy, which issues at least as many copy commands and a compaction
  // launch besides (46-56 us a layer at the small and medium scale of the notify
  // microbenchmark, against 15-28 us staged): few commands are always worth it there, and
  // more while they cost no more than the bytes themselves.
  int free_commands = 0;
  if (!kernel_allowed) {
    free_commands = 4;
    pol.staged_overhead_pct = std::max(pol.staged_overhead_pct, 100);
  }
  out->route = staged_route(d.cpu_block_ids, d.num_blocks, batch_row_bytes, pieces, pol, &out->segs,
                            &total_rows, free_commands);
  if (out->route == kRouteKernel)
    return FKV_OK;
  const bool gathered = out->route == kRouteGathered;
  const int64_t slot_bytes = total_rows * batch_row_bytes;
  out->total_rows = (int32_t)total_rows;
  out->max_lk = lk;
  out->batch_layers = nl;
  out->kv_dim = d.kv_dim;
  out->chunk = d.chunk_size;
  out->cpu_kv_stride = d.cpu_kv_stride;
  out->cpu_layer_stride = d.cpu_layer_stride;
  out->cpu_block_stride = d.cpu_block_stride;
  out->host0 = static_cast<const uint8_t *>(d.cpu_ptr) + d.cpu_startoff_inside_chunks;
  out->num_blocks = d.num_blocks;

  // Whatever the set-up lacks from here on (device or pinned memory, plan memory), the
  // kernel path needs none of it: the restore goes that way and the call succeeds.
  auto kernel_path_instead = [&]() {
    clear_error();
    out->route = kRouteKernel;
    return FKV_OK;
  };
  if (ring_prepare(ring, pol.staged_ring, (size_t)slot_bytes) != FKV_OK)
    return kernel_path_instead();
  if (gathered && pinned_prepare(pinned, pol.gather_ring, (size_t)slot_bytes) != FKV_OK)
    return kernel_path_instead();
  const int slots = (int)ring.buf.size();
  const size_t tab = (size_t)slots * lk * 8, rows_bytes = gathered ? 0 : (size_t)d.num_blocks * 8;
  PlanSlot *slot = plan_acquire(device, tab + rows_bytes);
  if (!slot)
    return kernel_path_instead();
  uint8_t *h = plan_host(slot);
  uint64_t *bases = reinterpret_cast<uint64_t *>(h);
  // staging layout of a batch: runs [piece][row][chunks of the piece]; gathered
  // [position][chunks of the batch]
  const int m = out->kind == 0 ? lk : out->kind == 1 ? d.kv_dim : 1; // chunks per piece (full batch)
  for (int k = 0; k < slots; ++k)
    for (int i = 0; i < lk; ++i) {
      // kind 0 has one piece whatever the batch length: chunk i of a row sits at i * chunk
      const uint64_t piece_off =
          gathered || out->kind == 0
              ? 0
              : (uint64_t)(i / m) * (uint64_t)total_rows * (uint64_t)(m * d.chunk_size);
      bases[(size_t)k * lk + i] = (uint64_t)(uintptr_t)ring.buf[k] + piece_off +
                                  (uint64_t)(gathered ? i : i % m) * (uint64_t)d.chunk_size;
    }
  if (gathered) {
    out->host_ids.assign(d.cpu_block_ids, d.cpu_block_ids + d.num_blocks);
    out->first_by_kernel = pol.gather_first_by_kernel != 0 && host_visible && kernel_allowed;
  } else {
    int64_t *rows = reinterpret_cast<int64_t *>(h + tab);
    for (int pos = 0; pos < d.num_blocks; ++pos)
      rows[pos] = staged_row_of(out->segs, d.cpu_block_ids[pos]);
  }
  uint8_t *dv = nullptr;
  if (plan_publish(slot, tab + rows_bytes, /*mirror=*/true, scatter_stream, &dv) != FKV_OK) {
    plan_release(slot, scatter_stream, false);
    return kernel_path_instead();
  }
  out->slot = slot;
  out->base_tables = reinterpret_cast<const uint64_t *>(dv);
  out->stage_rows = gathered ? nullptr : reinterpret_cast<const int64_t *>(dv + tab);
  out->usable = true;
  ring.idle_calls = 0;
  ring.touched = true;
  if (gathered) {
    pinned.idle_calls = 0;
    pinned.touched = true;
  }
  return FKV_OK;
}

namespace {

// Staging buffer k -> the engine's blocks, layers [l0, l0 + lk / kv_dim) of the plan.
int staged_scatter(const StagedPlan &sp, StagedRing &ring, const KernelPlan &kp, int k, int l0,
                   int lk, int64_t stride_src, hipStream_t scatter_stream) {
  FKV_HIP_TRY(hipStreamWaitEvent(scatter_stream, ring.copied[k], 0));
  CopyKernelArgs a{};
  a.base_src = sp.base_tables + (size_t)k * sp.max_lk;
  a.base_dst = kp.gpu_base + (size_t)l0 * kp.kv_dim;
  a.ids_src = sp.stage_rows; // nullptr: row of position p is p
  a.ids_dst = kp.gpu_ids;
  a.stride_src = stride_src;
  a.stride_dst = kp.gpu_block_stride;
  a.chunk_bytes = sp.chunk;
  a.num_blocks = sp.num_blocks;
  a.lk = lk;
  a.vec = kp.vec; // staging addresses are multiples of the chunk size off a 2 MiB-aligned buffer
  a.nt_store = 1;
  a.xcd_mask = 0;
  const fkv_launch_policy pol = policy_of(kp.device);
  a.unroll = pol.hbm_unroll;
  // Small workgroups: the launch is short (one 8 KiB slice per wavefront for a 36 MiB batch)
  // and runs next to the engine's kernels, where a workgroup of 1024 lanes waits for a CU
  // with room for all of it.
  FKV_TRY(launch_copy_kernel(a, pol.hbm_workgroups, pol.staged_scatter_threads, scatter_stream));
  FKV_HIP_TRY(hipEventRecord(ring.freed[k], scatter_stream));
  ring.used[k] = true;
  stats().staged_batches.fetch_add(1, std::memory_order_relaxed);
  return FKV_OK;
}

} // namespace

int staged_launch(const StagedPlan &sp, StagedRing &ring, const KernelPlan &kp, int l0, int nl,
                  hipStream_t dma_stream, hipStream_t scatter_stream) {
  if (!sp.usable || sp.route != kRouteRuns || nl < 1 || nl > sp.batch_layers ||
      nl * sp.kv_dim > sp.max_lk)
    return fail(FKV_ERR_RUNTIME, "staged restore: batch of %d layers does not fit its plan", nl);
  const int k = ring.next;
  ring.next = (ring.next + 1) % (int)ring.buf.size();
  if (ring.used[k]) // the scatter that read this buffer last
    FKV_HIP_TRY(hipStreamWaitEvent(dma_stream, ring.freed[k], 0));
  const int lk = nl * sp.kv_dim;
  const int m = sp.kind == 0 ? lk : sp.kind == 1 ? sp.kv_dim : 1;
  const int pieces = lk / m;
  const int64_t w = (int64_t)m * sp.chunk;
  uint64_t copies = 0;
  for (int p = 0; p < pieces; ++p) {
    const int i0 = p * m;
    const int64_t layer = l0 + i0 / sp.kv_dim, kv = i0 % sp.kv_dim;
    const uint8_t *src0 = sp.host0 + layer * sp.cpu_layer_stride + kv * sp.cpu_kv_stride;
    uint8_t *dst0 = ring.buf[k] + (sp.kind == 0 ? 0 : (int64_t)p * sp.total_rows * w);
    for (const StagedPlan::Seg &s : sp.segs) {
      const uint8_t *src = src0 + s.first_id * sp.cpu_block_stride;
      uint8_t *dst = dst0 + (int64_t)s.row0 * w;
      // Always the 2-D call, also for one row or adjacent rows: the runtime hands 2-D
      // copies to the copy engines, while it is free to run hipMemcpyAsync between pinned
      // host and device memory as a kernel on the compute units (kernel traces show one
      // __amd_rocclr_copyBuffer launch per 1-D copy of any size, none for 2-D copies),
      // which is what this path exists to avoid.
      const size_t pitch = s.rows == 1 ? (size_t)w : (size_t)sp.cpu_block_stride;
      FKV_HIP_TRY(hipMemcpy2DAsync(dst, (size_t)w, src, pitch, (size_t)w, (size_t)s.rows,
                                   hipMemcpyHostToDevice, dma_stream));
      ++copies;
    }
  }
  FKV_HIP_TRY(hipEventRecord(ring.copied[k], dma_stream));
  stats().dma_copies.fetch_add(copies, std::memory_order_relaxed);
  return staged_scatter(sp, ring, kp, k, l0, lk, w, scatter_stream);
}

int gathered_launch(const StagedPlan &sp, StagedRing &ring, GatherRing &pinned, HostCrew &crew,
                    const KernelPlan &kp, int l0, int nl, hipStream_t dma_stream,
                    hipStream_t scatter_stream) {
  if (!sp.usable || sp.route != kRouteGathered || nl < 1 || nl > sp.batch_layers ||
      nl * sp.kv_dim > sp.max_lk)
    return fail(FKV_ERR_RUNTIME, "gathered restore: batch of %d layers does not fit its plan", nl);
  const int p = pinned.next;
  pinned.next = (pinned.next + 1) % (int)pinned.buf.size();
  if (pinned.used[p]) // the copy that read this buffer last
    FKV_HIP_TRY(hipEventSynchronize(pinned.read[p]));
  const int lk = nl * sp.kv_dim;
  const uint8_t *row0 = sp.host0 + (int64_t)l0 * sp.cpu_layer_stride;
  uint64_t busy_ns;
  if (sp.kind == 0)
    busy_ns = host_gather_rows(crew, pinned.buf[p], row0, sp.host_ids.data(), sp.num_blocks,
                               sp.cpu_block_stride, 1, 0, 1, 0, (int64_t)lk * sp.chunk);
  else if (sp.kind == 1)
    busy_ns = host_gather_rows(crew, pinned.buf[p], row0, sp.host_ids.data(), sp.num_blocks,
                               sp.cpu_block_stride, nl, sp.cpu_layer_stride, 1, 0,
                               (int64_t)sp.kv_dim * sp.chunk);
  else
    busy_ns = host_gather_rows(crew, pinned.buf[p], row0, sp.host_ids.data(), sp.num_blocks,
                               sp.cpu_block_stride, nl, sp.cpu_layer_stride, sp.kv_dim,
                               sp.cpu_kv_stride, sp.chunk);
  const int k = ring.next;
  ring.next = (ring.next + 1) % (int)ring.buf.size();
  if (ring.used[k]) // the scatter that read this buffer last
    FKV_HIP_TRY(hipStreamWaitEvent(dma_stream, ring.freed[k], 0));
  const size_t bytes = (size_t)sp.num_blocks * (size_t)lk * (size_t)sp.chunk;
  // a 2-D copy of one row: the runtime hands those to the copy engines (see staged_launch)
  FKV_HIP_TRY(hipMemcpy2DAsync(ring.buf[k], bytes, pinned.buf[p], bytes, bytes, 1,
                               hipMemcpyHostToDevice, dma_stream));
  FKV_HIP_TRY(hipEventRecord(pinned.read[p], dma_stream));
  pinned.used[p] = true;
  FKV_HIP_TRY(hipEventRecord(ring.copied[k], dma_stream));
  stats().dma_copies.fetch_add(1, std::memory_order_relaxed);
  stats().gathered_batches.fetch_add(1, std::memory_order_relaxed);
  stats().gather_busy_ns.fetch_add(busy_ns, std::memory_order_relaxed);
  return staged_scatter(sp, ring, kp, k, l0, lk, (int64_t)lk * sp.chunk, scatter_stream);
}

} // namespace fkv

extern "C" int fkv_staged_restore_plan(const int64_t *cpu_block_ids, int32_t num_blocks,
                                       int64_t row_bytes, int32_t pieces,
                                       const fkv_launch_policy *policy, int32_t *staged,
                                       int32_t *num_runs, int64_t *total_rows,
                                       fkv_staged_run *runs, int32_t run_capacity,
                                       int64_t *row_of_position) try {
  using namespace fkv;
  clear_error();
  if (!policy || !staged || num_blocks < 0 || (num_blocks > 0 && !cpu_block_ids))
    return fail(FKV_ERR_INVALID_ARG, "fkv_staged_restore_plan: bad arguments");
  std::vector<StagedPlan::Seg> segs;
  int64_t rows = 0;
  const fkv_launch_policy pol = policy_sanitized(*policy);
  *staged = staged_route(cpu_block_ids, num_blocks, row_bytes, pieces, pol, &segs, &rows);
  if (num_runs)
    *num_runs = (int32_t)segs.size();
  if (total_rows)
    *total_rows = rows;
  if (runs)
    for (int i = 0; i < (int)segs.size() && i < run_capacity; ++i)
      runs[i] = fkv_staged_run{segs[i].first_id, segs[i].rows, segs[i].row0};
  if (row_of_position && *staged == kRouteRuns)
    for (int pos = 0; pos < num_blocks; ++pos)
      row_of_position[pos] = staged_row_of(segs, cpu_block_ids[pos]);
  if (row_of_position && *staged == kRouteGathered)
    for (int pos = 0; pos < num_blocks; ++pos)
      row_of_position[pos] = pos;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

namespace fkv {

void staged_plan_release(StagedPlan *sp, hipStream_t scatter_stream) {
  if (sp->slot)
    plan_release(sp->slot, scatter_stream, false);
  sp->slot = nullptr;
  sp->usable = false;
}

} // namespace fkv
