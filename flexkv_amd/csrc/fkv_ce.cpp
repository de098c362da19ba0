// Copy-engine path: block-id analysis, strategy choice and the strategies.
//
// Replaces csrc/ce_transfer.cu of the reference.  The DMA work is
// hipMemcpyAsync / hipMemcpy2DAsync on the caller's stream; the device-side row
// gather/scatter that the reference delegates to ATen index_select /
// index_copy_ is the library's own copy kernel (fkv_kernels.hip) run with a
// full-chip grid, because that pass is HBM-bound, not link-bound.
//
// Differences from the reference that do not change which bytes move:
//   * the direct strategies (PER_BLOCK, CONTIG_DIRECT, SEGMENT_DIRECT,
//     GATHER_DIRECT, and the 2-D copy branches) never block the host: they
//     only enqueue work, so `sync == 0` callers (layerwise restore) stay
//     asynchronous.  The staging strategies still run host copies and therefore
//     return with their stream drained, as in the reference.
//   * GATHER_DIRECT bounds its device staging buffer and walks the block list
//     in groups instead of staging the whole transfer at once.
//   * host->GPU staging is double-buffered like GPU->host.
#include "fkv_host_copy.h"
#include "fkv_internal.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <unordered_map>

namespace fkv {
namespace {

struct Analysis {
  fkv_ce_analysis a{};
  std::vector<fkv_ce_segment> segs;
};

void analyze(const int64_t *gpu_ids, const int64_t *cpu_ids, int n, int64_t cpu_block_stride,
             int64_t chunk, int64_t gpu_block_stride, Analysis &out) {
  out.a.gpu_log_contig = 1;
  out.a.cpu_log_contig = 1;
  out.a.cpu_phys_contig = cpu_block_stride == chunk;
  out.a.gpu_phys_contig = gpu_block_stride == 0 || gpu_block_stride == chunk;
  out.a.num_segments = 0;
  out.a.reserved = 0;
  out.segs.clear();
  if (n <= 0)
    return;
  int run_start = 0;
  for (int k = 1; k < n; ++k) {
    const bool g_next = gpu_ids[k] == gpu_ids[k - 1] + 1;
    const bool c_next = cpu_ids[k] == cpu_ids[k - 1] + 1;
    out.a.gpu_log_contig &= (int)g_next;
    out.a.cpu_log_contig &= (int)c_next;
    if (!(g_next && c_next)) {
      out.segs.push_back({run_start, k - run_start});
      run_start = k;
    }
  }
  out.segs.push_back({run_start, n - run_start});
  out.a.num_segments = (int)out.segs.size();
}

int choose(const fkv_ce_analysis &a, const fkv_ce_config &cfg, int64_t chunk, bool h2d,
           bool full_block) {
  // strategies that view a chunk as int64 rows in the reference need chunk % 8 == 0
  const bool odd_chunk = chunk > 0 && (chunk % 8) != 0;
  const int many = odd_chunk ? FKV_CE_SEGMENT_SCATTER : FKV_CE_GATHER_SCATTER;
  if (cfg.is_blockfirst && !a.cpu_phys_contig && a.gpu_phys_contig) {
    if (!h2d && cfg.num_kv_heads == 1) {
      if (a.num_segments > cfg.segment_threshold)
        return many;
      if (!full_block)
        return FKV_CE_SEGMENT_SCATTER;
    }
    return FKV_CE_GATHER_DIRECT;
  }
  if (a.gpu_log_contig && a.cpu_log_contig && a.cpu_phys_contig && a.gpu_phys_contig)
    return FKV_CE_CONTIG_DIRECT;
  if (!a.gpu_phys_contig)
    return FKV_CE_GATHER_SCATTER;
  if (a.num_segments <= cfg.segment_threshold)
    return a.cpu_phys_contig ? FKV_CE_SEGMENT_DIRECT : FKV_CE_SEGMENT_SCATTER;
  return many;
}

// ---- cached staging memory, one set per (calling thread, device) ----------
struct DeviceStage {
  uint8_t *buf = nullptr;
  size_t cap = 0;
  hipEvent_t last_use = nullptr; // recorded after the last enqueued user
};
struct HostStage {
  uint8_t *buf = nullptr;
  size_t cap = 0;
};
struct StageSet {
  DeviceStage dev[2];
  HostStage host;
  hipEvent_t pingpong[2] = {nullptr, nullptr};
  // second DMA stream + the events that fork it off / join it back into the
  // caller's stream
  hipStream_t aux = nullptr;
  int device = -1; // of `aux`: the key this set is kept under
  hipEvent_t fork = nullptr, join = nullptr;
  // the per-buffer events of a pipelined GATHER_DIRECT: compaction launches stay on the
  // caller's stream, copies run on `aux`
  hipEvent_t kernel_done[2] = {nullptr, nullptr}, copied[2] = {nullptr, nullptr};
  // Creates what is missing; false (and nothing half-made in use) when the runtime refuses.
  bool ensure_fan() {
    if (aux && fork && join)
      return true;
    if ((!aux && pooled_stream_acquire(device, true, &aux) != hipSuccess) ||
        (!fork && hipEventCreateWithFlags(&fork, hipEventDisableTiming) != hipSuccess) ||
        (!join && hipEventCreateWithFlags(&join, hipEventDisableTiming) != hipSuccess)) {
      (void)hipGetLastError();
      return false;
    }
    return true;
  }
  bool ensure_pipeline() {
    if (!ensure_fan())
      return false;
    bool ok = true;
    for (int k = 0; k < 2 && ok; ++k) {
      ok = ok && (kernel_done[k] ||
                  hipEventCreateWithFlags(&kernel_done[k], hipEventDisableTiming) == hipSuccess);
      ok = ok && (copied[k] || hipEventCreateWithFlags(&copied[k], hipEventDisableTiming) == hipSuccess);
    }
    if (!ok)
      (void)hipGetLastError();
    return ok;
  }
  ~StageSet() {
    if (aux) { // to the next thread that stages on this device
      (void)hipStreamSynchronize(aux);
      pooled_stream_release(device, true, aux);
    }
    for (hipEvent_t e : {fork, join, kernel_done[0], kernel_done[1], copied[0], copied[1]})
      if (e)
        (void)hipEventDestroy(e);
    // Best effort: the thread is ending; errors (including a runtime that is
    // already shutting down) are ignored.
    for (auto &d : dev) {
      if (d.buf)
        (void)hipFree(d.buf);
      if (d.last_use)
        (void)hipEventDestroy(d.last_use);
    }
    if (host.buf)
      (void)hipHostFree(host.buf);
    for (auto &e : pingpong)
      if (e)
        (void)hipEventDestroy(e);
    (void)hipGetLastError();
  }
};
StageSet &stage_set(int device) {
  thread_local std::unordered_map<int, StageSet> sets;
  StageSet &s = sets[device];
  s.device = device;
  return s;
}

// Device staging of at least `bytes`; nullptr when HBM is exhausted (callers
// fall back to PER_BLOCK like the reference, csrc/ce_transfer.cu:149-169).
// Work already enqueued on other streams that still uses the buffer is ordered
// before `stream`.
uint8_t *device_stage(int device, int slot, size_t bytes, hipStream_t stream) {
  DeviceStage &s = stage_set(device).dev[slot];
  if (!s.last_use) {
    if (hipEventCreateWithFlags(&s.last_use, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      s.last_use = nullptr;
      return nullptr;
    }
  }
  if (bytes > s.cap) {
    if (s.buf) {
      (void)hipEventSynchronize(s.last_use);
      (void)hipFree(s.buf);
      s.buf = nullptr;
      s.cap = 0;
    }
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    s.buf = static_cast<uint8_t *>(p);
    s.cap = bytes;
  } else if (hipStreamWaitEvent(stream, s.last_use, 0) != hipSuccess) {
    // the order behind the buffer's last user is not optional: the host waits instead
    (void)hipGetLastError();
    if (hipEventSynchronize(s.last_use) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
  }
  return s.buf;
}
void device_stage_mark(int device, int slot, hipStream_t stream) {
  DeviceStage &s = stage_set(device).dev[slot];
  if (s.last_use && hipEventRecord(s.last_use, stream) != hipSuccess) {
    // no mark for the next user to wait for: the buffer is idle before this returns
    (void)hipGetLastError();
    if (hipStreamSynchronize(stream) != hipSuccess)
      (void)hipGetLastError();
  }
}

uint8_t *host_stage(int device, size_t bytes) {
  HostStage &s = stage_set(device).host;
  if (bytes > s.cap) {
    if (s.buf)
      (void)hipHostFree(s.buf);
    s.buf = nullptr;
    s.cap = 0;
    void *p = nullptr;
    if (hipHostMalloc(&p, bytes, hipHostMallocPortable) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    s.buf = static_cast<uint8_t *>(p);
    s.cap = bytes;
  }
  return s.buf;
}
hipEvent_t *pingpong_events(int device) {
  StageSet &s = stage_set(device);
  for (auto &e : s.pingpong)
    if (!e && hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      e = nullptr;
      return nullptr;
    }
  return s.pingpong;
}

// Status of a runtime call that the strategies issue in a loop.
int hip_rc(hipError_t e) {
  if (e == hipSuccess)
    return FKV_OK;
  (void)hipGetLastError();
  return fail(FKV_ERR_RUNTIME, "copy-engine path: %s", hipGetErrorString(e));
}

int current_device() {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return device;
}
size_t staging_cap_bytes() { return (size_t)policy_of(current_device()).ce_staging_mb << 20; }
bool fan_enabled() { return policy_of(current_device()).ce_two_streams != 0; }
bool pipeline_enabled() { return policy_of(current_device()).ce_two_streams == 1; }

// ---- one transfer's state ------------------------------------------------
struct Job {
  const fkv_transfer_desc &d;
  hipStream_t stream;
  int device;
  bool h2d;
  hipMemcpyKind kind;
  Analysis an;
  // While fanned out, independent DMAs alternate between the caller's stream and
  // a second stream: the fixed cost of one copy (about 10 us) then overlaps the
  // transfer time of the other.  Two streams measured best; more are slower.
  mutable hipStream_t aux = nullptr;
  mutable unsigned turn = 0;
  // Pipelined GATHER_DIRECT: every copy goes to this stream and none to the caller's,
  // which carries the compaction launches.
  mutable hipStream_t lane = nullptr;
  int64_t rect_min_bytes = -1; // from ce_rect_min_kb of the launch policy (run_ce_path)
  bool host_pinned = true;     // the host pool is pinned or registered memory (run_ce_path);
                               // the runtime stages 2-D copies of pageable memory synchronously
  // set by the strategies whose host thread waits for each copy (staging ping-pong)
  mutable bool host_waits = false;

  // Call when at least `copies` independent DMAs follow.  Work already on
  // `stream` is ordered before everything issued on the second stream.
  int fan_out(size_t copies) const {
    if (aux || copies < 8 || !fan_enabled())
      return FKV_OK;
    StageSet &s = stage_set(device);
    if (!s.ensure_fan())
      return FKV_OK; // stay on one stream
    FKV_HIP_TRY(hipEventRecord(s.fork, stream));
    FKV_HIP_TRY(hipStreamWaitEvent(s.aux, s.fork, 0));
    aux = s.aux;
    turn = 0;
    return FKV_OK;
  }
  // Everything issued since fan_out() is ordered before later work on `stream`.
  int fan_in() const {
    if (!aux)
      return FKV_OK;
    StageSet &s = stage_set(device);
    aux = nullptr;
    // Also after an error part-way: nothing issued on the second stream may outlive the
    // order of the caller's stream.  Where the runtime refuses the join, the host waits.
    if (hipEventRecord(s.join, s.aux) != hipSuccess ||
        hipStreamWaitEvent(stream, s.join, 0) != hipSuccess) {
      (void)hipGetLastError();
      FKV_HIP_TRY(hipStreamSynchronize(s.aux));
    }
    return FKV_OK;
  }
  hipStream_t next_stream() const {
    if (lane)
      return lane;
    return (aux && (turn++ & 1u)) ? aux : stream;
  }

  uint8_t *gpu(int layer_local, int kv, int64_t block) const {
    return reinterpret_cast<uint8_t *>(
        (uintptr_t)gpu_chunk_addr(d, (int64_t)d.start_layer_id + layer_local, kv, block));
  }
  uint8_t *cpu(int layer_local, int kv, int64_t block) const {
    return cpu_chunk_ptr(d, (int64_t)d.start_layer_id + layer_local, kv, block);
  }
  // The runtime is free to run a 1-D hipMemcpyAsync between pinned host and device
  // memory as a kernel on the compute units (one __amd_rocclr_copyBuffer launch per copy
  // in a kernel trace, whatever the size); 2-D copies it hands to the copy engines,
  // which leaves the compute units to the engine's own kernels.  A 2-D copy costs about
  // 9 us of fixed time against about 3 us (5 MiB copies: 51 against 56 GB/s; 2 MiB: 45
  // against 55 GB/s; 32 MiB and more: the same rate either way), and its completion
  // reaches a waiting host thread late (8 MiB copies with a host scatter behind each:
  // 10 against 44 GB/s).  So copies of `ce_rect_min_kb` and more go as 2-D copies of one
  // row unless a host thread waits for each of them; everything else as the runtime
  // likes.
  int dma(void *dst, const void *src, size_t bytes, hipMemcpyKind k) const {
    stats().dma_copies.fetch_add(1, std::memory_order_relaxed);
    // (a row of a 2-D copy, and its pitch, stay below 2 GiB)
    if (rect_min_bytes >= 0 && (int64_t)bytes >= rect_min_bytes && !host_waits &&
        bytes < ((size_t)1 << 31))
      FKV_HIP_TRY(hipMemcpy2DAsync(dst, bytes, src, bytes, bytes, 1, k, next_stream()));
    else
      FKV_HIP_TRY(hipMemcpyAsync(dst, src, bytes, k, next_stream()));
    return FKV_OK;
  }
  // gpu <-> cpu copy in the direction of the transfer
  int dma_dir(uint8_t *gpu_p, uint8_t *cpu_p, size_t bytes) const {
    return h2d ? dma(gpu_p, cpu_p, bytes, kind) : dma(cpu_p, gpu_p, bytes, kind);
  }
  int dma2d(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width,
            size_t height, hipMemcpyKind k) const {
    stats().dma_copies.fetch_add(1, std::memory_order_relaxed);
    FKV_HIP_TRY(hipMemcpy2DAsync(dst, dpitch, src, spitch, width, height, k, next_stream()));
    return FKV_OK;
  }
};

// csrc/ce_transfer.cu:196-229
int per_block(const Job &j) {
  const auto &d = j.d;
  FKV_TRY(j.fan_out((size_t)d.num_layers * d.kv_dim * d.num_blocks));
  int rc = FKV_OK;
  for (int i = 0; i < d.num_layers && rc == FKV_OK; ++i)
    for (int kv = 0; kv < d.kv_dim && rc == FKV_OK; ++kv)
      for (int b = 0; b < d.num_blocks && rc == FKV_OK; ++b)
        rc = j.dma_dir(j.gpu(i, kv, d.gpu_block_ids[b]), j.cpu(i, kv, d.cpu_block_ids[b]),
                       (size_t)d.chunk_size);
  int rc2 = j.fan_in();
  return rc != FKV_OK ? rc : rc2;
}

// csrc/ce_transfer.cu:235-267
int contig_direct(const Job &j) {
  const auto &d = j.d;
  const size_t run = (size_t)d.chunk_size * (size_t)d.num_blocks;
  FKV_TRY(j.fan_out((size_t)d.num_layers * d.kv_dim));
  int rc = FKV_OK;
  for (int i = 0; i < d.num_layers && rc == FKV_OK; ++i)
    for (int kv = 0; kv < d.kv_dim && rc == FKV_OK; ++kv)
      rc = j.dma_dir(j.gpu(i, kv, d.gpu_block_ids[0]), j.cpu(i, kv, d.cpu_block_ids[0]), run);
  int rc2 = j.fan_in();
  return rc != FKV_OK ? rc : rc2;
}

// csrc/ce_transfer.cu:271-309
int segment_direct(const Job &j) {
  const auto &d = j.d;
  FKV_TRY(j.fan_out((size_t)d.num_layers * d.kv_dim * j.an.segs.size()));
  int rc = FKV_OK;
  for (int i = 0; i < d.num_layers && rc == FKV_OK; ++i)
    for (int kv = 0; kv < d.kv_dim && rc == FKV_OK; ++kv)
      for (size_t si = 0; si < j.an.segs.size() && rc == FKV_OK; ++si) {
        const auto &s = j.an.segs[si];
        rc = j.dma_dir(j.gpu(i, kv, d.gpu_block_ids[s.start_k]),
                       j.cpu(i, kv, d.cpu_block_ids[s.start_k]),
                       (size_t)s.nr_blocks * (size_t)d.chunk_size);
      }
  int rc2 = j.fan_in();
  return rc != FKV_OK ? rc : rc2;
}

bool use_memcpy2d(const Job &j) {
  return j.d.ce.enable_memcpy2d && j.an.a.num_segments <= j.d.ce.segment_threshold;
}

// Host rows of (layer, kv): base of block 0 including all offsets.
uint8_t *cpu_row_base(const Job &j, int layer_local, int kv) { return j.cpu(layer_local, kv, 0); }

void rows_to_from_cpu(const Job &j, uint8_t *staging, int layer_local, int kv, bool to_cpu) {
  const auto &d = j.d;
  host_rows_copy(staging, cpu_row_base(j, layer_local, kv), d.cpu_block_ids, d.num_blocks,
                 d.cpu_block_stride, d.chunk_size, to_cpu, j.an.a.cpu_phys_contig != 0,
                 d.ce.gather_threads, d.ce.gather_nt != 0);
}

// Runs `produce(it, buf)` (enqueue the GPU->host DMA of iteration `it` into
// pinned buffer `buf`) and the host scatter of the previous iteration in
// alternation, so the scatter of (layer, kv) overlaps the DMA of the next one
// (csrc/ce_transfer.cu:713-810, 1023-1143).
template <typename Produce>
int d2h_pingpong(const Job &j, Produce produce) {
  const auto &d = j.d;
  const size_t layer_bytes = (size_t)d.num_blocks * (size_t)d.chunk_size;
  uint8_t *base = host_stage(j.device, 2 * layer_bytes);
  hipEvent_t *ev = pingpong_events(j.device);
  if (!base || !ev)
    return fail(FKV_ERR_RUNTIME, "cannot allocate %zu B of pinned staging", 2 * layer_bytes);
  stats().staging_bytes_host.fetch_add((uint64_t)layer_bytes * d.num_layers * d.kv_dim);
  uint8_t *bufs[2] = {base, base + layer_bytes};
  const int iters = d.num_layers * d.kv_dim;
  j.host_waits = true;
  for (int it = 0; it <= iters; ++it) {
    if (it < iters) {
      FKV_TRY(produce(it, bufs[it & 1]));
      FKV_HIP_TRY(hipEventRecord(ev[it & 1], j.stream));
    }
    if (it >= 1) {
      const int p = it - 1;
      FKV_HIP_TRY(hipEventSynchronize(ev[p & 1]));
      rows_to_from_cpu(j, bufs[p & 1], p / d.kv_dim, p % d.kv_dim, /*to_cpu=*/true);
    }
  }
  return FKV_OK;
}

// Host->GPU mirror image: gather (layer, kv) rows into one of two pinned
// buffers, `consume(it, buf)` enqueues the DMA(s) out of it; a buffer is reused
// only after the DMA that read it has finished.  Returns with the stream idle
// with respect to the staging buffers.
template <typename Consume>
int h2d_pingpong(const Job &j, Consume consume) {
  const auto &d = j.d;
  const size_t layer_bytes = (size_t)d.num_blocks * (size_t)d.chunk_size;
  uint8_t *base = host_stage(j.device, 2 * layer_bytes);
  hipEvent_t *ev = pingpong_events(j.device);
  if (!base || !ev)
    return fail(FKV_ERR_RUNTIME, "cannot allocate %zu B of pinned staging", 2 * layer_bytes);
  stats().staging_bytes_host.fetch_add((uint64_t)layer_bytes * d.num_layers * d.kv_dim);
  uint8_t *bufs[2] = {base, base + layer_bytes};
  const int iters = d.num_layers * d.kv_dim;
  j.host_waits = true;
  // The calling thread reads the host pool itself, now: what the caller enqueued on the stream
  // before this transfer (a put into the same host blocks, say) has to have landed, as it would
  // have for a copy in stream order.  Workers wait for every op, so their streams are idle here.
  if (iters > 0)
    FKV_HIP_TRY(hipStreamSynchronize(j.stream));
  for (int it = 0; it < iters; ++it) {
    if (it >= 2)
      FKV_HIP_TRY(hipEventSynchronize(ev[it & 1]));
    rows_to_from_cpu(j, bufs[it & 1], it / d.kv_dim, it % d.kv_dim, /*to_cpu=*/false);
    FKV_TRY(consume(it, bufs[it & 1]));
    FKV_HIP_TRY(hipEventRecord(ev[it & 1], j.stream));
  }
  for (int k = 0; k < 2 && k < iters; ++k)
    FKV_HIP_TRY(hipEventSynchronize(ev[k]));
  return FKV_OK;
}

// csrc/ce_transfer.cu:645-812
int segment_scatter(const Job &j) {
  const auto &d = j.d;
  if (use_memcpy2d(j)) {
    // one strided 2-D copy per (layer, kv, segment): rows = blocks of the segment
    FKV_TRY(j.fan_out((size_t)d.num_layers * d.kv_dim * j.an.segs.size()));
    int rc = FKV_OK;
    for (int i = 0; i < d.num_layers && rc == FKV_OK; ++i)
      for (int kv = 0; kv < d.kv_dim && rc == FKV_OK; ++kv)
        for (size_t si = 0; si < j.an.segs.size() && rc == FKV_OK; ++si) {
          const auto &s = j.an.segs[si];
          uint8_t *g = j.gpu(i, kv, d.gpu_block_ids[s.start_k]);
          uint8_t *c = j.cpu(i, kv, d.cpu_block_ids[s.start_k]);
          rc = j.h2d ? j.dma2d(g, (size_t)d.gpu_block_stride, c, (size_t)d.cpu_block_stride,
                               (size_t)d.chunk_size, (size_t)s.nr_blocks, j.kind)
                     : j.dma2d(c, (size_t)d.cpu_block_stride, g, (size_t)d.gpu_block_stride,
                               (size_t)d.chunk_size, (size_t)s.nr_blocks, j.kind);
        }
    int rc2 = j.fan_in();
    return rc != FKV_OK ? rc : rc2;
  }
  if (!j.h2d) {
    return d2h_pingpong(j, [&](int it, uint8_t *buf) {
      size_t off = 0;
      for (const auto &s : j.an.segs) {
        const size_t n = (size_t)s.nr_blocks * (size_t)d.chunk_size;
        FKV_TRY(j.dma(buf + off, j.gpu(it / d.kv_dim, it % d.kv_dim, d.gpu_block_ids[s.start_k]),
                      n, hipMemcpyDeviceToHost));
        off += n;
      }
      return (int)FKV_OK;
    });
  }
  return h2d_pingpong(j, [&](int it, uint8_t *buf) {
    size_t off = 0;
    for (const auto &s : j.an.segs) {
      const size_t n = (size_t)s.nr_blocks * (size_t)d.chunk_size;
      FKV_TRY(j.dma(j.gpu(it / d.kv_dim, it % d.kv_dim, d.gpu_block_ids[s.start_k]), buf + off, n,
                    hipMemcpyHostToDevice));
      off += n;
    }
    return (int)FKV_OK;
  });
}

} // namespace

// Device-side compaction.  `it` numbers the (layer, kv) pairs of the call:
// it = layer_local * kv_dim + kv.  Moves the chunks of pairs [it0, it0+nit) x
// block positions [p0, p0+np) between the engine's KV tensors and a packed
// device buffer laid out [np][nit][chunk] (blockfirst) or [nit][np][chunk].
int device_staging_copy(const fkv_transfer_desc &d, int it0, int nit, int p0, int np,
                        uint8_t *staging, bool blockfirst, bool to_staging,
                        hipStream_t stream) {
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  const fkv_launch_policy pol = policy_of(device);
  const int kStagingWorkgroups = pol.hbm_workgroups, kStagingThreads = pol.hbm_wg_threads;
  for (int b0 = 0; b0 < nit; b0 += kCopyMaxLK) {
    const int lk = std::min(kCopyMaxLK, nit - b0);
    const size_t tab = (size_t)lk * 8, ids = (size_t)np * 8;
    PlanSlot *slot = plan_acquire(device, 2 * tab + ids);
    if (!slot)
      return FKV_ERR_RUNTIME;
    PlanSlotHold hold{slot, stream};
    uint8_t *h = plan_host(slot);
    uint64_t *gbase = reinterpret_cast<uint64_t *>(h);
    uint64_t *sbase = reinterpret_cast<uint64_t *>(h + tab);
    const int64_t stg_stride = blockfirst ? (int64_t)nit * d.chunk_size : d.chunk_size;
    uint64_t acc = (uint64_t)d.chunk_size | (uint64_t)d.gpu_block_stride | (uint64_t)stg_stride;
    for (int i = 0; i < lk; ++i) {
      const int it = it0 + b0 + i;
      gbase[i] = gpu_chunk_addr(d, (int64_t)d.start_layer_id + it / d.kv_dim, it % d.kv_dim, 0);
      const uint64_t slot_in_stage = (uint64_t)(b0 + i);
      sbase[i] = (uint64_t)(uintptr_t)staging +
                 (blockfirst ? slot_in_stage * (uint64_t)d.chunk_size
                             : slot_in_stage * (uint64_t)np * (uint64_t)d.chunk_size);
      acc |= gbase[i] | sbase[i];
    }
    std::memcpy(h + 2 * tab, d.gpu_block_ids + p0, ids);
    uint8_t *dv = nullptr;
    int rc = plan_publish(slot, 2 * tab + ids, /*mirror=*/true, stream, &dv);
    if (rc == FKV_OK) {
      CopyKernelArgs a{};
      const uint64_t *dg = reinterpret_cast<const uint64_t *>(dv);
      const uint64_t *ds = reinterpret_cast<const uint64_t *>(dv + tab);
      const int64_t *dids = reinterpret_cast<const int64_t *>(dv + 2 * tab);
      a.base_src = to_staging ? dg : ds;
      a.base_dst = to_staging ? ds : dg;
      a.ids_src = to_staging ? dids : nullptr;
      a.ids_dst = to_staging ? nullptr : dids;
      a.stride_src = to_staging ? d.gpu_block_stride : stg_stride;
      a.stride_dst = to_staging ? stg_stride : d.gpu_block_stride;
      a.chunk_bytes = d.chunk_size;
      a.num_blocks = np;
      a.lk = lk;
      a.vec = common_vector_width(&acc, 1);
      a.nt_store = 1;
      a.unroll = pol.hbm_unroll;
      rc = launch_copy_kernel(a, kStagingWorkgroups, kStagingThreads, stream);
    }
    if (rc != FKV_OK)
      return rc;
  }
  stats().staging_bytes_device.fetch_add((uint64_t)nit * (uint64_t)np * (uint64_t)d.chunk_size);
  return FKV_OK;
}

namespace {

// Whole-block shortcut.  When the (layer, kv) chunks of a block are adjacent and
// in the same order on the GPU (single-tensor, block-major engine layout) as in
// the host block, the bytes of a block form one run on both sides: no staging
// and no per-(layer, kv) pass is needed, one DMA moves a block, or a run of
// adjacent blocks.  The reference stages such transfers through GATHER_SCATTER.
bool blocks_are_runs_on_both_sides(const Job &j) {
  const auto &d = j.d;
  if (d.backend != FKV_BACKEND_TRTLLM)
    return false;
  const bool gpu_dense = (d.kv_dim == 1 || d.gpu_kv_stride == d.chunk_size) &&
                         (d.num_layers == 1 || d.gpu_layer_stride == (int64_t)d.kv_dim * d.chunk_size);
  const bool cpu_dense = (d.kv_dim == 1 || d.cpu_kv_stride == d.chunk_size) &&
                         (d.num_layers == 1 || d.cpu_layer_stride == (int64_t)d.kv_dim * d.chunk_size);
  return gpu_dense && cpu_dense;
}

int block_runs_direct(const Job &j) {
  const auto &d = j.d;
  const size_t width = (size_t)d.num_layers * d.kv_dim * (size_t)d.chunk_size;
  const bool linear = (int64_t)width == d.gpu_block_stride && (int64_t)width == d.cpu_block_stride;
  FKV_TRY(j.fan_out(linear || d.ce.enable_memcpy2d ? j.an.segs.size() : (size_t)d.num_blocks));
  int rc = FKV_OK;
  for (size_t si = 0; si < j.an.segs.size() && rc == FKV_OK; ++si) {
    const auto &s = j.an.segs[si];
    uint8_t *g = j.gpu(0, 0, d.gpu_block_ids[s.start_k]);
    uint8_t *c = j.cpu(0, 0, d.cpu_block_ids[s.start_k]);
    const size_t rows = (size_t)s.nr_blocks;
    if (linear) {
      rc = j.dma_dir(g, c, rows * width);
    } else if (d.ce.enable_memcpy2d) {
      rc = j.h2d ? j.dma2d(g, (size_t)d.gpu_block_stride, c, (size_t)d.cpu_block_stride, width,
                           rows, j.kind)
                 : j.dma2d(c, (size_t)d.cpu_block_stride, g, (size_t)d.gpu_block_stride, width,
                           rows, j.kind);
    } else {
      for (size_t r = 0; r < rows && rc == FKV_OK; ++r)
        rc = j.dma_dir(g + r * (size_t)d.gpu_block_stride, c + r * (size_t)d.cpu_block_stride,
                       width);
    }
  }
  int rc2 = j.fan_in();
  return rc != FKV_OK ? rc : rc2;
}

// csrc/ce_transfer.cu:816-1179
int gather_scatter(const Job &j) {
  const auto &d = j.d;
  if (blocks_are_runs_on_both_sides(j))
    return block_runs_direct(j);
  const bool gpu_run = j.an.a.gpu_log_contig && j.an.a.gpu_phys_contig; // one linear GPU run
  const bool cpu_run = j.an.a.cpu_log_contig && j.an.a.cpu_phys_contig; // one linear host run
  const size_t layer_bytes = (size_t)d.num_blocks * (size_t)d.chunk_size;
  uint8_t *dev[2] = {nullptr, nullptr};
  if (!gpu_run) {
    for (int k = 0; k < 2; ++k) {
      dev[k] = device_stage(j.device, k, layer_bytes, j.stream);
      if (!dev[k])
        return per_block(j); // HBM exhausted, csrc/ce_transfer.cu:859
    }
  }
  auto mark_dev = [&] {
    if (!gpu_run)
      for (int k = 0; k < 2; ++k)
        device_stage_mark(j.device, k, j.stream);
  };
  const int iters = d.num_layers * d.kv_dim;
  auto pack = [&](int it, bool to_staging) {
    return device_staging_copy(d, it, 1, 0, d.num_blocks, dev[it & 1], false, to_staging,
                               j.stream);
  };

  if (use_memcpy2d(j)) {
    // device compaction + one strided 2-D DMA per segment, no host staging
    // (csrc/ce_transfer.cu:933-1018)
    int rc = FKV_OK;
    for (int it = 0; it < iters && rc == FKV_OK; ++it) {
      const int i = it / d.kv_dim, kv = it % d.kv_dim;
      uint8_t *packed = gpu_run ? j.gpu(i, kv, d.gpu_block_ids[0]) : dev[it & 1];
      const size_t pitch = gpu_run ? (size_t)d.gpu_block_stride : (size_t)d.chunk_size;
      if (!j.h2d && !gpu_run)
        rc = pack(it, true);
      for (size_t si = 0; si < j.an.segs.size() && rc == FKV_OK; ++si) {
        const auto &s = j.an.segs[si];
        uint8_t *c = j.cpu(i, kv, d.cpu_block_ids[s.start_k]);
        uint8_t *p = packed + (size_t)s.start_k * pitch;
        rc = j.h2d ? j.dma2d(p, pitch, c, (size_t)d.cpu_block_stride, (size_t)d.chunk_size,
                             (size_t)s.nr_blocks, j.kind)
                   : j.dma2d(c, (size_t)d.cpu_block_stride, p, pitch, (size_t)d.chunk_size,
                             (size_t)s.nr_blocks, j.kind);
      }
      if (rc == FKV_OK && j.h2d && !gpu_run)
        rc = pack(it, false);
    }
    mark_dev();
    return rc;
  }

  int rc = FKV_OK;
  if (!j.h2d) {
    auto produce = [&](int it, uint8_t *host_dst) {
      const uint8_t *src = dev[it & 1];
      if (gpu_run)
        src = j.gpu(it / d.kv_dim, it % d.kv_dim, d.gpu_block_ids[0]);
      else
        FKV_TRY(pack(it, true));
      return j.dma(host_dst, src, layer_bytes, hipMemcpyDeviceToHost);
    };
    if (cpu_run) {
      // destination rows are one linear run: DMA straight into place
      for (int it = 0; it < iters && rc == FKV_OK; ++it)
        rc = produce(it, j.cpu(it / d.kv_dim, it % d.kv_dim, d.cpu_block_ids[0]));
    } else {
      rc = d2h_pingpong(j, produce);
    }
  } else {
    auto consume = [&](int it, uint8_t *host_src) {
      if (gpu_run)
        return j.dma(j.gpu(it / d.kv_dim, it % d.kv_dim, d.gpu_block_ids[0]), host_src,
                     layer_bytes, hipMemcpyHostToDevice);
      FKV_TRY(j.dma(dev[it & 1], host_src, layer_bytes, hipMemcpyHostToDevice));
      return pack(it, false);
    };
    if (cpu_run) {
      for (int it = 0; it < iters && rc == FKV_OK; ++it)
        rc = consume(it, j.cpu(it / d.kv_dim, it % d.kv_dim, d.cpu_block_ids[0]));
    } else {
      rc = h2d_pingpong(j, consume);
    }
  }
  mark_dev();
  return rc;
}

// csrc/ce_transfer.cu:1183-1400.  Device staging holds whole host blocks
// ([block][layer*kv][chunk] == the block-first host layout), so every DMA moves
// at least one complete block and cpu-adjacent blocks merge into one DMA.
// Positions of a transfer in ascending order of their host block ids, and the ids in
// that order.  The device side of GATHER_DIRECT goes through the compaction kernel,
// which takes the GPU blocks in any order; staging them in host order makes every
// run of consecutive host blocks one copy command, however the GPU blocks lie
// (1024 pages into host blocks 0..1023: 8 commands of 1 GiB instead of 578).
struct HostOrder {
  std::vector<int64_t> gpu_ids, cpu_ids;
  std::vector<int> run_start; // first sorted position of every run, then the count as sentinel
};
HostOrder host_order(const fkv_transfer_desc &d) {
  HostOrder o;
  std::vector<int> pos(d.num_blocks);
  for (int i = 0; i < d.num_blocks; ++i)
    pos[i] = i;
  std::stable_sort(pos.begin(), pos.end(),
                   [&](int a, int b) { return d.cpu_block_ids[a] < d.cpu_block_ids[b]; });
  o.gpu_ids.resize(d.num_blocks);
  o.cpu_ids.resize(d.num_blocks);
  for (int i = 0; i < d.num_blocks; ++i) {
    o.gpu_ids[i] = d.gpu_block_ids[pos[i]];
    o.cpu_ids[i] = d.cpu_block_ids[pos[i]];
    if (i == 0 || o.cpu_ids[i] != o.cpu_ids[i - 1] + 1)
      o.run_start.push_back(i);
  }
  o.run_start.push_back(d.num_blocks);
  return o;
}

// How GATHER_DIRECT cuts a transfer into staging groups (also what the engine choice
// prices): copy commands per run of consecutive host blocks, blocks per group, and
// whether two half-size buffers alternate.
struct GatherDirectShape {
  size_t block_bytes = 0;
  bool full_block = false;
  size_t cap_blocks = 1, total_cmds = 0, group = 1;
  bool pipelined = false;
  bool enable_memcpy2d = false;
  bool rows_as_2d = true; // pinned host pool: runs of three rows and more go as one 2-D copy
  // Copy commands of `rows` consecutive host blocks: one where the bytes are one run
  // (whole blocks) or a 2-D copy takes the rows (asked for by the caller, or three rows
  // and more of a pinned pool: a layer-by-layer restore of 512 adjacent host blocks,
  // 72 KiB of each per layer, runs at 53.5 GB/s with one 2-D copy per layer, and a
  // multi-group restore went from 9.9 to 40.8 GB/s); else one per row.  A pageable pool
  // gets 2-D copies only where the caller asks for them, as in the reference.
  bool two_d(size_t rows) const { return enable_memcpy2d || (rows_as_2d && rows >= 3); }
  size_t cmds_of(size_t rows) const { return full_block || two_d(rows) ? (size_t)1 : rows; }
};
GatherDirectShape gather_direct_shape(const fkv_transfer_desc &d, const HostOrder &order,
                                      size_t staging_cap, bool may_pipeline, bool host_pinned) {
  GatherDirectShape g;
  g.rows_as_2d = host_pinned;
  g.block_bytes = (size_t)d.num_layers * d.kv_dim * (size_t)d.chunk_size;
  g.full_block = (int64_t)g.block_bytes == d.cpu_block_stride;
  g.enable_memcpy2d = d.ce.enable_memcpy2d != 0;
  g.cap_blocks = std::max<size_t>(1, staging_cap / std::max<size_t>(1, g.block_bytes));
  for (size_t r = 0; r + 1 < order.run_start.size(); ++r)
    g.total_cmds += g.cmds_of((size_t)(order.run_start[r + 1] - order.run_start[r]));
  // A transfer that needs several groups and moves in few, large copies alternates
  // between two buffers of half the size: the compaction launch of a group runs next
  // to the copies of its neighbour instead of between them (8 GiB in 1 GiB groups:
  // 8 x 0.36 ms of launches off the critical path of 8 x 18.7 ms of copies; 55.9 ->
  // 56.6 GB/s).  Transfers of many small copies stay on the one-buffer path, whose
  // copies alternate between two streams: that hides the fixed cost per copy, which is
  // worth more there, and GPU->host transfers of 2 MiB copies on two copy streams next
  // to the compaction launches ran at half rate every few calls.
  const size_t half = std::max<size_t>(1, g.cap_blocks / 2);
  const size_t groups_if_pipelined = ((size_t)d.num_blocks + half - 1) / half;
  g.pipelined = may_pipeline && (size_t)d.num_blocks > g.cap_blocks && g.cap_blocks >= 2 &&
                g.total_cmds <= 2 * groups_if_pipelined;
  g.group = std::min<size_t>((size_t)std::max(d.num_blocks, 1), g.pipelined ? half : g.cap_blocks);
  return g;
}

int gather_direct(const Job &j) {
  const auto &d0 = j.d;
  const int lk = d0.num_layers * d0.kv_dim;
  const bool dense = (d0.kv_dim == 1 || d0.cpu_kv_stride == d0.chunk_size) &&
                     (d0.num_layers == 1 || d0.cpu_layer_stride == (int64_t)d0.kv_dim * d0.chunk_size);
  if (!dense)
    return gather_scatter(j); // host chunks of a block are not adjacent: stage per (layer, kv)
  const HostOrder order = host_order(d0);
  fkv_transfer_desc d = d0; // the same transfer, positions in host order
  d.gpu_block_ids = order.gpu_ids.data();
  d.cpu_block_ids = order.cpu_ids.data();
  StageSet &ss = stage_set(j.device);
  GatherDirectShape shape =
      gather_direct_shape(d, order, staging_cap_bytes(), pipeline_enabled(), j.host_pinned);
  if (shape.pipelined && !ss.ensure_pipeline())
    shape = gather_direct_shape(d, order, staging_cap_bytes(), false, j.host_pinned);
  const size_t block_bytes = shape.block_bytes;
  const bool full_block = shape.full_block, pipelined = shape.pipelined;
  auto two_d = [&](size_t rows) { return shape.two_d(rows); };
  auto cmds_of = [&](size_t rows) { return shape.cmds_of(rows); };
  const int nbuf = pipelined ? 2 : 1;
  const int group = (int)shape.group;
  uint8_t *stages[2] = {nullptr, nullptr};
  for (int k = 0; k < nbuf; ++k) {
    stages[k] = device_stage(j.device, k, (size_t)group * block_bytes, j.stream);
    if (!stages[k])
      return per_block(j);
  }
  int rc = FKV_OK;
  if (pipelined) {
    // earlier work of the caller's stream comes before the first copy
    FKV_HIP_TRY(hipEventRecord(ss.fork, j.stream));
    FKV_HIP_TRY(hipStreamWaitEvent(ss.aux, ss.fork, 0));
    j.lane = ss.aux;
  }
  size_t run_i = 0;
  int gi = 0;
  bool used[2] = {false, false};
  for (int p0 = 0; p0 < d.num_blocks && rc == FKV_OK; p0 += group, ++gi) {
    const int np = std::min(group, d.num_blocks - p0);
    const int k = gi % nbuf;
    uint8_t *stage = stages[k];
    if (pipelined) {
      if (!j.h2d) {
        if (used[k]) // the copies that read this buffer two groups ago
          rc = hip_rc(hipStreamWaitEvent(j.stream, ss.copied[k], 0));
        if (rc == FKV_OK)
          rc = device_staging_copy(d, 0, lk, p0, np, stage, true, true, j.stream);
        if (rc == FKV_OK)
          rc = hip_rc(hipEventRecord(ss.kernel_done[k], j.stream));
        if (rc == FKV_OK)
          rc = hip_rc(hipStreamWaitEvent(j.lane, ss.kernel_done[k], 0));
      } else if (used[k]) { // the scatter that read this buffer two groups ago
        rc = hip_rc(hipStreamWaitEvent(j.lane, ss.kernel_done[k], 0));
      }
    } else {
      if (!j.h2d)
        rc = device_staging_copy(d, 0, lk, p0, np, stage, true, true, j.stream);
      // copy commands of this group: runs of consecutive host blocks, clipped to it
      size_t cmds = 0;
      for (size_t r = run_i; r + 1 < order.run_start.size() && order.run_start[r] < p0 + np; ++r)
        cmds += cmds_of((size_t)(std::min(order.run_start[r + 1], p0 + np) -
                                 std::max(order.run_start[r], p0)));
      if (rc == FKV_OK)
        rc = j.fan_out(cmds);
    }
    while (run_i + 1 < order.run_start.size() && rc == FKV_OK) {
      const int b = std::max(order.run_start[run_i], p0);
      const int e = std::min(order.run_start[run_i + 1], p0 + np);
      if (b < e) {
        uint8_t *c = cpu_chunk_ptr(d, (int64_t)d.start_layer_id, 0, d.cpu_block_ids[b]);
        uint8_t *g = stage + (size_t)(b - p0) * block_bytes;
        const size_t rows = (size_t)(e - b);
        if (full_block) {
          rc = j.dma_dir(g, c, rows * block_bytes);
        } else if (two_d(rows)) {
          rc = j.h2d ? j.dma2d(g, block_bytes, c, (size_t)d.cpu_block_stride, block_bytes, rows,
                               j.kind)
                     : j.dma2d(c, (size_t)d.cpu_block_stride, g, block_bytes, block_bytes, rows,
                               j.kind);
        } else {
          for (size_t r = 0; r < rows && rc == FKV_OK; ++r)
            rc = j.dma_dir(g + r * block_bytes, c + r * (size_t)d.cpu_block_stride, block_bytes);
        }
      }
      if (order.run_start[run_i + 1] > p0 + np)
        break; // the rest of this run belongs to the next group
      ++run_i;
    }
    if (pipelined) {
      if (rc == FKV_OK)
        rc = hip_rc(hipEventRecord(ss.copied[k], j.lane));
      if (rc == FKV_OK) {
        used[k] = true;
        if (j.h2d) {
          rc = hip_rc(hipStreamWaitEvent(j.stream, ss.copied[k], 0));
          if (rc == FKV_OK)
            rc = device_staging_copy(d, 0, lk, p0, np, stage, true, false, j.stream);
          if (rc == FKV_OK)
            rc = hip_rc(hipEventRecord(ss.kernel_done[k], j.stream));
        }
      }
    } else {
      int rc2 = j.fan_in();
      if (rc == FKV_OK)
        rc = rc2;
      if (rc == FKV_OK && j.h2d)
        rc = device_staging_copy(d, 0, lk, p0, np, stage, true, false, j.stream);
    }
  }
  if (pipelined) {
    j.lane = nullptr;
    // Everything issued on the copy stream comes before later work of the caller's
    // stream, also after an error part-way.
    if (hipEventRecord(ss.join, ss.aux) != hipSuccess ||
        hipStreamWaitEvent(j.stream, ss.join, 0) != hipSuccess) {
      (void)hipGetLastError();
      (void)hipStreamSynchronize(ss.aux);
    }
  }
  for (int k = 0; k < nbuf; ++k)
    device_stage_mark(j.device, k, j.stream);
  return rc;
}

const char *path_name(int p) {
  switch (p) {
  case FKV_CE_CONTIG_DIRECT: return "CONTIG_DIRECT";
  case FKV_CE_SEGMENT_DIRECT: return "SEGMENT_DIRECT";
  case FKV_CE_SEGMENT_SCATTER: return "SEGMENT_SCATTER";
  case FKV_CE_GATHER_SCATTER: return "GATHER_SCATTER";
  case FKV_CE_GATHER_DIRECT: return "GATHER_DIRECT";
  default: return "PER_BLOCK";
  }
}

} // namespace

namespace {

// Strategy for this transfer: PER_BLOCK, the forced one, or choose()'s.
int resolve_path(const Job &j, int *path_out) {
  const auto &d = j.d;
  const auto &a = j.an.a;
  if (!d.ce.path_opt_enabled) { // csrc/transfer.cu:201-208
    *path_out = FKV_CE_PER_BLOCK;
    return FKV_OK;
  }
  int path;
  if (d.ce.force_path >= 0) {
    if (d.ce.force_path > 4) // csrc/transfer.cu:213-214
      return fail(FKV_ERR_RUNTIME, "force_path out of range [0,4]: %d", d.ce.force_path);
    path = d.ce.force_path;
    // A forced strategy whose layout assumptions do not hold would copy the
    // wrong addresses; refuse instead.
    const bool ok =
        (path == FKV_CE_CONTIG_DIRECT)
            ? (a.gpu_log_contig && a.cpu_log_contig && a.cpu_phys_contig && a.gpu_phys_contig)
        : (path == FKV_CE_SEGMENT_DIRECT) ? (a.cpu_phys_contig && a.gpu_phys_contig)
        : (path == FKV_CE_SEGMENT_SCATTER) ? (a.gpu_phys_contig || use_memcpy2d(j))
                                           : true;
    if (!ok)
      return fail(FKV_ERR_INVALID_ARG,
                  "forced copy-engine strategy %s does not fit this transfer "
                  "(gpu_log=%d cpu_log=%d cpu_phys=%d gpu_phys=%d)",
                  path_name(path), a.gpu_log_contig, a.cpu_log_contig, a.cpu_phys_contig,
                  a.gpu_phys_contig);
  } else {
    const bool full_block = // csrc/transfer.cu:219-220
        (int64_t)d.num_layers * d.kv_dim * d.chunk_size == d.cpu_block_stride;
    path = choose(a, d.ce, d.chunk_size, j.h2d, full_block);
  }
  *path_out = path;
  return FKV_OK;
}

// What a strategy costs beyond moving the bytes over the link once.
struct CeWork {
  double dmas = 0;          // separate DMA commands
  double device_staged = 0; // bytes through a device compaction pass
  double host_staged = 0;   // bytes through a host scatter/gather pass
};

bool host_block_dense(const fkv_transfer_desc &d) {
  return (d.kv_dim == 1 || d.cpu_kv_stride == d.chunk_size) &&
         (d.num_layers == 1 || d.cpu_layer_stride == (int64_t)d.kv_dim * d.chunk_size);
}

CeWork ce_work(const Job &j, int path) {
  const auto &d = j.d;
  const auto &a = j.an.a;
  const double iters = (double)d.num_layers * d.kv_dim, n = d.num_blocks;
  const double segs = (double)j.an.segs.size(), bytes = iters * n * (double)d.chunk_size;
  const bool two_d = use_memcpy2d(j);
  const bool gpu_run = a.gpu_log_contig && a.gpu_phys_contig;
  const bool cpu_run = a.cpu_log_contig && a.cpu_phys_contig;
  CeWork w;
  auto staged = [&] { // GATHER_SCATTER proper
    w.dmas = iters * (two_d ? segs : 1);
    w.device_staged = gpu_run ? 0 : bytes;
    w.host_staged = (two_d || cpu_run) ? 0 : bytes;
  };
  switch (path) {
  case FKV_CE_PER_BLOCK: w.dmas = iters * n; break;
  case FKV_CE_CONTIG_DIRECT: w.dmas = iters; break;
  case FKV_CE_SEGMENT_DIRECT: w.dmas = iters * segs; break;
  case FKV_CE_SEGMENT_SCATTER:
    w.dmas = iters * segs;
    w.host_staged = two_d ? 0 : bytes;
    break;
  case FKV_CE_GATHER_SCATTER:
    if (blocks_are_runs_on_both_sides(j)) {
      const bool linear = iters * (double)d.chunk_size == (double)d.gpu_block_stride &&
                          iters * (double)d.chunk_size == (double)d.cpu_block_stride;
      w.dmas = (linear || d.ce.enable_memcpy2d) ? segs : n;
    } else {
      staged();
    }
    break;
  default: // GATHER_DIRECT
    if (host_block_dense(d)) {
      // one command per run of consecutive host blocks, whatever the GPU side looks like;
      // with two staging buffers only the first group's compaction is on the critical path
      const fkv_launch_policy pol = policy_peek(d.device < 0 ? current_device() : d.device);
      // priced for a pinned pool (no device call here to ask the runtime about the pointer)
      const GatherDirectShape g = gather_direct_shape(d, host_order(d), (size_t)pol.ce_staging_mb << 20,
                                                      pol.ce_two_streams == 1, true);
      w.dmas = (double)g.total_cmds;
      w.device_staged = g.pipelined ? (double)g.group * (double)g.block_bytes : bytes;
    } else {
      staged();
    }
  }
  return w;
}

} // namespace

int choose_engine(const fkv_transfer_desc &d, int *use_ce, double *kernel_s, double *ce_s) {
  Job j{d, nullptr, 0, d.is_host_to_device != 0,
        d.is_host_to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost, {}};
  analyze(d.gpu_block_ids, d.cpu_block_ids, d.num_blocks, d.cpu_block_stride, d.chunk_size,
          d.gpu_block_stride, j.an);
  int path = FKV_CE_PER_BLOCK;
  FKV_TRY(resolve_path(j, &path));
  const CeWork w = ce_work(j, path);
  const double bytes = (double)d.num_blocks * d.num_layers * d.kv_dim * (double)d.chunk_size;
  // the rates and costs of the model are fields of the launch policy (no device call:
  // a device whose table has not been built yet gets the defaults)
  int device = d.device;
  if (device < 0 && hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    device = 0;
  }
  const fkv_launch_policy pol = policy_peek(device);
  const double tk = bytes / ((j.h2d ? pol.model_kernel_h2d_mbps : pol.model_kernel_d2h_mbps) * 1e6) +
                    pol.model_launch_ns * 1e-9;
  const double tc = bytes / (pol.model_link_mbps * 1e6) + w.dmas * pol.model_dma_ns * 1e-9 +
                    w.device_staged / (pol.model_compaction_gbps * 1e9) +
                    w.host_staged / (pol.model_host_pass_mbps * 1e6);
  if (kernel_s)
    *kernel_s = tk;
  if (ce_s)
    *ce_s = tc;
  *use_ce = tc * 100.0 <= pol.model_prefer_ce_pct * tk ? 1 : 0;
  return FKV_OK;
}

int run_ce_path(const fkv_transfer_desc &d, hipStream_t stream) {
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  Job j{d, stream, device, d.is_host_to_device != 0,
        d.is_host_to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost, {}};
  const int rect_min_kb = policy_of(device).ce_rect_min_kb;
  j.rect_min_bytes = rect_min_kb < 0 ? -1 : (int64_t)rect_min_kb * 1024;
  {
    // 2-D copies the caller did not ask for are for pinned host memory only: the runtime
    // stages pageable memory through buffers of its own whatever the call
    hipPointerAttribute_t at{};
    if (hipPointerGetAttributes(&at, d.cpu_ptr) != hipSuccess || at.type != hipMemoryTypeHost) {
      (void)hipGetLastError();
      j.rect_min_bytes = -1;
      j.host_pinned = false;
    }
  }
  analyze(d.gpu_block_ids, d.cpu_block_ids, d.num_blocks, d.cpu_block_stride, d.chunk_size,
          d.gpu_block_stride, j.an);
  int path = FKV_CE_PER_BLOCK;
  FKV_TRY(resolve_path(j, &path));
  set_last_path(path);
  switch (path) {
  case FKV_CE_PER_BLOCK: return per_block(j);
  case FKV_CE_CONTIG_DIRECT: return contig_direct(j);
  case FKV_CE_SEGMENT_DIRECT: return segment_direct(j);
  case FKV_CE_SEGMENT_SCATTER: return segment_scatter(j);
  case FKV_CE_GATHER_SCATTER: return gather_scatter(j);
  default: return gather_direct(j);
  }
}

} // namespace fkv

extern "C" {

int fkv_ce_analyze(const int64_t *gpu_block_ids, const int64_t *cpu_block_ids,
                   int32_t num_blocks, int64_t cpu_block_stride, int64_t chunk_size,
                   int64_t gpu_block_stride, fkv_ce_analysis *out, fkv_ce_segment *segments,
                   int32_t segment_capacity) try {
  fkv::clear_error();
  if (!out || num_blocks < 0 || (num_blocks > 0 && (!gpu_block_ids || !cpu_block_ids)))
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_ce_analyze: bad arguments");
  fkv::Analysis an;
  fkv::analyze(gpu_block_ids, cpu_block_ids, num_blocks, cpu_block_stride, chunk_size,
               gpu_block_stride, an);
  *out = an.a;
  if (segments)
    for (int i = 0; i < (int)an.segs.size() && i < segment_capacity; ++i)
      segments[i] = an.segs[i];
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_ce_choose_path(const fkv_ce_analysis *analysis, const fkv_ce_config *cfg,
                       int64_t chunk_size, int32_t is_host_to_device, int32_t is_full_block) try {
  return fkv::choose(*analysis, *cfg, chunk_size, is_host_to_device != 0, is_full_block != 0);
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
