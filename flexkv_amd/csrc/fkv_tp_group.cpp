// Tensor-parallel transfer group: one persistent thread and one stream per GPU
// of a node, all moving their share of the same block list into / out of one
// shared host pool.  Replaces TPTransferThreadGroup of the reference
// (csrc/tp_transfer_thread_group.{h,cpp}).
//
// Ranks never exchange data: a rank's bytes land at a rank-specific offset
// inside each host chunk (or in a rank-specific region), so the only
// cross-rank logic is the placement rule in fkv_tp_rank_plan_compute().
#include "fkv_internal.h"

#include <exception>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>

namespace {

bool is(const char *a, const char *b) { return std::strcmp(a, b) == 0; }

// csrc/tp_transfer_thread_group.cpp:222-230: unknown names degrade to "sharded"
// (only meaningful when KV is shared across ranks, i.e. num_kv_heads == 1).
const char *canonical_mode(const char *mode, int num_kv_heads, bool *degraded) {
  *degraded = false;
  if (!mode)
    mode = "sharded";
  if (num_kv_heads == 1 && !is(mode, "sharded") && !is(mode, "all_write") &&
      !is(mode, "rank0_only") && !is(mode, "layer_parallel") && !is(mode, "rank_rotate")) {
    *degraded = true;
    return "sharded";
  }
  return mode;
}

} // namespace

extern "C" int fkv_tp_rank_plan_compute(int32_t rank, int32_t num_gpus, int32_t num_kv_heads,
                                        int32_t is_host_to_device, const char *mode_in,
                                        int32_t designated_rank, int32_t rotate_counter,
                                        int32_t layer_id, int32_t layer_granularity,
                                        int32_t num_blocks, int64_t gpu_chunk_size,
                                        int64_t cpu_block_stride, int64_t cpu_tp_stride,
                                        fkv_tp_rank_plan *out) try {
  if (!out || num_gpus < 1 || rank < 0 || rank >= num_gpus)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_tp_rank_plan_compute: bad rank %d of %d", rank,
                     num_gpus);
  bool degraded = false;
  const char *mode = canonical_mode(mode_in, num_kv_heads, &degraded);
  const bool shared_d2h = num_kv_heads == 1 && !is_host_to_device;

  fkv_tp_rank_plan p{};
  p.active = 1;
  p.start_layer = layer_id;
  p.num_layers = layer_granularity;
  p.chunk_size = gpu_chunk_size;

  if (shared_d2h && is(mode, "sharded") && num_gpus > 1 && gpu_chunk_size % num_gpus != 0)
    return fkv::fail(
        FKV_ERR_RUNTIME,
        "sharded kv_shared_across_ranks D2H mode requires gpu_chunk_size divisible by num_gpus, "
        "but chunk_size=%lld and num_gpus=%d. Use 'all_write' or 'rank0_only' mode, or adjust "
        "head_dim/tokens_per_block so chunk_size is divisible.",
        (long long)gpu_chunk_size, num_gpus);

  if (shared_d2h && (is(mode, "rank0_only") || is(mode, "rank_rotate"))) {
    // one writer: the designated rank, or the round-robin counter's value
    const int writer = is(mode, "rank_rotate") ? rotate_counter : designated_rank;
    if (rank != writer)
      p.active = 0;
  } else if (shared_d2h && is(mode, "layer_parallel")) {
    // contiguous layer slices; the first (L mod N) ranks take one layer more
    const int base = layer_granularity / num_gpus, extra = layer_granularity % num_gpus;
    const int mine = base + (rank < extra ? 1 : 0);
    const int before = rank * base + std::min(rank, extra);
    if (mine == 0) {
      p.active = 0;
    } else {
      p.start_layer = layer_id + before;
      p.num_layers = mine;
    }
  }
  if (p.active) {
    if (num_kv_heads > 1) {
      p.cpu_startoff = (int64_t)rank * cpu_tp_stride; // head slice of this rank
    } else if (is(mode, "sharded") && !is_host_to_device) {
      const int64_t shard = gpu_chunk_size / num_gpus; // byte range of every chunk
      p.cpu_startoff = rank * shard;
      p.gpu_startoff = rank * shard;
      p.chunk_size = shard;
    } else if (is(mode, "all_write")) {
      p.cpu_startoff = (int64_t)rank * num_blocks * cpu_block_stride; // a region per rank
    }
  }
  *out = p;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

struct fkv_tp_group {
  int num_gpus = 0;
  int num_tensors_per_gpu = 0;
  int num_layers = 0;
  int backend = 0;
  void *cpu_blocks = nullptr;
  std::vector<uint64_t> gpu_ptrs; // [num_gpus][num_tensors_per_gpu]
  std::vector<int64_t> kv_strides, block_strides, layer_strides, chunk_sizes;
  std::vector<int> device_ids;
  std::vector<hipStream_t> streams;
  fkv_ce_config ce{};
  int rotate_counter = 0;

  struct Lane { // one per GPU
    std::thread th;
    std::mutex mu;
    std::condition_variable cv;
    std::deque<std::function<void()>> q;
    bool stop = false;
  };
  std::vector<std::unique_ptr<Lane>> lanes;

  void lane_loop(int i) {
    (void)hipSetDevice(device_ids[i]);
    Lane &ln = *lanes[i];
    for (;;) {
      std::function<void()> job;
      {
        std::unique_lock<std::mutex> lk(ln.mu);
        ln.cv.wait(lk, [&] { return ln.stop || !ln.q.empty(); });
        if (ln.q.empty())
          return; // stop requested and nothing left
        job = std::move(ln.q.front());
        ln.q.pop_front();
      }
      job();
    }
  }
};

namespace {
struct Completion {
  std::mutex mu;
  std::condition_variable cv;
  int remaining = 0;
  int status = FKV_OK;
  std::string message;
  void finish(int rc, const char *msg) {
    std::lock_guard<std::mutex> lk(mu);
    if (rc != FKV_OK && status == FKV_OK) {
      status = rc;
      message = msg ? msg : "";
    }
    if (--remaining == 0)
      cv.notify_all();
  }
};
} // namespace

extern "C" {

int fkv_tp_group_create(const fkv_tp_group_params *p, fkv_tp_group **out) try {
  using namespace fkv;
  clear_error();
  if (!p || !out || p->num_gpus < 1 || p->num_tensors_per_gpu < 1 || !p->gpu_block_ptrs_flat ||
      !p->gpu_kv_strides || !p->gpu_block_strides || !p->gpu_layer_strides ||
      !p->gpu_chunk_sizes || !p->gpu_device_ids)
    return fail(FKV_ERR_INVALID_ARG, "fkv_tp_group_create: bad arguments");
  int backend;
  if (p->num_tensors_per_gpu == 1)
    backend = FKV_BACKEND_TRTLLM;
  else if (p->num_tensors_per_gpu == p->num_layers)
    backend = FKV_BACKEND_VLLM;
  else if (p->num_tensors_per_gpu == 2 * p->num_layers)
    backend = FKV_BACKEND_SGLANG;
  else // csrc/tp_transfer_thread_group.cpp:77-80
    return fail(FKV_ERR_RUNTIME, "Unsupported GPU block type: %d", p->num_tensors_per_gpu);

  auto g = std::make_unique<fkv_tp_group>();
  g->num_gpus = p->num_gpus;
  g->num_tensors_per_gpu = p->num_tensors_per_gpu;
  g->num_layers = p->num_layers;
  g->backend = backend;
  g->cpu_blocks = p->cpu_blocks_ptr;
  g->ce = p->ce;
  const size_t nptr = (size_t)p->num_gpus * p->num_tensors_per_gpu;
  g->gpu_ptrs.assign(p->gpu_block_ptrs_flat, p->gpu_block_ptrs_flat + nptr);
  g->kv_strides.assign(p->gpu_kv_strides, p->gpu_kv_strides + p->num_gpus);
  g->block_strides.assign(p->gpu_block_strides, p->gpu_block_strides + p->num_gpus);
  g->layer_strides.assign(p->gpu_layer_strides, p->gpu_layer_strides + p->num_gpus);
  g->chunk_sizes.assign(p->gpu_chunk_sizes, p->gpu_chunk_sizes + p->num_gpus);
  for (int i = 0; i < p->num_gpus; ++i)
    g->device_ids.push_back((int)p->gpu_device_ids[i]);

  {
    DeviceGuard restore(-1);
    g->streams.assign(p->num_gpus, nullptr);
    for (int i = 0; i < p->num_gpus; ++i) {
      hipError_t e = hipSetDevice(g->device_ids[i]);
      if (e == hipSuccess)
        e = pooled_stream_acquire(g->device_ids[i], false, &g->streams[i]);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        for (int k = 0; k < i; ++k) {
          (void)hipSetDevice(g->device_ids[k]);
          pooled_stream_release(g->device_ids[k], false, g->streams[k]);
        }
        (void)hipSetDevice(restore.device());
        return fail(FKV_ERR_RUNTIME, "stream creation on device %d failed: %s", g->device_ids[i],
                    hipGetErrorString(e));
      }
    }
    (void)hipSetDevice(restore.device());
  }
  for (int i = 0; i < p->num_gpus; ++i)
    g->lanes.push_back(std::make_unique<fkv_tp_group::Lane>());
  fkv_tp_group *raw = g.get();
  try {
    for (int i = 0; i < p->num_gpus; ++i)
      raw->lanes[i]->th = std::thread([raw, i] { raw->lane_loop(i); });
  } catch (const std::exception &e) { // nothing may cross the C ABI
    const std::string what = e.what();
    fkv_tp_group_destroy(g.release()); // stops and joins the threads that did start
    return fail(FKV_ERR_RUNTIME, "fkv_tp_group_create: cannot start the rank threads: %s",
                what.c_str());
  }
  *out = g.release();
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_tp_group_update_gpu_block_ptrs(fkv_tp_group *g, const uint64_t *ptrs, int64_t count) try {
  using namespace fkv;
  clear_error();
  if (!g || !ptrs)
    return fail(FKV_ERR_INVALID_ARG, "fkv_tp_group_update_gpu_block_ptrs: null argument");
  if (count != (int64_t)g->gpu_ptrs.size()) // csrc/tp_transfer_thread_group.cpp:144-146
    return fail(FKV_ERR_INVALID_ARG, "GPU pointer count does not match transfer group");
  DeviceGuard restore(-1);
  for (int i = 0; i < g->num_gpus; ++i) { // no transfer may still read the old table
    FKV_HIP_TRY(hipSetDevice(g->device_ids[i]));
    FKV_HIP_TRY(fkv::quiet_stream_wait(g->streams[i], g->device_ids[i]));
  }
  (void)hipSetDevice(restore.device());
  g->gpu_ptrs.assign(ptrs, ptrs + count);
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_tp_group_transfer(fkv_tp_group *g, const int64_t *gpu_block_ids,
                          const int64_t *cpu_block_ids, int32_t num_blocks,
                          int64_t cpu_kv_stride, int64_t cpu_layer_stride,
                          int64_t cpu_block_stride, int64_t cpu_tp_stride,
                          int32_t transfer_num_cta, int32_t is_host_to_device,
                          int32_t use_ce_transfer, int32_t layer_id, int32_t layer_granularity,
                          int32_t kv_dim, int32_t num_kv_heads, const char *mode,
                          int32_t designated_rank) try {
  using namespace fkv;
  clear_error();
  if (!g)
    return fail(FKV_ERR_INVALID_ARG, "fkv_tp_group_transfer: null group");
  bool degraded = false;
  const char *eff_mode = canonical_mode(mode, num_kv_heads, &degraded);
  if (degraded)
    fprintf(stderr,
            "[fkv] warning: kv_shared_across_ranks_mode \"%s\" is unknown, using sharded\n",
            mode ? mode : "(null)");
  const bool shared_d2h = num_kv_heads == 1 && !is_host_to_device;
  const int rotate_now = g->rotate_counter;
  if (shared_d2h && is(eff_mode, "rank_rotate")) // one step per D2H call, :249-254
    g->rotate_counter = (g->rotate_counter + 1) % g->num_gpus;

  std::vector<fkv_tp_rank_plan> plans((size_t)g->num_gpus);
  for (int i = 0; i < g->num_gpus; ++i)
    FKV_TRY(fkv_tp_rank_plan_compute(i, g->num_gpus, num_kv_heads, is_host_to_device, eff_mode,
                                     designated_rank, rotate_now, layer_id, layer_granularity,
                                     num_blocks, g->chunk_sizes[i], cpu_block_stride,
                                     cpu_tp_stride, &plans[i]));

  Completion done;
  done.remaining = g->num_gpus;
  for (int i = 0; i < g->num_gpus; ++i) {
    const fkv_tp_rank_plan plan = plans[i];
    auto job = [=, &done] {
      if (!plan.active) {
        done.finish(FKV_OK, nullptr);
        return;
      }
      fkv_transfer_desc d{};
      d.backend = g->backend;
      d.num_layers_total = g->num_layers;
      d.gpu_tensor_ptrs = g->gpu_ptrs.data() + (size_t)i * g->num_tensors_per_gpu;
      d.num_gpu_tensor_ptrs = g->num_tensors_per_gpu;
      d.device = g->device_ids[i];
      d.gpu_kv_stride = g->kv_strides[i];
      d.gpu_block_stride = g->block_strides[i];
      d.gpu_layer_stride = g->layer_strides[i];
      d.gpu_startoff_inside_chunks = plan.gpu_startoff;
      d.cpu_ptr = g->cpu_blocks;
      d.cpu_kv_stride = cpu_kv_stride;
      d.cpu_layer_stride = cpu_layer_stride;
      d.cpu_block_stride = cpu_block_stride;
      d.cpu_startoff_inside_chunks = plan.cpu_startoff;
      d.chunk_size = plan.chunk_size;
      d.start_layer_id = plan.start_layer;
      d.num_layers = plan.num_layers;
      d.kv_dim = kv_dim;
      d.num_blocks = num_blocks;
      d.gpu_block_ids = gpu_block_ids;
      d.cpu_block_ids = cpu_block_ids;
      d.is_host_to_device = is_host_to_device;
      d.use_ce_transfer = use_ce_transfer;
      d.transfer_num_cta = transfer_num_cta;
      d.sync = 1;
      d.ce = g->ce;
      int rc = fkv_transfer_kv_blocks(&d, g->streams[i]);
      done.finish(rc, rc == FKV_OK ? nullptr : fkv_last_error());
    };
    {
      std::lock_guard<std::mutex> lk(g->lanes[i]->mu);
      g->lanes[i]->q.emplace_back(std::move(job));
    }
    g->lanes[i]->cv.notify_one();
  }
  {
    std::unique_lock<std::mutex> lk(done.mu);
    done.cv.wait(lk, [&] { return done.remaining == 0; });
  }
  if (done.status != FKV_OK) // csrc/tp_transfer_thread_group.cpp:378-380
    return fail(done.status, "tp_group_transfer failed: %s", done.message.c_str());
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

void fkv_tp_group_destroy(fkv_tp_group *g) {
  if (!g)
    return;
  for (auto &ln : g->lanes) {
    {
      std::lock_guard<std::mutex> lk(ln->mu);
      ln->stop = true;
    }
    ln->cv.notify_all();
  }
  for (auto &ln : g->lanes)
    if (ln->th.joinable())
      ln->th.join();
  fkv::DeviceGuard restore(-1);
  for (int i = 0; i < g->num_gpus; ++i) {
    (void)hipSetDevice(g->device_ids[i]);
    (void)hipStreamSynchronize(g->streams[i]);
    fkv::pooled_stream_release(g->device_ids[i], false, g->streams[i]);
  }
  (void)hipSetDevice(restore.device());
  (void)hipGetLastError();
  delete g;
}

} // extern "C"
