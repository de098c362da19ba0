// Layer-by-layer host->GPU restore with per-layer completion signalling, so
// that attention on layer L can start while layer L+1 is still on the link.
// Replaces the single-group, main-KV part of LayerwiseTransferGroup in the
// reference (csrc/layerwise.{h,cpp}).
//
// Per call, layers go out in batches of `layer_granularity` on one
// non-blocking stream per GPU.  Behind every batch a hip event is recorded on
// each GPU's stream.  Completion of a batch is announced
//   * to consumers in other processes through semaphore eventfds, one
//     write(1) per (layer, tp_rank) — csrc/layerwise.cpp:15-137, 907-942.
//     HOSTFUNC mode returns after all copies have landed: the calling thread
//     waits on the batch events in order and writes the eventfds as each batch
//     completes.  (The reference enqueues a host function behind every batch;
//     on this runtime a host function holds its stream for about 50 us, which
//     would serialise an 80-layer restore by 4 ms, and nothing observable
//     depends on which thread does the write.)  POLLING mode returns right
//     after the launches and a thread polls the batch events in order;
//   * to consumers in this process through fkv_layerwise_wait_layer(), which
//     makes their stream wait on the batch event (no host round trip).
//
// The transfer streams keep the default priority.
#include "fkv_internal.h"

#include <sys/eventfd.h>
#include <unistd.h>

#include <atomic>
#include <cstring>
#include <memory>
#include <thread>

struct fkv_layerwise {
  int num_gpus = 0;
  int num_tensors_per_gpu = 0;
  int num_layers = 0;
  int tp_size = 1;
  int backend = 0;
  void *cpu_blocks = nullptr;
  std::vector<uint64_t> gpu_ptrs;
  std::vector<int64_t> kv_strides, block_strides, layer_strides, chunk_sizes;
  std::vector<int> device_ids;
  std::vector<hipStream_t> streams;
  fkv_ce_config ce{};

  std::vector<int32_t> eventfds; // [num_counters][tp_size][num_layers]
  int num_counters = 0;

  // state of the most recent transfer
  struct Batch {
    int start_layer = 0;
    int layers = 0;
    std::vector<hipEvent_t> done; // one per GPU
    fkv_layerwise *owner = nullptr;
  };
  std::vector<std::unique_ptr<Batch>> batches;
  hipEvent_t started = nullptr; // on streams[0], before the first batch
  int granularity = 1;
  int counter_id = 0;
  int notify_mode = FKV_NOTIFY_HOSTFUNC;
  std::thread poller;
  std::atomic<bool> poller_stop{false};

  // csrc/layerwise.cpp:15-34
  void notify(const Batch &b) const {
    if (eventfds.empty())
      return;
    const int32_t *base = eventfds.data() + (size_t)counter_id * tp_size * num_layers;
    for (int layer = b.start_layer; layer < b.start_layer + b.layers; ++layer)
      for (int r = 0; r < tp_size; ++r) {
        const int fd = base[(size_t)r * num_layers + layer];
        if (fd >= 0) {
          const uint64_t one = 1;
          ssize_t w = write(fd, &one, sizeof(one));
          (void)w;
        }
      }
  }

  void poll_loop() {
    size_t next = 0;
    while (next < batches.size() && !poller_stop.load(std::memory_order_acquire)) {
      Batch &b = *batches[next];
      bool all = true;
      for (int g = 0; g < num_gpus && all; ++g) {
        (void)hipSetDevice(device_ids[g]);
        hipError_t e = hipEventQuery(b.done[g]);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          all = false;
        }
      }
      if (all) {
        notify(b);
        ++next;
      } else {
        std::this_thread::yield();
      }
    }
  }

  // Ends the notification machinery of the previous transfer and frees its
  // events.  All work of that transfer has completed when this returns.
  void retire_previous() {
    if (poller.joinable())
      poller.join(); // runs until every batch has been announced
    fkv::DeviceGuard restore(-1);
    for (int g = 0; g < num_gpus; ++g) {
      (void)hipSetDevice(device_ids[g]);
      (void)hipStreamSynchronize(streams[g]);
    }
    for (auto &b : batches)
      for (int g = 0; g < num_gpus; ++g) {
        (void)hipSetDevice(device_ids[g]);
        if (b->done[g])
          (void)hipEventDestroy(b->done[g]);
      }
    batches.clear();
    if (started) {
      (void)hipSetDevice(device_ids[0]);
      (void)hipEventDestroy(started);
      started = nullptr;
    }
    (void)hipSetDevice(restore.device());
    (void)hipGetLastError();
  }
};

namespace {

bool is(const char *a, const char *b) { return std::strcmp(a, b) == 0; }

} // namespace

extern "C" {

int fkv_layerwise_create(const fkv_layerwise_params *p, fkv_layerwise **out) {
  using namespace fkv;
  clear_error();
  if (!p || !out || p->num_gpus < 1 || p->num_tensors_per_gpu < 1 || p->num_layers < 1 ||
      p->tp_size < 1 || !p->gpu_block_ptrs_flat || !p->gpu_kv_strides ||
      !p->gpu_block_strides || !p->gpu_layer_strides || !p->gpu_chunk_sizes ||
      !p->gpu_device_ids)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_create: bad arguments");
  int backend;
  if (p->num_tensors_per_gpu == 1)
    backend = FKV_BACKEND_TRTLLM;
  else if (p->num_tensors_per_gpu == p->num_layers)
    backend = FKV_BACKEND_VLLM;
  else if (p->num_tensors_per_gpu == 2 * p->num_layers)
    backend = FKV_BACKEND_SGLANG;
  else // csrc/layerwise.cpp:586-595
    return fail(FKV_ERR_RUNTIME, "Unsupported GPU block type: %d", p->num_tensors_per_gpu);
  if (p->num_layer_eventfds > 0) {
    if (!p->layer_eventfds || p->num_layer_eventfds % (p->tp_size * p->num_layers) != 0)
      return fail(FKV_ERR_INVALID_ARG,
                  "layer_eventfds must hold a multiple of tp_size*num_layers = %d entries, got %d",
                  p->tp_size * p->num_layers, p->num_layer_eventfds);
  }
  auto g = std::make_unique<fkv_layerwise>();
  g->num_gpus = p->num_gpus;
  g->num_tensors_per_gpu = p->num_tensors_per_gpu;
  g->num_layers = p->num_layers;
  g->tp_size = p->tp_size;
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
  if (p->num_layer_eventfds > 0) {
    g->eventfds.assign(p->layer_eventfds, p->layer_eventfds + p->num_layer_eventfds);
    g->num_counters = p->num_layer_eventfds / (p->tp_size * p->num_layers);
  }
  DeviceGuard restore(-1);
  g->streams.assign(p->num_gpus, nullptr);
  for (int i = 0; i < p->num_gpus; ++i) {
    hipError_t e = hipSetDevice(g->device_ids[i]);
    if (e == hipSuccess)
      e = hipStreamCreateWithFlags(&g->streams[i], hipStreamNonBlocking);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      for (int k = 0; k < i; ++k) {
        (void)hipSetDevice(g->device_ids[k]);
        (void)hipStreamDestroy(g->streams[k]);
      }
      (void)hipSetDevice(restore.device());
      return fail(FKV_ERR_RUNTIME, "stream creation on device %d failed: %s", g->device_ids[i],
                  hipGetErrorString(e));
    }
  }
  (void)hipSetDevice(restore.device());
  *out = g.release();
  return FKV_OK;
}

int fkv_layerwise_transfer(fkv_layerwise *g, const int64_t *gpu_block_ids,
                           const int64_t *cpu_block_ids, int32_t num_blocks,
                           int64_t cpu_block_stride, int64_t h2d_cpu_kv_stride,
                           int64_t h2d_cpu_layer_stride, int64_t cpu_tp_stride,
                           int32_t transfer_cta_num, int32_t use_ce_transfer,
                           int32_t num_layers, int32_t layer_granularity, int32_t kv_dim,
                           int32_t num_kv_heads, int32_t counter_id, const char *mode_in,
                           int32_t notify_mode, int32_t enable_trace) {
  using namespace fkv;
  clear_error();
  if (!g)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer: null group");
  if (num_layers < 0 || num_layers > g->num_layers || layer_granularity < 1 || num_blocks < 0)
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_layerwise_transfer: num_layers=%d (group has %d) layer_granularity=%d "
                "num_blocks=%d",
                num_layers, g->num_layers, layer_granularity, num_blocks);
  if (!g->eventfds.empty() && (counter_id < 0 || counter_id >= g->num_counters))
    return fail(FKV_ERR_INVALID_ARG, "counter_id %d outside [0, %d)", counter_id,
                g->num_counters);
  if (notify_mode != FKV_NOTIFY_HOSTFUNC && notify_mode != FKV_NOTIFY_POLLING)
    return fail(FKV_ERR_INVALID_ARG, "unknown notify mode %d", notify_mode);

  g->retire_previous();
  g->counter_id = counter_id;
  g->granularity = layer_granularity;
  g->notify_mode = notify_mode;

  // csrc/layerwise.cpp:1112-1121: only these three names are meaningful for a
  // restore; anything else is treated as "sharded".
  const char *mode = mode_in ? mode_in : "sharded";
  if (num_kv_heads == 1 && !is(mode, "sharded") && !is(mode, "all_write") &&
      !is(mode, "rank0_only")) {
    fprintf(stderr,
            "[fkv] warning: kv_shared_across_ranks_mode \"%s\" is not valid for layerwise "
            "restore, using sharded\n",
            mode);
    mode = "sharded";
  }

  DeviceGuard restore(-1);
  const int num_batches = (num_layers + layer_granularity - 1) / layer_granularity;
  for (int b = 0; b < num_batches; ++b) {
    auto batch = std::make_unique<fkv_layerwise::Batch>();
    batch->start_layer = b * layer_granularity;
    batch->layers = std::min(layer_granularity, num_layers - batch->start_layer);
    batch->owner = g;
    batch->done.assign(g->num_gpus, nullptr);
    for (int i = 0; i < g->num_gpus; ++i) {
      FKV_HIP_TRY(hipSetDevice(g->device_ids[i]));
      FKV_HIP_TRY(hipEventCreate(&batch->done[i]));
    }
    g->batches.push_back(std::move(batch));
  }
  FKV_HIP_TRY(hipSetDevice(g->device_ids[0]));
  FKV_HIP_TRY(hipEventCreate(&g->started));
  FKV_HIP_TRY(hipEventRecord(g->started, g->streams[0]));

  // descriptor of rank i for layers [start, start + layers)
  auto describe = [&](int i, int start, int layers) {
    // host offset of rank i, csrc/layerwise.cpp:1143-1166
    int64_t cpu_off = (int64_t)i * cpu_tp_stride;
    if (num_kv_heads == 1)
      cpu_off = is(mode, "all_write") ? (int64_t)i * num_blocks * cpu_block_stride : 0;
    fkv_transfer_desc d{};
    d.backend = g->backend;
    d.num_layers_total = g->num_layers;
    d.gpu_tensor_ptrs = g->gpu_ptrs.data() + (size_t)i * g->num_tensors_per_gpu;
    d.num_gpu_tensor_ptrs = g->num_tensors_per_gpu;
    d.device = g->device_ids[i];
    d.gpu_kv_stride = g->kv_strides[i];
    d.gpu_block_stride = g->block_strides[i];
    d.gpu_layer_stride = g->layer_strides[i];
    d.gpu_startoff_inside_chunks = 0;
    d.cpu_ptr = g->cpu_blocks;
    d.cpu_kv_stride = h2d_cpu_kv_stride;
    d.cpu_layer_stride = h2d_cpu_layer_stride;
    d.cpu_block_stride = cpu_block_stride;
    d.cpu_startoff_inside_chunks = cpu_off;
    d.chunk_size = g->chunk_sizes[i];
    d.start_layer_id = start;
    d.num_layers = layers;
    d.kv_dim = kv_dim;
    d.num_blocks = num_blocks;
    d.gpu_block_ids = gpu_block_ids;
    d.cpu_block_ids = cpu_block_ids;
    d.is_host_to_device = 1;
    d.use_ce_transfer = use_ce_transfer;
    d.transfer_num_cta = transfer_cta_num;
    d.sync = 0;
    d.ce = g->ce;
    return d;
  };

  int rc = FKV_OK;
  // Kernel path: the id lists and the base tables of all layers go to the device
  // once per GPU; every batch is then a single kernel launch.
  const bool direct = !use_ce_transfer && num_blocks > 0 && num_layers > 0;
  std::vector<KernelPlan> plans(direct ? g->num_gpus : 0);
  if (direct) {
    for (int i = 0; i < g->num_gpus && rc == FKV_OK; ++i) {
      fkv_transfer_desc d = describe(i, 0, num_layers);
      if (!d.gpu_tensor_ptrs || !d.cpu_ptr || !gpu_block_ids || !cpu_block_ids ||
          d.chunk_size <= 0 || kv_dim < 1) {
        rc = fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer: bad pointers or sizes");
        break;
      }
      (void)hipSetDevice(g->device_ids[i]);
      rc = kernel_plan_build(d, g->streams[i], &plans[i]);
    }
  }
  for (int b = 0; b < num_batches && rc == FKV_OK; ++b) {
    fkv_layerwise::Batch &batch = *g->batches[b];
    for (int i = 0; i < g->num_gpus && rc == FKV_OK; ++i) {
      (void)hipSetDevice(g->device_ids[i]);
      if (direct) {
        rc = kernel_plan_launch(plans[i], batch.start_layer, batch.layers, g->streams[i]);
        if (rc == FKV_OK) {
          stats().calls.fetch_add(1, std::memory_order_relaxed);
          stats().bytes_h2d.fetch_add((uint64_t)num_blocks * batch.layers * kv_dim *
                                          (uint64_t)g->chunk_sizes[i],
                                      std::memory_order_relaxed);
        }
      } else {
        fkv_transfer_desc d = describe(i, batch.start_layer, batch.layers);
        rc = fkv_transfer_kv_blocks(&d, g->streams[i]);
      }
      if (rc != FKV_OK)
        break;
      (void)hipSetDevice(g->device_ids[i]);
      hipError_t e = hipEventRecord(batch.done[i], g->streams[i]);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        rc = fail(FKV_ERR_RUNTIME, "layerwise_transfer failed on GPU %d: %s", i,
                  hipGetErrorString(e));
      }
    }
  }
  std::string saved_error = fkv_last_error();
  for (int i = 0; i < (int)plans.size(); ++i) {
    (void)hipSetDevice(g->device_ids[i]);
    kernel_plan_release(&plans[i], g->streams[i]);
  }
  if (rc != FKV_OK) {
    // Drain what was enqueued so no callback outlives this call's batches.
    for (int i = 0; i < g->num_gpus; ++i) {
      (void)hipSetDevice(g->device_ids[i]);
      (void)hipStreamSynchronize(g->streams[i]);
    }
    (void)hipSetDevice(restore.device());
    (void)hipGetLastError();
    return fail(rc, "%s", saved_error.c_str());
  }

  if (notify_mode == FKV_NOTIFY_POLLING) {
    g->poller_stop.store(false, std::memory_order_release);
    // Nobody listens when no eventfd table was given: in-process consumers wait
    // on the batch events directly, so there is nothing to poll for.
    if (num_batches > 0 && !g->eventfds.empty())
      g->poller = std::thread([g] { g->poll_loop(); });
  } else {
    // announce every batch as soon as all GPUs have finished it, in order
    for (int b = 0; b < num_batches; ++b) {
      for (int i = 0; i < g->num_gpus; ++i) {
        (void)hipSetDevice(g->device_ids[i]);
        hipError_t e = hipEventSynchronize(g->batches[b]->done[i]);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          (void)hipSetDevice(restore.device());
          return fail(FKV_ERR_RUNTIME, "layerwise_transfer failed on GPU %d: %s", i,
                      hipGetErrorString(e));
        }
      }
      g->notify(*g->batches[b]);
    }
    for (int i = 0; i < g->num_gpus; ++i) { // csrc/layerwise.cpp:1249-1256
      (void)hipSetDevice(g->device_ids[i]);
      hipError_t e = hipStreamSynchronize(g->streams[i]);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipSetDevice(restore.device());
        return fail(FKV_ERR_RUNTIME, "layerwise_transfer failed on GPU %d: %s", i,
                    hipGetErrorString(e));
      }
    }
    if (enable_trace && num_batches > 0) {
      // per-batch line with the fields of csrc/layerwise.cpp:1281-1285
      (void)hipSetDevice(g->device_ids[0]);
      float prev = 0;
      for (int b = 0; b < num_batches; ++b) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, g->started, g->batches[b]->done[0]) != hipSuccess) {
          (void)hipGetLastError();
          continue;
        }
        const fkv_layerwise::Batch &bt = *g->batches[b];
        double bytes = 0;
        for (int i = 0; i < g->num_gpus; ++i)
          bytes += (double)g->chunk_sizes[i] * kv_dim * bt.layers * num_blocks;
        const double mb = bytes / (1024.0 * 1024.0);
        const double dt = ms - prev;
        fprintf(stderr,
                "[XFER] type=layerwise_h2d layer_range=[%d,%d) blocks=%d data=%.2fMB "
                "sync_ms=%.3f bw=%.0fMB/s\n",
                bt.start_layer, bt.start_layer + bt.layers, num_blocks, mb, dt,
                dt > 0 ? mb / (dt / 1000.0) : 0.0);
        prev = ms;
      }
    }
  }
  (void)hipSetDevice(restore.device());
  return FKV_OK;
}

int fkv_layerwise_wait_layer(fkv_layerwise *g, int32_t gpu_index, int32_t layer,
                             void *consumer_stream) {
  using namespace fkv;
  clear_error();
  if (!g || gpu_index < 0 || gpu_index >= g->num_gpus)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_wait_layer: bad group or GPU index");
  const int b = layer / g->granularity;
  if (layer < 0 || b >= (int)g->batches.size())
    return fail(FKV_ERR_INVALID_ARG, "layer %d was not part of the last transfer", layer);
  FKV_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(consumer_stream),
                                 g->batches[b]->done[gpu_index], 0));
  return FKV_OK;
}

int fkv_layerwise_synchronize(fkv_layerwise *g) {
  using namespace fkv;
  clear_error();
  if (!g)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_synchronize: null group");
  if (g->poller.joinable())
    g->poller.join();
  DeviceGuard restore(-1);
  for (int i = 0; i < g->num_gpus; ++i) {
    FKV_HIP_TRY(hipSetDevice(g->device_ids[i]));
    FKV_HIP_TRY(hipStreamSynchronize(g->streams[i]));
  }
  (void)hipSetDevice(restore.device());
  return FKV_OK;
}

int fkv_layerwise_batch_times_ms(fkv_layerwise *g, float *out_ms, int32_t capacity,
                                 int32_t *num_batches) {
  using namespace fkv;
  clear_error();
  if (!g || !num_batches)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_batch_times_ms: null argument");
  *num_batches = (int32_t)g->batches.size();
  DeviceGuard restore(g->device_ids[0]);
  for (int b = 0; b < (int)g->batches.size() && b < capacity; ++b)
    FKV_HIP_TRY(hipEventElapsedTime(&out_ms[b], g->started, g->batches[b]->done[0]));
  return FKV_OK;
}

void fkv_layerwise_destroy(fkv_layerwise *g) {
  if (!g)
    return;
  g->retire_previous();
  fkv::DeviceGuard restore(-1);
  for (int i = 0; i < g->num_gpus; ++i) {
    (void)hipSetDevice(g->device_ids[i]);
    (void)hipStreamDestroy(g->streams[i]);
  }
  (void)hipSetDevice(restore.device());
  (void)hipGetLastError();
  delete g;
}

} // extern "C"
