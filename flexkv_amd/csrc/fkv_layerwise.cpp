// Layer-by-layer host->GPU restore with per-layer completion signalling, so
// that attention on layer L can start while layer L+1 is still on the link.
// Replaces LayerwiseTransferGroup of the reference (csrc/layerwise.{h,cpp})
// without its SSD pre-load: the single-group form, the multi-group form (layer
// groups of different KV shape that share the original layers of the model) and
// the sliding-window sidecars of both.
//
// A restore is a sequence of batches on one non-blocking stream per GPU.  A
// batch is `layer_granularity` consecutive layers (single group) or everything
// attached to one original layer (multi-group: the members of every group, then
// the sidecar).  Behind every batch a hip event is recorded on each GPU's
// stream.  Completion of a batch is announced
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
// On the kernel path the id lists and the base tables of every layer of a group
// go to the device once per call and GPU; each (batch, group) is then a single
// kernel launch.
//
// A restore whose host rows are gathered by host threads first (see
// fkv_staged_restore.cpp) cannot enqueue everything at once: the copy of a batch is
// enqueued when its rows have been gathered.  Such a restore is launched batch by
// batch from a thread of its own, and everything that looks at a batch event first
// waits until that event has been recorded.
//
// The transfer streams keep the default priority.
#include "fkv_gate.h"
#include "fkv_host_copy.h"
#include "fkv_internal.h"
#include "fkv_poll.h"

#include <sys/eventfd.h>
#include <unistd.h>

#include <exception>
#include <atomic>
#include <condition_variable>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <thread>

namespace {

bool is(const char *a, const char *b) { return std::strcmp(a, b) == 0; }

// csrc/layerwise.cpp:586-595, 792-806
int backend_of(int tensors_per_gpu, int num_layers) {
  if (tensors_per_gpu == 1)
    return FKV_BACKEND_TRTLLM;
  if (tensors_per_gpu == num_layers)
    return FKV_BACKEND_VLLM;
  if (tensors_per_gpu == 2 * num_layers)
    return FKV_BACKEND_SGLANG;
  return -1;
}

// Device tensors of one layer group and where the group lives inside a host
// block (GroupParams of the reference).
struct Source {
  int num_layers = 0;
  int num_tensors_per_gpu = 0;
  int backend = 0;
  std::vector<uint64_t> gpu_ptrs; // [num_gpus][num_tensors_per_gpu]
  std::vector<int64_t> kv_strides, block_strides, layer_strides, chunk_sizes; // per GPU
  int64_t cpu_offset_bytes = 0;
  int64_t h2d_cpu_kv_stride = 0, h2d_cpu_layer_stride = 0;
  int64_t cpu_block_stride = 0, cpu_tp_stride = 0;
};

bool fill_source(Source &s, const fkv_layer_group &in, int num_gpus) {
  if (in.num_layers < 1 || in.num_tensors_per_gpu < 1 || !in.gpu_block_ptrs_flat ||
      !in.gpu_kv_strides || !in.gpu_block_strides || !in.gpu_layer_strides ||
      !in.gpu_chunk_sizes)
    return false;
  s.num_layers = in.num_layers;
  s.num_tensors_per_gpu = in.num_tensors_per_gpu;
  s.backend = backend_of(in.num_tensors_per_gpu, in.num_layers);
  const size_t nptr = (size_t)num_gpus * in.num_tensors_per_gpu;
  s.gpu_ptrs.assign(in.gpu_block_ptrs_flat, in.gpu_block_ptrs_flat + nptr);
  s.kv_strides.assign(in.gpu_kv_strides, in.gpu_kv_strides + num_gpus);
  s.block_strides.assign(in.gpu_block_strides, in.gpu_block_strides + num_gpus);
  s.layer_strides.assign(in.gpu_layer_strides, in.gpu_layer_strides + num_gpus);
  s.chunk_sizes.assign(in.gpu_chunk_sizes, in.gpu_chunk_sizes + num_gpus);
  s.cpu_offset_bytes = in.cpu_offset_bytes;
  s.h2d_cpu_kv_stride = in.h2d_cpu_kv_stride;
  s.h2d_cpu_layer_stride = in.h2d_cpu_layer_stride;
  s.cpu_block_stride = in.cpu_block_stride;
  s.cpu_tp_stride = in.cpu_tp_stride;
  return true;
}

using MemberTable = std::vector<std::vector<fkv_layer_member>>;

// Unpacks the CSR member lists and checks every entry against the groups.
int fill_members(MemberTable &out, int num_original_layers, const int32_t *offsets,
                 const fkv_layer_member *members, const std::vector<Source> &groups,
                 const char *what) {
  using namespace fkv;
  if (!offsets)
    return fail(FKV_ERR_INVALID_ARG, "%s: member_offsets is null", what);
  out.assign(num_original_layers, {});
  for (int l = 0; l < num_original_layers; ++l) {
    if (offsets[l + 1] < offsets[l] || offsets[l] < 0)
      return fail(FKV_ERR_INVALID_ARG, "%s: member_offsets must be non-decreasing", what);
    for (int k = offsets[l]; k < offsets[l + 1]; ++k) {
      const fkv_layer_member m = members[k];
      if (m.group < 0 || m.group >= (int)groups.size() || m.local_layer < 0 ||
          m.local_layer >= groups[m.group].num_layers)
        return fail(FKV_ERR_INVALID_ARG,
                    "%s: member (group %d, layer %d) of original layer %d is out of range", what,
                    m.group, m.local_layer, l);
      out[l].push_back(m);
    }
  }
  return FKV_OK;
}

// A Source as one call uses it: block ids, host strides and per-GPU host
// offsets resolved, plus the uploaded kernel plans.
struct Lane {
  const Source *src = nullptr;
  void *cpu_ptr = nullptr;
  int64_t cpu_kv_stride = 0, cpu_layer_stride = 0, cpu_block_stride = 0;
  std::vector<int64_t> cpu_off; // per GPU
  const int64_t *gpu_ids = nullptr, *cpu_ids = nullptr;
  std::vector<int64_t> own_gpu_ids, own_cpu_ids; // copies, where the launch outlives the call
  int num_blocks = 0;
  int kv_dim = 1;
  bool used = false;
  std::vector<fkv::KernelPlan> plans; // per GPU, kernel path only
  std::vector<fkv::StagedPlan> staged; // per GPU: usable where this call goes through the copy engines
};

struct Item {
  int lane = 0;
  int start_layer = 0;
  int layers = 0;
};

} // namespace

struct fkv_layerwise {
  int num_gpus = 0;
  int num_layers = 0; // original layers: the extent of the eventfd table
  int tp_size = 1;
  bool multi_group = false;
  void *cpu_blocks = nullptr;
  std::vector<Source> groups; // exactly one for a single-group instance
  MemberTable members;        // multi-group only
  bool has_swa = false, swa_multi_group = false;
  void *swa_cpu_blocks = nullptr;
  std::vector<Source> swa_groups; // exactly one for the uniform sidecar
  MemberTable swa_members;
  std::vector<int> device_ids;
  std::vector<hipStream_t> streams;
  // Restores through the copy engines (fkv_staged_restore.cpp): a second stream per
  // GPU for the copies, created on first use, and the staging buffers by
  // (lane, GPU), kept from call to call.
  std::vector<hipStream_t> dma_streams;
  // A second one per GPU: the copies of consecutive batches alternate between the two, so
  // that the event record and wait around one copy run next to the other stream's copy
  // instead of between two copies (the engine takes the copies in the order of submission
  // either way).  Created with the first; nullptr = all copies on the first.
  std::vector<hipStream_t> dma_streams2;
  std::vector<unsigned> dma_turn;
  // Restores by kernel in small batches: every other batch is launched on a second stream
  // per GPU, which starts behind the first batch of the call (and so behind its plan
  // uploads) and is joined back into `streams` before the plans are released, so that a batch starts while its predecessor's last requests are in
  // flight and its event is being recorded (8 us between two launches on one stream,
  // next to 18 us of link time for 1 MiB).  Created on first use.
  std::vector<hipStream_t> alt_streams;
  std::vector<hipEvent_t> alt_join;
  std::map<std::pair<int, int>, fkv::StagedRing> rings;
  // Restores whose rows host threads gather first: pinned buffers by (lane, GPU), the
  // helper threads, and the thread that launches such a restore batch by batch.
  std::map<std::pair<int, int>, fkv::GatherRing> pinned_rings;
  std::unique_ptr<fkv::HostCrew> crew;
  std::thread feeder;
  std::vector<Lane> feed_lanes; // what the feeder works on
  int feed_use_ce = 0, feed_num_cta = 0;
  fkv::BatchGate gate;          // which batches have had their events recorded, or never will
  int feed_rc = 0;              // why the launching thread gave up (read once it has been joined)
  std::string feed_error;
  fkv_ce_config ce{};

  std::vector<int32_t> eventfds; // [num_counters][tp_size][num_layers]
  int num_counters = 0;

  // state of the most recent transfer
  struct Batch {
    int start_layer = 0;
    int layers = 0;
    std::vector<Item> items;
    std::vector<hipEvent_t> done; // one per GPU
    int num_members = 0;          // multi-group: main members of the original layer
    double trace_bytes = 0;
  };
  std::vector<std::unique_ptr<Batch>> batches;
  std::vector<int> layer_batch; // layer -> index into batches, -1: nothing in flight
  hipEvent_t started = nullptr; // on streams[0], before the first batch
  int counter_id = 0;
  std::thread poller;
  std::atomic<bool> poller_stop{false};
  // hipError_t of the first device error the poller or a retire saw (0 = none); the
  // layers behind it were not announced.  Reported, and cleared, by the next call.
  std::atomic<int> restore_error{0};

  // csrc/layerwise.cpp:15-34
  void notify_layers(int start_layer, int layers) const {
    if (eventfds.empty())
      return;
    const int32_t *base = eventfds.data() + (size_t)counter_id * tp_size * num_layers;
    for (int layer = start_layer; layer < start_layer + layers; ++layer)
      for (int r = 0; r < tp_size; ++r) {
        const int fd = base[(size_t)r * num_layers + layer];
        if (fd >= 0) {
          const uint64_t one = 1;
          ssize_t w = write(fd, &one, sizeof(one));
          (void)w;
        }
      }
  }
  void notify(const Batch &b) const { notify_layers(b.start_layer, b.layers); }

  void poll_loop() {
    int status;
    try {
      status = poll_batches();
    } catch (...) { // as a device error would: the layers behind it are not announced
      status = (int)hipErrorUnknown;
    }
    if (status != (int)hipSuccess) {
      // A real device error: the layers behind it were not announced; the next call
      // on the group reports it.
      int none = 0;
      restore_error.compare_exchange_strong(none, status);
    }
  }

  int poll_batches() {
    return fkv::poll_batches_in_order(
        batches.size(), num_gpus, (int)hipSuccess, (int)hipErrorNotReady,
        [this](size_t b, int g) {
          // an event that has not been recorded yet reads as complete
          const int state = gate.peek((int)b);
          if (state <= 0)
            return (int)(state < 0 ? hipErrorLaunchFailure : hipErrorNotReady);
          (void)hipSetDevice(device_ids[g]);
          const hipError_t e = hipEventQuery(batches[b]->done[g]);
          if (e != hipSuccess)
            (void)hipGetLastError();
          return (int)e;
        },
        [this](size_t b) { notify(*batches[b]); }, poller_stop);
  }

  // The launching thread ends by itself: it waits for nothing but copies that are
  // already enqueued.
  void join_feeder() {
    if (feeder.joinable())
      feeder.join();
  }

  // Waits for the poller: it ends by itself once every batch has been announced or
  // a device error has been seen.  Should the streams drain and the poller still
  // run (a failed stream leaves its events unready for good), it is told to stop.
  void join_poller() {
    join_feeder();
    if (!poller.joinable())
      return;
    fkv::DeviceGuard restore(-1);
    for (int g = 0; g < num_gpus; ++g) {
      (void)hipSetDevice(device_ids[g]);
      hipError_t e = hipStreamSynchronize(streams[g]);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        int none = 0;
        restore_error.compare_exchange_strong(none, (int)e);
        poller_stop.store(true, std::memory_order_release);
      }
    }
    (void)hipSetDevice(restore.device());
    // Streams drained without error: every batch event is ready, so the poller
    // announces what is left and returns.
    poller.join();
  }

  // The error of the previous restore, if any, as a status of the current call.
  int take_restore_error(const char *where) {
    const int e = restore_error.exchange(0);
    if (gate.failed()) { // the launching thread has been joined
      gate.clear_failure();
      return fkv::fail(feed_rc ? feed_rc : FKV_ERR_RUNTIME,
                       "%s: the previous layerwise restore failed while it was launched: %s", where,
                       feed_error.c_str());
    }
    if (e == 0)
      return FKV_OK;
    return fkv::fail(FKV_ERR_RUNTIME, "%s: the previous layerwise restore failed on the device: %s",
                     where, hipGetErrorString((hipError_t)e));
  }

  // Ends the notification machinery of the previous transfer and frees its
  // events.  All work of that transfer has completed when this returns.
  void retire_previous() {
    join_feeder();
    join_poller();
    fkv::DeviceGuard restore(-1);
    for (int g = 0; g < num_gpus; ++g) {
      (void)hipSetDevice(device_ids[g]);
      hipError_t e = hipStreamSynchronize(streams[g]);
      if (e != hipSuccess) {
        int none = 0;
        restore_error.compare_exchange_strong(none, (int)e);
      }
    }
    for (int g = 0; g < (int)dma_streams.size(); ++g)
      for (hipStream_t s : {dma_streams[g], dma_streams2[g]})
        if (s) {
          (void)hipSetDevice(device_ids[g]);
          (void)hipStreamSynchronize(s);
        }
    for (auto &b : batches)
      for (int g = 0; g < num_gpus; ++g) {
        (void)hipSetDevice(device_ids[g]);
        if (b->done[g])
          (void)hipEventDestroy(b->done[g]);
      }
    batches.clear();
    layer_batch.clear();
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

// Devices, eventfd table and streams: what both constructors share.
int finish_create(std::unique_ptr<fkv_layerwise> &g, const int64_t *gpu_device_ids,
                  const int32_t *layer_eventfds, int num_layer_eventfds) {
  using namespace fkv;
  if (num_layer_eventfds > 0) {
    const int per_counter = g->tp_size * g->num_layers;
    if (!layer_eventfds || num_layer_eventfds % per_counter != 0)
      return fail(FKV_ERR_INVALID_ARG,
                  "layer_eventfds must hold a multiple of tp_size*num_layers = %d entries, got %d",
                  per_counter, num_layer_eventfds);
    g->eventfds.assign(layer_eventfds, layer_eventfds + num_layer_eventfds);
    g->num_counters = num_layer_eventfds / per_counter;
  }
  for (int i = 0; i < g->num_gpus; ++i)
    g->device_ids.push_back((int)gpu_device_ids[i]);
  DeviceGuard restore(-1);
  g->streams.assign(g->num_gpus, nullptr);
  g->dma_streams.assign(g->num_gpus, nullptr);
  g->dma_streams2.assign(g->num_gpus, nullptr);
  g->dma_turn.assign(g->num_gpus, 0u);
  g->alt_streams.assign(g->num_gpus, nullptr);
  g->alt_join.assign(g->num_gpus, nullptr);
  for (int i = 0; i < g->num_gpus; ++i) {
    hipError_t e = hipSetDevice(g->device_ids[i]);
    if (e == hipSuccess)
      e = pooled_stream_acquire(g->device_ids[i], true, &g->streams[i]);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      for (int k = 0; k < i; ++k) {
        (void)hipSetDevice(g->device_ids[k]);
        pooled_stream_release(g->device_ids[k], true, g->streams[k]);
      }
      (void)hipSetDevice(restore.device());
      return fail(FKV_ERR_RUNTIME, "stream creation on device %d failed: %s", g->device_ids[i],
                  hipGetErrorString(e));
    }
  }
  (void)hipSetDevice(restore.device());
  return FKV_OK;
}

// What a call asks for that every transfer of it shares.
struct EngineChoice {
  int use_ce_transfer = 0;
  int transfer_cta_num = 0;
};

fkv_transfer_desc describe(const fkv_layerwise *g, const Lane &lane, int gpu, int start,
                           int layers, const EngineChoice &c) {
  const Source &s = *lane.src;
  fkv_transfer_desc d{};
  d.backend = s.backend;
  d.num_layers_total = s.num_layers;
  d.gpu_tensor_ptrs = s.gpu_ptrs.data() + (size_t)gpu * s.num_tensors_per_gpu;
  d.num_gpu_tensor_ptrs = s.num_tensors_per_gpu;
  d.device = g->device_ids[gpu];
  d.gpu_kv_stride = s.kv_strides[gpu];
  d.gpu_block_stride = s.block_strides[gpu];
  d.gpu_layer_stride = s.layer_strides[gpu];
  d.gpu_startoff_inside_chunks = 0;
  d.cpu_ptr = lane.cpu_ptr;
  d.cpu_kv_stride = lane.cpu_kv_stride;
  d.cpu_layer_stride = lane.cpu_layer_stride;
  d.cpu_block_stride = lane.cpu_block_stride;
  d.cpu_startoff_inside_chunks = lane.cpu_off[gpu];
  d.chunk_size = s.chunk_sizes[gpu];
  d.start_layer_id = start;
  d.num_layers = layers;
  d.kv_dim = lane.kv_dim;
  d.num_blocks = lane.num_blocks;
  d.gpu_block_ids = lane.gpu_ids;
  d.cpu_block_ids = lane.cpu_ids;
  d.is_host_to_device = 1;
  d.use_ce_transfer = c.use_ce_transfer;
  d.transfer_num_cta = c.transfer_cta_num;
  d.sync = 0;
  d.ce = g->ce;
  return d;
}

// Enqueues every batch of the restore that is being set up, in order, records the batch
// events and hands the plan memory back; `rc` is the status of the set-up so far (a
// failed set-up enqueues nothing).  Runs on the calling thread, or on the group's
// launching thread where host threads gather rows.  Every item goes the way its lane
// was set up for: through the copy engines and a staging buffer (one copy per run of
// host blocks, or rows gathered first), else by kernel (`choice.use_ce_transfer == 0`)
// or through the copy-engine strategies of fkv_transfer_kv_blocks.
int launch_batches(fkv_layerwise *g, std::vector<Lane> &lanes, const EngineChoice &choice,
                   bool on_feeder, int rc) {
  using namespace fkv;
  DeviceGuard restore(-1);
  const bool direct = choice.use_ce_transfer == 0;
  const int num_batches = (int)g->batches.size();
  const int give_up_at = policy_of(g->device_ids[0]).test_fail_restore_batch; // tests only
  // Fewer batches than this and the call is bound by the host's launches, not by the gaps
  // between them on the device (8 batches of 256 KiB: 0.15 ms either way).
  constexpr int kAltMinBatches = 12;
  std::vector<char> two_dma_streams(g->num_gpus);
  std::vector<int64_t> alt_max_bytes(g->num_gpus, 0); // batches by kernel up to this size alternate
  for (int i = 0; i < g->num_gpus; ++i) {
    const fkv_launch_policy pol = policy_of(g->device_ids[i]);
    two_dma_streams[i] = pol.staged_dma_streams >= 2;
    if (!direct || pol.kernel_alt_stream_kb <= 0 || num_batches < kAltMinBatches || rc != FKV_OK)
      continue;
    (void)hipSetDevice(g->device_ids[i]);
    if (!g->alt_streams[i] &&
        pooled_stream_acquire(g->device_ids[i], true, &g->alt_streams[i]) != hipSuccess) {
      (void)hipGetLastError(); // everything on the one stream then
      g->alt_streams[i] = nullptr;
      continue;
    }
    if (!g->alt_join[i] &&
        hipEventCreateWithFlags(&g->alt_join[i], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      g->alt_join[i] = nullptr;
      continue;
    }
    alt_max_bytes[i] = (int64_t)pol.kernel_alt_stream_kb * 1024;
  }
  std::vector<char> alt_used(g->num_gpus, 0);
  try { // an exception ends the launches like an error: the plans below are given back either way
    for (int b = 0; b < num_batches && rc == FKV_OK; ++b) {
      if (give_up_at > 0 && b == give_up_at - 1) {
        rc = fail(FKV_ERR_RUNTIME, "layerwise restore made to give up before batch %d (test_fail_restore_batch)", b);
        break;
      }
      fkv_layerwise::Batch &batch = *g->batches[b];
      for (int i = 0; i < g->num_gpus && rc == FKV_OK; ++i) {
        (void)hipSetDevice(g->device_ids[i]);
        // the members of one batch that go by kernel go out together: up to kCopyMaxJobs per launch
        const KernelPlan *plans[kCopyMaxJobs];
        int first[kCopyMaxJobs], count[kCopyMaxJobs];
        std::vector<const Item *> by_kernel, by_strategy;
        auto account = [&](const Item &it) {
          const Lane &lane = lanes[it.lane];
          stats().calls.fetch_add(1, std::memory_order_relaxed);
          stats().bytes_h2d.fetch_add((uint64_t)lane.num_blocks * it.layers * lane.kv_dim *
                                          (uint64_t)lane.src->chunk_sizes[i],
                                      std::memory_order_relaxed);
        };
        for (const Item &it : batch.items) {
          if (rc != FKV_OK)
            break;
          Lane &lane = lanes[it.lane];
          const StagedPlan *sp =
              i < (int)lane.staged.size() && lane.staged[i].usable ? &lane.staged[i] : nullptr;
          if (!sp || (b == 0 && sp->first_by_kernel)) {
            (direct ? by_kernel : by_strategy).push_back(&it);
            continue;
          }
          // gathered batches are enqueued one by one as their rows become ready: nothing to hide
          // there, and next to other work of the process the second stream cost 1 % (c3 with
          // scattered host blocks behind c3 in one process: 42.3 ms against 41.9 ms)
          const bool second = two_dma_streams[i] && g->dma_streams2[i] && sp->route == kRouteRuns &&
                              (g->dma_turn[i]++ & 1u);
          const hipStream_t dma = second ? g->dma_streams2[i] : g->dma_streams[i];
          if (sp->route == kRouteGathered)
            rc = gathered_launch(*sp, g->rings[{it.lane, i}], g->pinned_rings[{it.lane, i}],
                                 *g->crew, lane.plans[i], it.start_layer, it.layers, dma,
                                 g->streams[i]);
          else
            rc = staged_launch(*sp, g->rings[{it.lane, i}], lane.plans[i], it.start_layer, it.layers,
                               dma, g->streams[i]);
          if (rc == FKV_OK)
            account(it);
        }
        // a small batch that goes by kernel as a whole: every other one on the second stream,
        // from the third on (the first one has the link to itself and lands as early as it can)
        hipStream_t batch_stream = g->streams[i];
        if (alt_max_bytes[i] > 0 && b >= 2 && !(b & 1) && !by_kernel.empty() &&
            by_kernel.size() == batch.items.size()) {
          int64_t bytes = 0;
          for (const Item *it : by_kernel) {
            const Lane &lane = lanes[it->lane];
            bytes += (int64_t)lane.num_blocks * it->layers * lane.kv_dim * lane.src->chunk_sizes[i];
          }
          // the second stream starts behind the first batch, which is behind the plan uploads
          if (bytes <= alt_max_bytes[i] &&
              (alt_used[i] ||
               hipStreamWaitEvent(g->alt_streams[i], g->batches[0]->done[i], 0) == hipSuccess)) {
            batch_stream = g->alt_streams[i];
            alt_used[i] = 1;
            stats().second_stream_batches.fetch_add(1, std::memory_order_relaxed);
          } else {
            (void)hipGetLastError();
          }
        }
        for (size_t k = 0; k < by_kernel.size() && rc == FKV_OK; k += kCopyMaxJobs) {
          const int n = (int)std::min<size_t>(kCopyMaxJobs, by_kernel.size() - k);
          for (int j = 0; j < n; ++j) {
            const Item &it = *by_kernel[k + j];
            plans[j] = &lanes[it.lane].plans[i];
            first[j] = it.start_layer;
            count[j] = it.layers;
          }
          rc = kernel_plans_launch(plans, first, count, n, batch_stream);
          for (int j = 0; j < n && rc == FKV_OK; ++j)
            account(*by_kernel[k + j]);
        }
        for (size_t k = 0; k < by_strategy.size() && rc == FKV_OK; ++k) {
          const Item &it = *by_strategy[k];
          fkv_transfer_desc d = describe(g, lanes[it.lane], i, it.start_layer, it.layers, choice);
          rc = fkv_transfer_kv_blocks(&d, g->streams[i]); // does its own accounting
          (void)hipSetDevice(g->device_ids[i]);
        }
        if (rc != FKV_OK)
          break;
        hipError_t e = hipEventRecord(batch.done[i], batch_stream);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          rc = fail(FKV_ERR_RUNTIME, "layerwise_transfer failed on GPU %d: %s", i,
                    hipGetErrorString(e));
        }
      }
      if (rc == FKV_OK)
        g->gate.publish(b + 1);
    }
  } catch (...) {
    rc = caught("launches of a layerwise restore");
  }
  // The second stream joins the first: what follows on `streams` (the release of the plan
  // memory, a synchronize, the next call) is behind every batch.
  for (int i = 0; i < g->num_gpus; ++i) {
    if (!alt_used[i])
      continue;
    (void)hipSetDevice(g->device_ids[i]);
    hipError_t e = hipEventRecord(g->alt_join[i], g->alt_streams[i]);
    if (e == hipSuccess)
      e = hipStreamWaitEvent(g->streams[i], g->alt_join[i], 0);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      (void)hipStreamSynchronize(g->alt_streams[i]); // the host waits instead
    }
  }
  std::string saved_error = fkv_last_error();
  for (Lane &lane : lanes)
    for (int i = 0; i < (int)lane.plans.size(); ++i) {
      (void)hipSetDevice(g->device_ids[i]);
      kernel_plan_release(&lane.plans[i], g->streams[i]);
      if (i < (int)lane.staged.size())
        staged_plan_release(&lane.staged[i], g->streams[i]);
    }
  if (rc != FKV_OK) {
    // Drain what was enqueued; nothing more of this call is announced.
    for (int i = 0; i < g->num_gpus; ++i) {
      (void)hipSetDevice(g->device_ids[i]);
      if (i < (int)g->dma_streams.size())
        for (hipStream_t s : {g->dma_streams[i], g->dma_streams2[i]})
          if (s)
            (void)hipStreamSynchronize(s);
      if (i < (int)g->alt_streams.size() && g->alt_streams[i])
        (void)hipStreamSynchronize(g->alt_streams[i]);
      (void)hipStreamSynchronize(g->streams[i]);
    }
    if (!on_feeder) // on the launching thread consumers may be reading the table
      g->layer_batch.assign(g->num_layers, -1);
    (void)hipSetDevice(restore.device());
    (void)hipGetLastError();
    return fail(rc, "%s", saved_error.c_str());
  }
  (void)hipSetDevice(restore.device());
  return FKV_OK;
}

} // namespace

extern "C" {

int fkv_layerwise_create(const fkv_layerwise_params *p, fkv_layerwise **out) try {
  using namespace fkv;
  clear_error();
  if (!p || !out || p->num_gpus < 1 || p->num_tensors_per_gpu < 1 || p->num_layers < 1 ||
      p->tp_size < 1 || !p->gpu_block_ptrs_flat || !p->gpu_kv_strides ||
      !p->gpu_block_strides || !p->gpu_layer_strides || !p->gpu_chunk_sizes ||
      !p->gpu_device_ids)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_create: bad arguments");
  if (backend_of(p->num_tensors_per_gpu, p->num_layers) < 0) // csrc/layerwise.cpp:586-595
    return fail(FKV_ERR_RUNTIME, "Unsupported GPU block type: %d", p->num_tensors_per_gpu);
  auto g = std::make_unique<fkv_layerwise>();
  g->num_gpus = p->num_gpus;
  g->num_layers = p->num_layers;
  g->tp_size = p->tp_size;
  g->cpu_blocks = p->cpu_blocks_ptr;
  g->ce = p->ce;
  fkv_layer_group in{};
  in.num_layers = p->num_layers;
  in.num_tensors_per_gpu = p->num_tensors_per_gpu;
  in.gpu_block_ptrs_flat = p->gpu_block_ptrs_flat;
  in.gpu_kv_strides = p->gpu_kv_strides;
  in.gpu_block_strides = p->gpu_block_strides;
  in.gpu_layer_strides = p->gpu_layer_strides;
  in.gpu_chunk_sizes = p->gpu_chunk_sizes;
  g->groups.resize(1);
  fill_source(g->groups[0], in, p->num_gpus);
  FKV_TRY(finish_create(g, p->gpu_device_ids, p->layer_eventfds, p->num_layer_eventfds));
  *out = g.release();
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_create_multi_group(const fkv_layerwise_mg_params *p, fkv_layerwise **out) try {
  using namespace fkv;
  clear_error();
  if (!p || !out || p->num_gpus < 1 || p->num_original_layers < 1 || p->tp_size < 1 ||
      p->num_groups < 1 || !p->groups || !p->gpu_device_ids)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_create_multi_group: bad arguments");
  auto g = std::make_unique<fkv_layerwise>();
  g->num_gpus = p->num_gpus;
  g->num_layers = p->num_original_layers;
  g->tp_size = p->tp_size;
  g->multi_group = true;
  g->cpu_blocks = p->cpu_blocks_ptr;
  g->ce = p->ce;
  g->groups.resize(p->num_groups);
  for (int gi = 0; gi < p->num_groups; ++gi) {
    if (!fill_source(g->groups[gi], p->groups[gi], p->num_gpus))
      return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_create_multi_group: group %d is incomplete",
                  gi);
    if (g->groups[gi].backend < 0) // csrc/layerwise.cpp:792-806
      return fail(FKV_ERR_RUNTIME,
                  "[LayerwiseTransferGroup multi-group] group %d has unsupported "
                  "tensors_per_gpu=%d for num_layers=%d",
                  gi, g->groups[gi].num_tensors_per_gpu, g->groups[gi].num_layers);
  }
  FKV_TRY(fill_members(g->members, p->num_original_layers, p->member_offsets, p->members,
                       g->groups, "fkv_layerwise_create_multi_group"));
  FKV_TRY(finish_create(g, p->gpu_device_ids, p->layer_eventfds, p->num_layer_eventfds));
  *out = g.release();
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_init_swa(fkv_layerwise *g, const fkv_layer_group *swa,
                           void *swa_cpu_blocks_ptr) try {
  using namespace fkv;
  clear_error();
  if (!g || !swa || !swa_cpu_blocks_ptr)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_init_swa: null argument");
  if (g->has_swa)
    return fail(FKV_ERR_RUNTIME, "[LayerwiseTransferGroup] SWA was already initialized");
  // The sidecar holds one ring per layer of the model (csrc/layerwise.cpp:180-190).
  fkv_layer_group in = *swa;
  in.num_layers = g->num_layers;
  Source s;
  if (!fill_source(s, in, g->num_gpus))
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_init_swa: incomplete group description");
  if (s.backend < 0)
    return fail(FKV_ERR_RUNTIME, "Unsupported SWA GPU block type: %d", s.num_tensors_per_gpu);
  g->retire_previous();
  g->swa_groups.assign(1, s);
  g->swa_members.clear();
  g->swa_cpu_blocks = swa_cpu_blocks_ptr;
  g->has_swa = true;
  g->swa_multi_group = false;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_init_swa_multi_group(fkv_layerwise *g, const fkv_layer_group *groups,
                                       int32_t num_groups, const int32_t *member_offsets,
                                       const fkv_layer_member *members,
                                       void *swa_cpu_blocks_ptr) try {
  using namespace fkv;
  clear_error();
  if (!g || !groups || num_groups < 1)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_init_swa_multi_group: null argument");
  if (g->has_swa) // csrc/layerwise.cpp:378-382
    return fail(FKV_ERR_RUNTIME,
                "[LayerwiseTransferGroup] init_swa_multi_group() called but SWA was "
                "already initialized (uniform or multi-group)");
  if (!swa_cpu_blocks_ptr) // :383-387
    return fail(FKV_ERR_RUNTIME,
                "[LayerwiseTransferGroup] init_swa_multi_group() requires non-empty "
                "swa_cpu_blocks");
  std::vector<Source> srcs(num_groups);
  for (int gi = 0; gi < num_groups; ++gi) {
    if (!fill_source(srcs[gi], groups[gi], g->num_gpus))
      return fail(FKV_ERR_INVALID_ARG,
                  "fkv_layerwise_init_swa_multi_group: group %d is incomplete", gi);
    if (srcs[gi].backend < 0) // :335-346
      return fail(FKV_ERR_RUNTIME,
                  "[LayerwiseTransferGroup SWA multi-group] group %d has unsupported "
                  "tensors_per_gpu=%d for num_layers=%d",
                  gi, srcs[gi].num_tensors_per_gpu, srcs[gi].num_layers);
  }
  MemberTable table;
  FKV_TRY(fill_members(table, g->num_layers, member_offsets, members, srcs,
                       "fkv_layerwise_init_swa_multi_group"));
  g->retire_previous();
  g->swa_groups = std::move(srcs);
  g->swa_members = std::move(table);
  g->swa_cpu_blocks = swa_cpu_blocks_ptr;
  g->has_swa = true;
  g->swa_multi_group = true;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_transfer_call(fkv_layerwise *g, const fkv_layerwise_call *call) try {
  using namespace fkv;
  clear_error();
  if (!g || !call)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer_call: null argument");
  const fkv_layerwise_call &c = *call;
  if (c.multi_group && !g->multi_group) // csrc/layerwise.cpp:1335-1339
    return fail(FKV_ERR_RUNTIME,
                "[LayerwiseTransferGroup] layerwise_transfer_multi_group() invoked on "
                "a single-group instance; use layerwise_transfer() instead.");
  if (!c.multi_group && g->multi_group) // :975-979
    return fail(FKV_ERR_RUNTIME,
                "[LayerwiseTransferGroup] layerwise_transfer() invoked on a "
                "multi-group instance; use layerwise_transfer_multi_group() instead.");
  if (c.num_blocks < 0 || c.swa_num_blocks < 0 || c.kv_dim < 1)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer: num_blocks=%d swa_num_blocks=%d "
                "kv_dim=%d", c.num_blocks, c.swa_num_blocks, c.kv_dim);
  if (!g->multi_group &&
      (c.num_layers < 0 || c.num_layers > g->num_layers || c.layer_granularity < 1))
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_layerwise_transfer: num_layers=%d (group has %d) layer_granularity=%d",
                c.num_layers, g->num_layers, c.layer_granularity);
  if (c.num_blocks > 0 && (!c.gpu_block_ids || !c.cpu_block_ids))
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer: null block id list");
  if (!g->eventfds.empty() && (c.counter_id < 0 || c.counter_id >= g->num_counters))
    return fail(FKV_ERR_INVALID_ARG, "counter_id %d outside [0, %d)", c.counter_id,
                g->num_counters);
  if (c.notify_mode != FKV_NOTIFY_HOSTFUNC && c.notify_mode != FKV_NOTIFY_POLLING)
    return fail(FKV_ERR_INVALID_ARG, "unknown notify mode %d", c.notify_mode);
  // csrc/layerwise.cpp:1091, 1362: the sidecar moves only when ids came along
  const bool swa_active = g->has_swa && c.swa_num_blocks > 0;
  if (swa_active && (!c.swa_gpu_block_ids || !c.swa_cpu_block_ids))
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_transfer: null SWA block id list");

  g->retire_previous();
  FKV_TRY(g->take_restore_error("fkv_layerwise_transfer"));
  g->gate.reset();
  g->feed_lanes.clear();
  g->counter_id = c.counter_id;
  Range range("fkv layerwise%s H2D %d blocks, %d sidecar blocks", g->multi_group ? " multi-group" : "",
              c.num_blocks, c.swa_num_blocks);

  // csrc/layerwise.cpp:1112-1121, 1349-1360: only these three names are
  // meaningful for a restore; anything else is treated as "sharded".
  const char *mode = c.kv_shared_across_ranks_mode ? c.kv_shared_across_ranks_mode : "sharded";
  if (c.num_kv_heads == 1 && !is(mode, "sharded") && !is(mode, "all_write") &&
      !is(mode, "rank0_only")) {
    fprintf(stderr,
            "[fkv] warning: kv_shared_across_ranks_mode \"%s\" is not valid for layerwise "
            "restore, using sharded\n",
            mode);
    mode = "sharded";
  }

  // ---- lanes: [0, groups) main KV, [groups, groups + swa_groups) sidecar ----
  const int num_main = (int)g->groups.size();
  std::vector<Lane> lanes(num_main + (swa_active ? g->swa_groups.size() : 0));
  // host offset of a rank, csrc/layerwise.cpp:1143-1166, 1519-1526, 448-453
  auto rank_offsets = [&](int num_kv_heads, int64_t tp_stride, int64_t block_stride,
                          int num_blocks) {
    std::vector<int64_t> off(g->num_gpus);
    for (int i = 0; i < g->num_gpus; ++i) {
      off[i] = (int64_t)i * tp_stride;
      if (num_kv_heads == 1)
        off[i] = is(mode, "all_write") ? (int64_t)i * num_blocks * block_stride : 0;
    }
    return off;
  };
  for (int gi = 0; gi < num_main; ++gi) {
    const Source &s = g->groups[gi];
    Lane &l = lanes[gi];
    l.src = &s;
    l.gpu_ids = c.gpu_block_ids;
    l.cpu_ids = c.cpu_block_ids;
    l.num_blocks = c.num_blocks;
    l.kv_dim = c.kv_dim;
    if (g->multi_group) {
      l.cpu_ptr = static_cast<char *>(g->cpu_blocks) + s.cpu_offset_bytes;
      l.cpu_kv_stride = s.h2d_cpu_kv_stride;
      l.cpu_layer_stride = s.h2d_cpu_layer_stride;
      l.cpu_block_stride = s.cpu_block_stride;
      l.cpu_off = rank_offsets(c.num_kv_heads, s.cpu_tp_stride, s.cpu_block_stride, c.num_blocks);
    } else {
      l.cpu_ptr = g->cpu_blocks;
      l.cpu_kv_stride = c.h2d_cpu_kv_stride;
      l.cpu_layer_stride = c.h2d_cpu_layer_stride;
      l.cpu_block_stride = c.cpu_block_stride;
      l.cpu_off = rank_offsets(c.num_kv_heads, c.cpu_tp_stride, c.cpu_block_stride, c.num_blocks);
    }
  }
  if (swa_active)
    for (int si = 0; si < (int)g->swa_groups.size(); ++si) {
      const Source &s = g->swa_groups[si];
      Lane &l = lanes[num_main + si];
      l.src = &s;
      l.gpu_ids = c.swa_gpu_block_ids;
      l.cpu_ids = c.swa_cpu_block_ids;
      l.num_blocks = c.swa_num_blocks;
      l.kv_dim = 1; // csrc/layerwise.cpp:231, 1599
      if (g->swa_multi_group) {
        l.cpu_ptr = static_cast<char *>(g->swa_cpu_blocks) + s.cpu_offset_bytes;
        l.cpu_kv_stride = s.h2d_cpu_kv_stride;
        l.cpu_layer_stride = s.h2d_cpu_layer_stride;
        l.cpu_block_stride = s.cpu_block_stride;
        l.cpu_off = rank_offsets(1, s.cpu_tp_stride, s.cpu_block_stride, c.swa_num_blocks);
      } else {
        l.cpu_ptr = g->swa_cpu_blocks;
        l.cpu_kv_stride = c.swa_h2d_cpu_kv_stride;
        l.cpu_layer_stride = c.swa_h2d_cpu_layer_stride;
        l.cpu_block_stride = c.swa_cpu_block_stride;
        l.cpu_off.assign(g->num_gpus, 0); // :229
      }
    }

  // ---- batches ----
  DeviceGuard restore(-1);
  g->layer_batch.assign(g->num_layers, -1);
  auto new_batch = [&](int start_layer, int layers) -> fkv_layerwise::Batch & {
    auto batch = std::make_unique<fkv_layerwise::Batch>();
    batch->start_layer = start_layer;
    batch->layers = layers;
    batch->done.assign(g->num_gpus, nullptr);
    for (int l = start_layer; l < start_layer + layers; ++l)
      g->layer_batch[l] = (int)g->batches.size();
    g->batches.push_back(std::move(batch));
    return *g->batches.back();
  };
  auto add_item = [&](fkv_layerwise::Batch &b, int lane, int start, int layers) {
    if (lanes[lane].num_blocks == 0 || layers == 0)
      return;
    lanes[lane].used = true;
    b.items.push_back(Item{lane, start, layers});
  };
  if (!g->multi_group) {
    for (int start = 0; start < c.num_layers; start += c.layer_granularity) {
      const int n = std::min(c.layer_granularity, c.num_layers - start);
      fkv_layerwise::Batch &b = new_batch(start, n);
      add_item(b, 0, start, n);
      // csrc/layerwise.cpp:1202-1209; the uniform form only (:219-221)
      if (swa_active && !g->swa_multi_group)
        add_item(b, num_main, start, n);
      for (int i = 0; i < g->num_gpus; ++i)
        b.trace_bytes += (double)g->groups[0].chunk_sizes[i] * c.kv_dim * n * c.num_blocks;
    }
  } else {
    for (int orig = 0; orig < g->num_layers; ++orig) {
      const int swa_slots = // swa_slots_for_orig_, csrc/layerwise.cpp:431-440
          !swa_active ? 0 : g->swa_multi_group ? (int)g->swa_members[orig].size() : 1;
      if (g->members[orig].empty() && swa_slots == 0) {
        g->notify_layers(orig, 1); // nothing will ever land: announce now (:1437-1457)
        continue;
      }
      fkv_layerwise::Batch &b = new_batch(orig, 1);
      b.num_members = (int)g->members[orig].size();
      for (const fkv_layer_member &m : g->members[orig]) {
        add_item(b, m.group, m.local_layer, 1);
        for (int i = 0; i < g->num_gpus; ++i)
          b.trace_bytes += (double)g->groups[m.group].chunk_sizes[i] * c.kv_dim * c.num_blocks;
      }
      if (swa_active) {
        if (g->swa_multi_group)
          for (const fkv_layer_member &m : g->swa_members[orig])
            add_item(b, num_main + m.group, m.local_layer, 1);
        else
          add_item(b, num_main, orig, 1);
      }
    }
  }
  const int num_batches = (int)g->batches.size();
  for (auto &b : g->batches)
    for (int i = 0; i < g->num_gpus; ++i) {
      FKV_HIP_TRY(hipSetDevice(g->device_ids[i]));
      // a restore writes device memory only: no system-scope fence (see kBookkeepingEvent)
      FKV_HIP_TRY(hipEventCreateWithFlags(&b->done[i], kTimingEventNoFence));
    }
  FKV_HIP_TRY(hipSetDevice(g->device_ids[0]));
  FKV_HIP_TRY(hipEventCreateWithFlags(&g->started, kTimingEventNoFence));
  FKV_HIP_TRY(hipEventRecord(g->started, g->streams[0]));

  int rc = FKV_OK;
  // One plan per used lane and GPU, covering all layers of its group: the kernel path of
  // a restore that was asked for on the kernel, and the device side of the batches that go
  // through the copy engines and a staging buffer, whichever engine was asked for (a
  // restore with use_ce_transfer whose host blocks are scattered would otherwise issue a
  // copy command per block and layer: 8.7 GB/s on 512 blocks of 72 KiB).
  const EngineChoice choice{c.use_ce_transfer, c.transfer_cta_num};
  const bool direct = choice.use_ce_transfer == 0;
  try { // an exception part-way ends the call like an error: launch_batches gives back what was built
    for (Lane &lane : lanes) {
      if (!lane.used || rc != FKV_OK)
        continue;
      lane.plans.resize(g->num_gpus);
      lane.staged.resize(g->num_gpus);
      const int layers = g->multi_group || lane.src != &g->groups[0] ? lane.src->num_layers
                                                                     : c.num_layers;
      const int lane_index = (int)(&lane - lanes.data());
      for (int i = 0; i < g->num_gpus && rc == FKV_OK; ++i) {
        fkv_transfer_desc d = describe(g, lane, i, 0, layers, choice);
        rc = validate(d);
        if (rc != FKV_OK)
          break;
        (void)hipSetDevice(g->device_ids[i]);
        // A host pool the device cannot read (ordinary pageable memory) still serves a
        // restore whose rows host threads gather; only the kernel path itself needs more.
        rc = kernel_plan_build(d, g->streams[i], &lane.plans[i], /*host_optional=*/true);
        if (rc != FKV_OK) {
          if (direct)
            break;
          clear_error(); // the copy-engine strategies need no plan
          rc = FKV_OK;
          continue;
        }
        rc = staged_plan_build(d, g->multi_group ? 1 : c.layer_granularity,
                               g->rings[{lane_index, i}], g->pinned_rings[{lane_index, i}],
                               g->streams[i], &lane.staged[i], lane.plans[i].host_visible,
                               /*kernel_allowed=*/direct, /*several_gpus=*/g->num_gpus > 1);
        if (rc == FKV_OK && lane.staged[i].usable && !g->dma_streams[i]) {
          hipError_t e = pooled_stream_acquire(g->device_ids[i], true, &g->dma_streams[i]);
          if (e != hipSuccess) {
            (void)hipGetLastError();
            g->dma_streams[i] = nullptr;
            staged_plan_release(&lane.staged[i], g->streams[i]); // kernel path then
          } else if (pooled_stream_acquire(g->device_ids[i], true, &g->dma_streams2[i]) !=
                     hipSuccess) {
            (void)hipGetLastError();
            g->dma_streams2[i] = nullptr; // all copies on the first then
          }
        }
        if (rc == FKV_OK && !lane.staged[i].usable) {
          if (!direct) // the strategies of the copy-engine path take it from here
            kernel_plan_release(&lane.plans[i], g->streams[i]);
          else if (!lane.plans[i].host_visible)
            rc = fail(FKV_ERR_INVALID_ARG,
                      "cpu_tensor at %p is not device-visible (allocate it pinned or register it "
                      "before a kernel transfer), and the restore cannot go through gathered rows "
                      "either (staged_gather of the launch policy, batch size)",
                      d.cpu_ptr);
        }
      }
    }
  } catch (...) {
    rc = caught("plans of a layerwise restore");
  }
  // Staging memory that several restores in a row had no use for goes back (a group
  // with many lanes would otherwise hold buffers for every route it ever took).
  constexpr int kRingIdleCalls = 8;
  for (auto &r : g->rings) {
    if (!r.second.touched && !r.second.buf.empty() && ++r.second.idle_calls >= kRingIdleCalls) {
      (void)hipSetDevice(g->device_ids[r.first.second]);
      r.second.release();
    }
    r.second.touched = false;
  }
  for (auto &r : g->pinned_rings) {
    if (!r.second.touched && !r.second.buf.empty() && ++r.second.idle_calls >= kRingIdleCalls) {
      (void)hipSetDevice(g->device_ids[r.first.second]);
      r.second.release();
    }
    r.second.touched = false;
  }
  // Rows gathered by host threads: the restore is launched from a thread of its own.
  bool gathered = false;
  for (const Lane &lane : lanes)
    for (const StagedPlan &sp : lane.staged)
      gathered = gathered || (sp.usable && sp.route == kRouteGathered);
  if (rc == FKV_OK && gathered) {
    const int helpers = gather_threads_of(policy_of(g->device_ids[0])) - 1;
    if (!g->crew || g->crew->helpers() != helpers) {
      try {
        g->crew = std::make_unique<HostCrew>(helpers);
      } catch (const std::exception &) { // no threads to be had: the launching thread gathers alone
        g->crew = std::make_unique<HostCrew>(0);
      }
    }
    g->feed_lanes = std::move(lanes);
    g->feed_use_ce = choice.use_ce_transfer;
    g->feed_num_cta = choice.transfer_cta_num;
    if (!direct) // the copy-engine strategies read the id lists when they are called
      for (Lane &lane : g->feed_lanes) {
        if (!lane.used)
          continue;
        lane.own_gpu_ids.assign(lane.gpu_ids, lane.gpu_ids + lane.num_blocks);
        lane.own_cpu_ids.assign(lane.cpu_ids, lane.cpu_ids + lane.num_blocks);
        lane.gpu_ids = lane.own_gpu_ids.data();
        lane.cpu_ids = lane.own_cpu_ids.data();
      }
    auto feed = [g] {
      const EngineChoice how{g->feed_use_ce, g->feed_num_cta};
      int frc;
      try {
        frc = launch_batches(g, g->feed_lanes, how, true, FKV_OK);
      } catch (...) { // a thread of the library ends with a status, not with std::terminate
        frc = caught("launching thread of a layerwise restore");
      }
      if (frc != FKV_OK) {
        g->feed_rc = frc; // read by others only after they have joined this thread
        g->feed_error = fkv_last_error();
        g->gate.fail();
      }
    };
    try {
      g->feeder = std::thread(feed);
    } catch (const std::exception &) {
      feed(); // no thread to be had: the same work on the calling thread, which then blocks for it
    }
  } else {
    const int lrc = launch_batches(g, lanes, choice, false, rc);
    if (lrc != FKV_OK) {
      (void)hipSetDevice(restore.device());
      return lrc;
    }
  }
  // The launching thread gave up: nothing of the call is announced from here on.
  auto launch_failure = [&]() {
    g->join_feeder();
    g->gate.clear_failure();
    (void)hipSetDevice(restore.device());
    return fail(g->feed_rc ? g->feed_rc : FKV_ERR_RUNTIME, "%s", g->feed_error.c_str());
  };

  if (c.notify_mode == FKV_NOTIFY_POLLING) {
    g->poller_stop.store(false, std::memory_order_release);
    // Nobody listens when no eventfd table was given: in-process consumers wait
    // on the batch events directly, so there is nothing to poll for.
    if (num_batches > 0 && !g->eventfds.empty()) {
      try {
        g->poller = std::thread([g] { g->poll_loop(); });
      } catch (const std::exception &) {
        g->poll_loop(); // no thread to be had: the calling thread announces the layers, and blocks for it
      }
    }
  } else {
    // announce every batch as soon as all GPUs have finished it, in order
    for (int b = 0; b < num_batches; ++b) {
      if (!g->gate.wait(b))
        return launch_failure();
      for (int i = 0; i < g->num_gpus; ++i) {
        (void)hipSetDevice(g->device_ids[i]);
        hipError_t e = quiet_event_wait(g->batches[b]->done[i], g->device_ids[i], 0);
        if (e != hipSuccess) {
          (void)hipGetLastError();
          (void)hipSetDevice(restore.device());
          return fail(FKV_ERR_RUNTIME, "layerwise_transfer failed on GPU %d: %s", i,
                      hipGetErrorString(e));
        }
      }
      g->notify(*g->batches[b]);
    }
    g->join_feeder();
    for (int i = 0; i < g->num_gpus; ++i) { // csrc/layerwise.cpp:1249-1256, 1634-1642
      (void)hipSetDevice(g->device_ids[i]);
      hipError_t e = quiet_stream_wait(g->streams[i], g->device_ids[i]);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipSetDevice(restore.device());
        return fail(FKV_ERR_RUNTIME, "%s failed on GPU %d: %s",
                    g->multi_group ? "layerwise_transfer_multi_group" : "layerwise_transfer", i,
                    hipGetErrorString(e));
      }
    }
    if (c.enable_trace && num_batches > 0) {
      // per-batch line with the fields of csrc/layerwise.cpp:1281-1285, 1655-1661
      (void)hipSetDevice(g->device_ids[0]);
      float prev = 0;
      for (int b = 0; b < num_batches; ++b) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, g->started, g->batches[b]->done[0]) != hipSuccess) {
          (void)hipGetLastError();
          continue;
        }
        const fkv_layerwise::Batch &bt = *g->batches[b];
        const double mb = bt.trace_bytes / (1024.0 * 1024.0);
        const double dt = ms - prev;
        const double bw = dt > 0 ? mb / (dt / 1000.0) : 0.0;
        if (g->multi_group)
          fprintf(stderr,
                  "[XFER] type=layerwise_mg_h2d orig=%d members=%d gpus=%d sync_ms=%.3f "
                  "data=%.2fMB bw=%.0fMB/s\n",
                  bt.start_layer, bt.num_members, g->num_gpus, dt, mb, bw);
        else
          fprintf(stderr,
                  "[XFER] type=layerwise_h2d layer_range=[%d,%d) blocks=%d data=%.2fMB "
                  "sync_ms=%.3f bw=%.0fMB/s\n",
                  bt.start_layer, bt.start_layer + bt.layers, c.num_blocks, mb, dt, bw);
        prev = ms;
      }
    }
  }
  (void)hipSetDevice(restore.device());
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_transfer(fkv_layerwise *g, const int64_t *gpu_block_ids,
                           const int64_t *cpu_block_ids, int32_t num_blocks,
                           int64_t cpu_block_stride, int64_t h2d_cpu_kv_stride,
                           int64_t h2d_cpu_layer_stride, int64_t cpu_tp_stride,
                           int32_t transfer_cta_num, int32_t use_ce_transfer,
                           int32_t num_layers, int32_t layer_granularity, int32_t kv_dim,
                           int32_t num_kv_heads, int32_t counter_id, const char *mode,
                           int32_t notify_mode, int32_t enable_trace) try {
  fkv_layerwise_call c{};
  c.gpu_block_ids = gpu_block_ids;
  c.cpu_block_ids = cpu_block_ids;
  c.num_blocks = num_blocks;
  c.multi_group = 0;
  c.cpu_block_stride = cpu_block_stride;
  c.h2d_cpu_kv_stride = h2d_cpu_kv_stride;
  c.h2d_cpu_layer_stride = h2d_cpu_layer_stride;
  c.cpu_tp_stride = cpu_tp_stride;
  c.num_layers = num_layers;
  c.layer_granularity = layer_granularity;
  c.transfer_cta_num = transfer_cta_num;
  c.use_ce_transfer = use_ce_transfer;
  c.kv_dim = kv_dim;
  c.num_kv_heads = num_kv_heads;
  c.counter_id = counter_id;
  c.notify_mode = notify_mode;
  c.enable_trace = enable_trace;
  c.kv_shared_across_ranks_mode = mode;
  return fkv_layerwise_transfer_call(g, &c);
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_wait_layer(fkv_layerwise *g, int32_t gpu_index, int32_t layer,
                             void *consumer_stream) try {
  using namespace fkv;
  clear_error();
  if (!g || gpu_index < 0 || gpu_index >= g->num_gpus)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_wait_layer: bad group or GPU index");
  if (layer < 0 || layer >= (int)g->layer_batch.size())
    return fail(FKV_ERR_INVALID_ARG, "layer %d was not part of the last transfer", layer);
  const int b = g->layer_batch[layer];
  if (b < 0) {
    // An original layer without members or sidecar work: nothing is in flight.
    if (g->multi_group)
      return FKV_OK;
    return fail(FKV_ERR_INVALID_ARG, "layer %d was not part of the last transfer", layer);
  }
  // A batch whose rows are still being gathered has no event on its stream yet, and a
  // wait on an event that was never recorded returns at once: wait for the record first.
  if (!g->gate.wait(b))
    return fail(FKV_ERR_RUNTIME, "layer %d will not land: the restore failed while it was launched",
                layer);
  FKV_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(consumer_stream),
                                 g->batches[b]->done[gpu_index], 0));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_set_compute_stream(fkv_layerwise *g, int32_t gpu_index, void *compute_stream,
                                     int32_t *streams_sharing) try {
  using namespace fkv;
  clear_error();
  if (!g)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_set_compute_stream: null group");
  if (gpu_index < 0 || gpu_index >= g->num_gpus)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_set_compute_stream: gpu_index %d of %d GPUs",
                gpu_index, g->num_gpus);
  g->retire_previous(); // the streams below are swapped: nothing may be in flight on them
  const int i = gpu_index, device = g->device_ids[i];
  DeviceGuard guard(device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", device);
  // Every stream of the group on this GPU, also those a restore would only make when it
  // first needs them: probing then would wait for the engine's stream in mid-service.
  // A candidate that shares the engine's queue is held back until the end, so that the
  // next one from the pool, or a new one, is another stream.
  //
  // Beyond that, where the queues allow: the scatter stream and the two copy streams on
  // three queues of their own (a batch's copy, its scatter and the next batch's copy are in
  // flight together), the second kernel stream off the first one's.
  const hipStream_t compute = static_cast<hipStream_t>(compute_stream);
  constexpr int kCandidates = 8;
  std::vector<hipStream_t> held_back;
  int sharing = 0, rc = FKV_OK;
  struct Own {
    hipStream_t *stream;
    std::vector<hipStream_t *> apart_from; // wished for, not required
  };
  const Own owns[] = {{&g->streams[i], {}},
                      {&g->dma_streams[i], {&g->streams[i]}},
                      {&g->dma_streams2[i], {&g->streams[i], &g->dma_streams[i]}},
                      {&g->alt_streams[i], {&g->streams[i]}}};
  // Two streams go together when their kernels run at the same time and an event gets from
  // one to the other and back about as fast as from a stream to itself: with more than four
  // hardware queues some pairs pass the first test and take four times as long for the
  // second, and a restore hands an event over per layer (61 layers next to compute: 52 ms
  // instead of 42).
  double own_round_trip_us = 0;
  FKV_TRY(fkv_streams_hand_over_us(device, compute, compute, &own_round_trip_us));
  // measured: 10 us for a stream with itself, 21-23 us for ordinary pairs, over 100 us for
  // the pairs that share hardware
  const double slow_us = 2 * own_round_trip_us + 30;
  auto go_together = [&](hipStream_t x, hipStream_t y, bool *yes) -> int {
    int32_t concurrent = 0;
    FKV_TRY(fkv_streams_run_concurrently(device, x, y, &concurrent));
    *yes = concurrent != 0;
    if (*yes) {
      double us = 0;
      FKV_TRY(fkv_streams_hand_over_us(device, x, y, &us));
      *yes = us < slow_us;
    }
    return FKV_OK;
  };
  // 2: goes together with the engine's stream and with those of ours it should be apart
  // from, 1: with the engine's stream only, 0: shares the engine's queue or hardware
  auto rank_of = [&](hipStream_t candidate, const Own &o, int *rank) -> int {
    bool yes = false;
    FKV_TRY(go_together(compute, candidate, &yes));
    *rank = yes ? 2 : 0;
    for (hipStream_t *other : o.apart_from) {
      if (*rank != 2 || !*other)
        break;
      FKV_TRY(go_together(*other, candidate, &yes));
      if (!yes)
        *rank = 1;
    }
    return FKV_OK;
  };
  for (const Own &o : owns) {
    hipStream_t best = nullptr;
    int best_rank = -1;
    for (int attempt = 0; attempt < kCandidates && best_rank < 2; ++attempt) {
      if (best_rank == 1 && attempt >= kCandidates / 2)
        break; // good enough
      hipStream_t candidate = *o.stream;
      *o.stream = nullptr;
      if (!candidate && pooled_stream_acquire(device, true, &candidate) != hipSuccess) {
        (void)hipGetLastError();
        break;
      }
      int rank = 0;
      rc = rank_of(candidate, o, &rank);
      if (rc != FKV_OK || rank <= best_rank) {
        held_back.push_back(candidate);
        if (rc != FKV_OK)
          break;
        continue;
      }
      if (best)
        held_back.push_back(best);
      best = candidate;
      best_rank = rank;
    }
    *o.stream = best; // none: a restore makes the stream when it needs it, as without this call
    if (best && best_rank == 0)
      ++sharing;
    if (rc != FKV_OK)
      break;
  }
  if (!g->streams[i] && !held_back.empty()) { // the group always has its first stream
    g->streams[i] = held_back.back();
    held_back.pop_back();
  }
  for (hipStream_t s : held_back)
    pooled_stream_release(device, true, s);
  if (!g->streams[i]) // cannot be: the group was made with one and gives it up only for another
    return fail(FKV_ERR_RUNTIME, "fkv_layerwise_set_compute_stream: no stream left for GPU %d", i);
  if (streams_sharing)
    *streams_sharing = sharing;
  return rc;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_synchronize(fkv_layerwise *g) try {
  using namespace fkv;
  clear_error();
  if (!g)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_synchronize: null group");
  g->join_poller();
  DeviceGuard restore(-1);
  for (int i = 0; i < g->num_gpus; ++i) {
    FKV_HIP_TRY(hipSetDevice(g->device_ids[i]));
    FKV_HIP_TRY(quiet_stream_wait(g->streams[i], g->device_ids[i]));
  }
  (void)hipSetDevice(restore.device());
  return g->take_restore_error("fkv_layerwise_synchronize");
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_layerwise_batch_times_ms(fkv_layerwise *g, float *out_ms, int32_t capacity,
                                 int32_t *num_batches) try {
  using namespace fkv;
  clear_error();
  if (!g || !num_batches)
    return fail(FKV_ERR_INVALID_ARG, "fkv_layerwise_batch_times_ms: null argument");
  *num_batches = (int32_t)g->batches.size();
  g->join_feeder();
  if (g->gate.recorded() < (int)g->batches.size())
    return fail(FKV_ERR_RUNTIME, "fkv_layerwise_batch_times_ms: the restore was not launched completely");
  DeviceGuard restore(g->device_ids[0]);
  for (int b = 0; b < (int)g->batches.size() && b < capacity; ++b)
    FKV_HIP_TRY(hipEventElapsedTime(&out_ms[b], g->started, g->batches[b]->done[0]));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

void fkv_layerwise_destroy(fkv_layerwise *g) {
  if (!g)
    return;
  g->retire_previous();
  fkv::DeviceGuard restore(-1);
  for (auto &ring : g->rings) {
    (void)hipSetDevice(g->device_ids[ring.first.second]);
    ring.second.release();
  }
  for (auto &ring : g->pinned_rings) {
    (void)hipSetDevice(g->device_ids[ring.first.second]);
    ring.second.release();
  }
  g->crew.reset();
  for (int i = 0; i < g->num_gpus; ++i) {
    (void)hipSetDevice(g->device_ids[i]);
    // every stream is idle (retire_previous), so the next group of the process may have it
    if (i < (int)g->dma_streams.size())
      for (hipStream_t s : {g->dma_streams[i], g->dma_streams2[i]})
        fkv::pooled_stream_release(g->device_ids[i], true, s);
    if (i < (int)g->alt_streams.size()) {
      if (g->alt_streams[i]) {
        (void)hipStreamSynchronize(g->alt_streams[i]);
        fkv::pooled_stream_release(g->device_ids[i], true, g->alt_streams[i]);
      }
      if (g->alt_join[i])
        (void)hipEventDestroy(g->alt_join[i]);
    }
    fkv::pooled_stream_release(g->device_ids[i], true, g->streams[i]);
  }
  (void)hipSetDevice(restore.device());
  (void)hipGetLastError();
  delete g;
}

} // extern "C"
