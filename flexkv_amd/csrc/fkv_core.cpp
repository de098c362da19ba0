// Errors, counters, plan memory and the dispatcher of fkv_transfer_kv_blocks.
//
// Host side of what csrc/transfer.cu:164-313 does in the reference: pick the
// kernel path or the copy-engine path, enqueue it on the caller's stream,
// optionally wait and trace.
#include "fkv_internal.h"

#include <map>

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>

namespace fkv {

// ---- errors -------------------------------------------------------------
namespace {
thread_local std::string t_last_error;
thread_local int t_last_path = FKV_PATH_KERNEL;
} // namespace

int fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  t_last_error = buf;
  return code;
}
void clear_error() { t_last_error.clear(); }

int caught(const char *where) noexcept {
  try {
    try {
      throw;
    } catch (const std::bad_alloc &) {
      return fail(FKV_ERR_RUNTIME, "%s: out of host memory", where);
    } catch (const std::exception &e) {
      return fail(FKV_ERR_RUNTIME, "%s: %s", where, e.what());
    } catch (...) {
      return fail(FKV_ERR_RUNTIME, "%s: unknown exception", where);
    }
  } catch (...) { // not even the text could be kept
    return FKV_ERR_RUNTIME;
  }
}
void set_last_path(int path) { t_last_path = path; }

Stats &stats() {
  static Stats s;
  return s;
}

DeviceGuard::DeviceGuard(int device) : device_(device) {
  if (hipGetDevice(&prev_) != hipSuccess) {
    (void)hipGetLastError();
    ok_ = false;
    return;
  }
  if (device < 0) {
    device_ = prev_;
    return;
  }
  if (device != prev_) {
    if (hipSetDevice(device) != hipSuccess) {
      (void)hipGetLastError();
      ok_ = false;
      return;
    }
    switched_ = true;
  }
}
DeviceGuard::~DeviceGuard() {
  if (switched_)
    (void)hipSetDevice(prev_);
}

// ---- waits that leave the cores alone ------------------------------------------
namespace {
// Threads of the process that are waiting for device work inside the library right now.
std::atomic<int> g_waiting{0};
struct Waiting {
  int others; // that were waiting already when this one came
  Waiting() : others(g_waiting.fetch_add(1, std::memory_order_relaxed)) {}
  ~Waiting() { g_waiting.fetch_sub(1, std::memory_order_relaxed); }
};
// As many waits as this may use the runtime's own, which returns soonest and costs a core
// each: a worker that waits for one transfer at a time loses nothing, and a process with 64
// requests in flight keeps two cores busy instead of thirteen.
constexpr int kRuntimeWaits = 2;
// ... unless the work is known to take this long: polling then costs a few parts in a
// thousand (a sleep towards the expected end, a spin of at most 160 us around it), and a
// transfer of gigabytes no longer holds a core for its whole length.
constexpr int64_t kLongWaitNs = 20 * 1000 * 1000;
} // namespace

hipError_t quiet_event_wait(hipEvent_t event, int device, int64_t expected_ns) {
  const int setting = policy_peek(device).quiet_wait_us;
  const int limit_us = setting < 0 ? -setting : setting;
  Waiting here;
  if (setting == 0 || (setting > 0 && here.others < kRuntimeWaits && expected_ns < kLongWaitNs))
    return hipEventSynchronize(event);
  using clock = std::chrono::steady_clock;
  const auto t0 = clock::now();
  // Where the work is expected to end: sleep up to shortly before that, look closely around
  // it, and fall back to longer and longer sleeps when it takes longer (work of others
  // queued ahead, traffic the other way).
  constexpr int64_t kCloseNs = 80 * 1000;
  const auto close_from = t0 + std::chrono::nanoseconds(std::max<int64_t>(0, expected_ns - kCloseNs));
  const auto close_until = t0 + std::chrono::nanoseconds(std::max<int64_t>(30 * 1000, expected_ns + kCloseNs));
  int nap_us = 20;
  for (;;) {
    const hipError_t q = hipEventQuery(event);
    if (q != hipErrorNotReady)
      return q;
    (void)hipGetLastError(); // "not ready" is no error of the caller's
    const auto now = clock::now();
    if (now < close_from) {
      // never long at a stretch: a core that has slept for tens of milliseconds can take
      // milliseconds to come back (seen on a virtual machine: +2 to +5 ms on a 188 ms wait)
      std::this_thread::sleep_for(std::min<clock::duration>(
          (close_from - now) / 2 + std::chrono::microseconds(10), std::chrono::milliseconds(1)));
    } else if (now < close_until) {
      // spinning: the end is near
    } else {
      std::this_thread::sleep_for(std::chrono::microseconds(nap_us));
      nap_us = std::min(nap_us * 2, limit_us);
    }
  }
}

hipError_t quiet_stream_wait(hipStream_t stream, int device) {
  constexpr int kMaxDevices = 64;
  const int setting = device < 0 || device >= kMaxDevices ? 0 : policy_peek(device).quiet_wait_us;
  if (setting == 0 || (setting > 0 && g_waiting.load(std::memory_order_relaxed) < kRuntimeWaits)) {
    Waiting here;
    return hipStreamSynchronize(stream);
  }
  // one event per thread and device; with the system-scope fence, since the host may read
  // what the stream wrote
  struct Mine { // given back when the thread ends
    hipEvent_t of_device[kMaxDevices] = {};
    ~Mine() {
      for (hipEvent_t e : of_device)
        if (e)
          (void)hipEventDestroy(e);
      (void)hipGetLastError();
    }
  };
  thread_local Mine mine;
  hipEvent_t &ev = mine.of_device[device];
  if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    ev = nullptr;
    return hipStreamSynchronize(stream);
  }
  if (hipEventRecord(ev, stream) != hipSuccess) {
    (void)hipGetLastError();
    return hipStreamSynchronize(stream);
  }
  return quiet_event_wait(ev, device, 0);
}

// ---- pooled streams ---------------------------------------------------------
namespace {
struct StreamPool {
  std::mutex mu;
  std::map<std::pair<int, bool>, std::vector<hipStream_t>> idle;
};
StreamPool &stream_pool() {
  static StreamPool *p = new StreamPool(); // never destructed, see pooled_stream_acquire
  return *p;
}
} // namespace

hipError_t pooled_stream_acquire(int device, bool non_blocking, hipStream_t *out) {
  {
    StreamPool &p = stream_pool();
    std::lock_guard<std::mutex> lk(p.mu);
    auto &v = p.idle[{device, non_blocking}];
    if (!v.empty()) {
      *out = v.back();
      v.pop_back();
      return hipSuccess;
    }
  }
  return non_blocking ? hipStreamCreateWithFlags(out, hipStreamNonBlocking) : hipStreamCreate(out);
}

void pooled_stream_release(int device, bool non_blocking, hipStream_t stream) {
  if (!stream)
    return;
  StreamPool &p = stream_pool();
  std::lock_guard<std::mutex> lk(p.mu);
  p.idle[{device, non_blocking}].push_back(stream);
}

// ---- plan memory ---------------------------------------------------------
namespace {
bool env_flag(const char *name) {
  const char *v = std::getenv(name);
  return v && *v && std::strcmp(v, "0") != 0;
}
} // namespace

struct PlanSlot {
  uint8_t *host = nullptr;
  uint8_t *dev = nullptr;
  size_t cap = 0;
  hipEvent_t done = nullptr;
  // kPlanCounters claim counters in device memory for launches whose workgroups
  // claim their work (CopyKernelArgs::claim)
  uint64_t *counters = nullptr;
  bool busy = false;          // handed out, not yet released
  bool event_pending = false; // released behind an event that may not have fired
  int device = 0;
};

namespace {
struct PlanPool {
  std::mutex mu;
  // Slots are never freed: the pool outlives every stream that may still read
  // them, and tearing HIP objects down from a static destructor is unsafe.
  std::vector<PlanSlot *> slots;
  // The claim counters of a device's slots are cut from chunks that are allocated and
  // cleared for many slots at once: clearing is a copy the host waits for, and under load
  // that wait is long and holds up every thread that needs a slot (a process with four
  // hardware queues has the null stream on the queue of some transfer stream: 64 requests
  // in flight, one new slot, 24 ms during which no thread launched anything).  The first
  // slot of a device pays for it, when nothing of the library is in flight there.
  struct CounterChunk {
    uint64_t *base = nullptr;
    int handed_out = 0; // slots that have their counters from this chunk
  };
  std::map<int, CounterChunk> counter_chunks; // by device: the chunk that still has room
};
PlanPool &pool() {
  static PlanPool *p = new PlanPool();
  return *p;
}
constexpr size_t kPlanMinBytes = 64 * 1024;
constexpr int kPlanCounters = 1024;
constexpr int kPlanSlotsPerChunk = 256; // as many as the pool holds before it waits for the oldest

// kPlanCounters counters for a new slot of `device` (current); p.mu is held.
uint64_t *counters_for_new_slot(PlanPool &p, int device) {
  PlanPool::CounterChunk &chunk = p.counter_chunks[device];
  if (!chunk.base || chunk.handed_out == kPlanSlotsPerChunk) {
    // Cleared for tidiness and against a leftover whose high half happens to be the number
    // of the first launch that uses it; a launch takes a counter over whatever else it
    // holds (Shares::adopt).  A copy that has finished when it returns: a hipMemset on the
    // null stream can still be under way when the first kernel on a non-blocking stream
    // claims from the counters.
    const size_t count = (size_t)kPlanCounters * kPlanSlotsPerChunk;
    // FKV_TEST_DIRTY_COUNTERS=1 (tests): start them with garbage instead
    static const std::vector<uint64_t> zeros(
        count, env_flag("FKV_TEST_DIRTY_COUNTERS") ? 0xdeadbeef00000007ull : 0u);
    void *c = nullptr;
    if (hipMalloc(&c, count * sizeof(uint64_t)) != hipSuccess ||
        hipMemcpy(c, zeros.data(), count * sizeof(uint64_t), hipMemcpyHostToDevice) != hipSuccess) {
      (void)hipGetLastError();
      if (c)
        (void)hipFree(c);
      return nullptr;
    }
    chunk.base = static_cast<uint64_t *>(c); // an exhausted chunk stays with its slots
    chunk.handed_out = 0;
  }
  return chunk.base + (size_t)kPlanCounters * chunk.handed_out++;
}

bool slot_grow(PlanSlot *s, size_t bytes) {
  if (s->cap >= bytes)
    return true;
  size_t cap = kPlanMinBytes;
  while (cap < bytes)
    cap *= 2;
  if (s->host)
    (void)hipHostFree(s->host);
  if (s->dev)
    (void)hipFree(s->dev);
  s->host = s->dev = nullptr;
  s->cap = 0;
  void *h = nullptr, *d = nullptr;
  if (hipHostMalloc(&h, cap, hipHostMallocPortable | hipHostMallocMapped) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (hipMalloc(&d, cap) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipHostFree(h);
    return false;
  }
  s->host = static_cast<uint8_t *>(h);
  s->dev = static_cast<uint8_t *>(d);
  s->cap = cap;
  return true;
}
} // namespace

PlanSlot *plan_acquire(int device, size_t bytes) {
  PlanPool &p = pool();
  PlanSlot *pick = nullptr;
  PlanSlot *waitable = nullptr;
  {
    std::lock_guard<std::mutex> lk(p.mu);
    for (PlanSlot *s : p.slots) {
      if (s->busy || s->device != device)
        continue;
      if (s->event_pending) {
        hipError_t q = hipEventQuery(s->done);
        if (q == hipSuccess) {
          s->event_pending = false;
        } else {
          (void)hipGetLastError();
          if (!waitable)
            waitable = s;
          continue;
        }
      }
      if (!pick || (pick->cap < bytes && s->cap > pick->cap))
        pick = s;
      if (pick->cap >= bytes)
        break;
    }
    if (!pick && waitable && p.slots.size() >= 256) {
      pick = waitable; // pool is large enough: wait for the oldest user instead
    }
    if (!pick) {
      pick = new PlanSlot();
      pick->device = device;
      if (hipEventCreateWithFlags(&pick->done, kBookkeepingEvent) != hipSuccess) {
        (void)hipGetLastError();
        delete pick;
        fail(FKV_ERR_RUNTIME, "plan memory: hipEventCreate failed");
        return nullptr;
      }
      pick->counters = counters_for_new_slot(p, device);
      if (!pick->counters) {
        (void)hipEventDestroy(pick->done);
        delete pick;
        fail(FKV_ERR_RUNTIME, "plan memory: cannot allocate the claim counters");
        return nullptr;
      }
      p.slots.push_back(pick);
    }
    pick->busy = true;
  }
  if (pick->event_pending) {
    stats().plan_slot_waits.fetch_add(1, std::memory_order_relaxed);
    (void)hipEventSynchronize(pick->done);
    pick->event_pending = false;
  }
  if (!slot_grow(pick, bytes)) {
    std::lock_guard<std::mutex> lk(p.mu);
    pick->busy = false;
    fail(FKV_ERR_RUNTIME, "plan memory: cannot allocate %zu bytes of pinned/device memory",
         bytes);
    return nullptr;
  }
  return pick;
}

void plan_pool_counts(int *slots, int *handed_out) {
  PlanPool &p = pool();
  std::lock_guard<std::mutex> lk(p.mu);
  *slots = (int)p.slots.size();
  *handed_out = 0;
  for (const PlanSlot *s : p.slots)
    *handed_out += s->busy ? 1 : 0;
}

uint8_t *plan_host(PlanSlot *s) { return s->host; }
uint64_t *plan_counters(PlanSlot *s, int count) {
  return count <= kPlanCounters ? s->counters : nullptr;
}

int plan_publish(PlanSlot *s, size_t bytes, bool mirror, hipStream_t stream,
                 uint8_t **device_visible) {
  if (!mirror) {
    *device_visible = s->host; // hipHostMalloc memory: same address on the device
    return FKV_OK;
  }
  // A kernel, not hipMemcpyAsync: copies of different streams share the copy
  // engines' queues, where the small upload of one stream waits behind the upload
  // of another stream that is itself waiting for that stream's previous transfer.
  // With a put stream next to a get stream that tied the start of every get to the
  // end of a put (0.8 ms idle per 3.8 ms transfer).
  FKV_TRY(launch_plan_upload(s->dev, s->host, bytes, stream));
  *device_visible = s->dev;
  return FKV_OK;
}

void plan_release(PlanSlot *s, hipStream_t stream, bool drained) {
  if (!s)
    return;
  bool pending = false;
  if (!drained) {
    if (hipEventRecord(s->done, stream) == hipSuccess) {
      pending = true;
    } else {
      (void)hipGetLastError();
      (void)hipStreamSynchronize(stream);
    }
  }
  std::lock_guard<std::mutex> lk(pool().mu);
  s->event_pending = pending;
  s->busy = false;
}

// ---- kernel path ---------------------------------------------------------
namespace {
int env_int(const char *name, int fallback) {
  const char *v = std::getenv(name);
  if (!v || !*v)
    return fallback;
  return (int)std::strtol(v, nullptr, 0); // decimal, 0x.. or 0.. as written
}
} // namespace

int default_num_cta(bool is_h2d) {
  // same default as FLEXKV_TRANSFER_NUM_CTA_{H2D,D2H} (flexkv/common/config.py:779-780)
  static const int h2d = env_int("FKV_NUM_CTA_H2D", 4);
  static const int d2h = env_int("FKV_NUM_CTA_D2H", 4);
  return is_h2d ? h2d : d2h;
}

// Launch shape of the link-bound kernel.  Measured on MI355X with 4 requested CTAs:
// GB/s over the link (a plain pinned hipMemcpy reaches 57.0 GPU->host / 57.3
// host->GPU) and the slowdown of a kernel running next to the copy (a 2048^3 bf16
// GEMM / fused attention / a streaming elementwise kernel):
//   host->GPU  16 x  64 lanes : 57.2 GB/s,  1.9x /  1.10x /  1.05x   <- default
//              24 x  64       : 57.4 GB/s,  2.9x /  1.16x /  1.10x
//              12 x 1024      : 57.1 GB/s, 16x   /  2.1x  / 11x (stalled until the copy ends)
//   GPU->host  48 x  64 lanes : 56.4 GB/s, streaming neighbour 2.7x   <- default
//              24 x  64       : 54.7 GB/s, streaming neighbour 1.9x
//              12 x 1024      : 56.6 GB/s, streaming neighbour 4.2x
// So every requested CTA becomes four (host->GPU) or twelve (GPU->host)
// single-wavefront workgroups: {h2d,d2h}_wg_per_cta and {h2d,d2h}_wg_threads of the
// launch policy.

// ---- both directions at once ---------------------------------------------
// A GPU->host and a host->GPU copy that share XCDs compete for the same
// memory-request queues: 62 GB/s in sum, against 87-90 GB/s when each direction
// keeps to its own half of the chip.  The library therefore remembers, per device
// and direction, the events recorded behind its most recent link-bound launches;
// a launch that finds the other direction still busy confines itself to its own
// XCDs (GPU->host: XCDs 1-2, host->GPU: 4-7) and asks for enough workgroups to
// saturate the link from there.  GPU->host keeps to two XCDs because the time a
// stream stands idle between two commands grows with the number of XCDs that
// post writes to the host at that moment: measured next to a writer on 1/2/3/4
// XCDs, a host->GPU stream with one small kernel between its copies idles
// 65/100/150/780 us per copy, while 48 workgroups write 43/48.5/49/50 GB/s; a
// writer that includes XCD 0 loses another 4 GB/s.  With the writer on two XCDs
// the reader also moves 55 instead of 49 GB/s.  A lone GPU->host transfer loses 2 %
// on two XCDs and nothing on three (1-3), a lone host->GPU transfer nothing on 4-7,
// so launches of 8 MiB and more (home_min_kb of the launch policy, -1: never) keep to these home
// XCDs even when the link is idle: a put launched alone and a get that arrives
// 1 ms later reach 93 GB/s instead of 61, in the other order 80 instead of 72.
// A direction also counts as busy for a short
// while after its last launch (busy_window_ms of the launch policy, default 20): with many
// small requests in flight the other direction is often between two kernels at
// the moment of a launch, and a full-chip launch would then collide with its next
// one.  Work recorded on the launching stream itself does not count: it has
// finished before the new launch starts.  Launches of other processes on the same
// GPU count through the board of fkv_linkboard.cpp.
// arbiter = 0 in the launch policy (FKV_LINK_ARBITER=0) switches this off.  Which
// XCDs these are on a given device is derived in fkv_policy.cpp.
namespace {
constexpr int kActivityRing = 16;
struct DirectionActivity {
  hipEvent_t ev[kActivityRing] = {};
  bool pending[kActivityRing] = {};
  hipStream_t stream[kActivityRing] = {};
  int64_t launched_ns[kActivityRing] = {}; // steady clock at launch
  int next = 0;
};
struct DeviceActivity {
  std::mutex mu;
  DirectionActivity dir[2]; // [0] GPU->host, [1] host->GPU
};
DeviceActivity &activity_of(int device) {
  static std::mutex mu;
  static std::map<int, DeviceActivity *> all; // entries live until the process ends
  std::lock_guard<std::mutex> lk(mu);
  DeviceActivity *&p = all[device];
  if (!p)
    p = new DeviceActivity();
  return *p;
}
int64_t steady_ns() {
  return std::chrono::duration_cast<std::chrono::nanoseconds>(
             std::chrono::steady_clock::now().time_since_epoch())
      .count();
}
} // namespace

bool link_direction_busy(int device, bool h2d, hipStream_t launching_stream) {
  DeviceActivity &a = activity_of(device);
  std::lock_guard<std::mutex> lk(a.mu);
  DirectionActivity &d = a.dir[h2d ? 1 : 0];
  const int64_t window_ns = (int64_t)policy_of(device).busy_window_ms * 1000000;
  const int64_t now = steady_ns();
  // launches of other processes on this GPU, as far as they post them
  bool busy = link_board_busy_elsewhere(device, h2d, window_ns);
  for (int i = 0; i < kActivityRing; ++i) {
    if (d.stream[i] != launching_stream && d.launched_ns[i] && now - d.launched_ns[i] < window_ns)
      busy = true;
    if (!d.pending[i])
      continue;
    if (hipEventQuery(d.ev[i]) == hipSuccess) {
      d.pending[i] = false;
    } else {
      (void)hipGetLastError();
      busy = busy || d.stream[i] != launching_stream;
    }
  }
  return busy;
}

void link_direction_mark(int device, bool h2d, hipStream_t stream, int64_t bytes) {
  const fkv_launch_policy pol = policy_of(device);
  if (pol.arbiter == 0)
    return;
  // what other processes get to see: the link is taken for about this long (the
  // estimate is low on purpose: rather a little too long than too short)
  link_board_post(device, h2d, bytes > 0 ? bytes / pol.link_gbps_estimate : 0);
  DeviceActivity &a = activity_of(device);
  std::lock_guard<std::mutex> lk(a.mu);
  DirectionActivity &d = a.dir[h2d ? 1 : 0];
  const int i = d.next;
  if (!d.ev[i] && hipEventCreateWithFlags(&d.ev[i], kBookkeepingEvent) != hipSuccess) {
    (void)hipGetLastError();
    d.ev[i] = nullptr;
    return;
  }
  if (hipEventRecord(d.ev[i], stream) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  d.pending[i] = true;
  d.stream[i] = stream;
  d.launched_ns[i] = steady_ns();
  d.next = (i + 1) % kActivityRing;
}

size_t kernel_plan_bytes(const fkv_transfer_desc &d) {
  return 2 * (size_t)d.num_layers * d.kv_dim * 8 + 2 * (size_t)d.num_blocks * 8;
}

int kernel_plan_fill(const fkv_transfer_desc &d, uint8_t *h, bool may_probe_device,
                     KernelPlan *out, bool host_optional) {
  // Device-visible alias of the host pool.  hipHostMalloc / torch pinned memory
  // map to the same address; hipHostRegister-ed memory may not.
  void *cpu_dev = nullptr;
  hipError_t e = hipHostGetDevicePointer(&cpu_dev, d.cpu_ptr, 0);
  out->host_visible = e == hipSuccess && cpu_dev;
  if (!out->host_visible) {
    (void)hipGetLastError();
    cpu_dev = nullptr;
    if (!host_optional)
      return fail(FKV_ERR_INVALID_ARG,
                  "cpu_tensor at %p is not device-visible (allocate it pinned or register it "
                  "before a kernel transfer): %s",
                  d.cpu_ptr, hipGetErrorString(e));
  }
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  const int lk = d.num_layers * d.kv_dim;
  const size_t tab_bytes = (size_t)lk * 8;
  const size_t ids_bytes = (size_t)d.num_blocks * 8;
  uint64_t *gbase = reinterpret_cast<uint64_t *>(h);
  uint64_t *cbase = reinterpret_cast<uint64_t *>(h + tab_bytes);
  uint64_t acc = (uint64_t)d.chunk_size | (uint64_t)d.gpu_block_stride |
                 (uint64_t)d.cpu_block_stride;
  for (int li = 0; li < d.num_layers; ++li) {
    const int64_t layer = (int64_t)d.start_layer_id + li;
    for (int kv = 0; kv < d.kv_dim; ++kv) {
      const uint64_t g = gpu_chunk_addr(d, layer, kv, 0);
      const uint64_t c =
          (uint64_t)(uintptr_t)cpu_dev + (uint64_t)(layer * d.cpu_layer_stride +
                                                    kv * d.cpu_kv_stride +
                                                    d.cpu_startoff_inside_chunks);
      gbase[li * d.kv_dim + kv] = g;
      cbase[li * d.kv_dim + kv] = out->host_visible ? c : 0;
      acc |= out->host_visible ? (g | c) : g;
    }
  }
  std::memcpy(h + 2 * tab_bytes, d.gpu_block_ids, ids_bytes);
  std::memcpy(h + 2 * tab_bytes + ids_bytes, d.cpu_block_ids, ids_bytes);
  // A CTA of the reference is 1024 threads on one SM (csrc/transfer.cu:176) and
  // its default of 4 CTAs is tuned for that hardware.  Here each requested CTA
  // becomes several small workgroups (see the note on the launch shape above).
  out->h2d = d.is_host_to_device != 0;
  const fkv_launch_policy pol = may_probe_device ? policy_of(device) : policy_peek(device);
  out->no_alloc = !may_probe_device;
  out->workgroups =
      (d.transfer_num_cta > 0 ? d.transfer_num_cta : default_num_cta(out->h2d)) *
      (out->h2d ? pol.h2d_wg_per_cta : pol.d2h_wg_per_cta);
  out->threads = out->h2d ? pol.h2d_wg_threads : pol.d2h_wg_threads;
  out->device = device;
  out->vec = common_vector_width(&acc, 1);
  out->kv_dim = d.kv_dim;
  out->num_layers = d.num_layers;
  out->num_blocks = d.num_blocks;
  out->chunk_size = d.chunk_size;
  out->gpu_block_stride = d.gpu_block_stride;
  out->cpu_block_stride = d.cpu_block_stride;
  return FKV_OK;
}

void kernel_plan_point(KernelPlan *out, const uint8_t *dv, uint64_t *claims) {
  const size_t tab_bytes = (size_t)out->num_layers * out->kv_dim * 8;
  const size_t ids_bytes = (size_t)out->num_blocks * 8;
  out->gpu_base = reinterpret_cast<const uint64_t *>(dv);
  out->cpu_base = reinterpret_cast<const uint64_t *>(dv + tab_bytes);
  out->gpu_ids = reinterpret_cast<const int64_t *>(dv + 2 * tab_bytes);
  out->cpu_ids = reinterpret_cast<const int64_t *>(dv + 2 * tab_bytes + ids_bytes);
  out->claims = claims;
}

int kernel_plan_build(const fkv_transfer_desc &d, hipStream_t stream, KernelPlan *out,
                      bool host_optional) {
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  const size_t plan_bytes = kernel_plan_bytes(d);
  PlanSlot *slot = plan_acquire(device, plan_bytes);
  if (!slot)
    return FKV_ERR_RUNTIME;
  int rc = kernel_plan_fill(d, plan_host(slot), /*may_probe_device=*/true, out, host_optional);
  if (rc != FKV_OK) {
    plan_release(slot, stream, true);
    return rc;
  }
  const fkv_launch_policy pol = policy_of(device);
  // Kernels read the plan from a device copy, which a small kernel uploads first,
  // or where it is, in the pinned slot.  Next to a transfer in the other direction
  // every command on a stream costs idle time, and the upload is one: two threads
  // that put and get 25 MB (100 MB) requests move 88.8 (95.4) instead of 87.0 (94.1)
  // GB/s without it.  A lone transfer is no faster for it and a multi-group restore
  // 1.5 % slower, so the plan is read in place only while the other direction is
  // busy.  plan_mirror of the launch policy = 1 / 0: always / never upload.
  const bool mirror_plan =
      pol.plan_mirror >= 0
          ? pol.plan_mirror != 0
          : !(pol.arbiter == 1 && link_direction_busy(device, !out->h2d, stream));
  uint8_t *dv = nullptr;
  rc = plan_publish(slot, plan_bytes, mirror_plan, stream, &dv);
  if (rc != FKV_OK) {
    plan_release(slot, stream, false);
    return rc;
  }
  out->slot = slot;
  kernel_plan_point(out, dv, plan_counters(slot, d.num_layers)); // nullptr: launches are not confined
  return FKV_OK;
}

namespace {
// The kernel's view of layers [l0, l0 + nl) of a plan.
CopyKernelArgs plan_job(const KernelPlan &p, int l0, int nl) {
  const uint64_t *gb = p.gpu_base + (size_t)l0 * p.kv_dim;
  const uint64_t *cb = p.cpu_base + (size_t)l0 * p.kv_dim;
  CopyKernelArgs a{};
  a.base_src = p.h2d ? cb : gb;
  a.base_dst = p.h2d ? gb : cb;
  a.ids_src = p.h2d ? p.cpu_ids : p.gpu_ids;
  a.ids_dst = p.h2d ? p.gpu_ids : p.cpu_ids;
  a.stride_src = p.h2d ? p.cpu_block_stride : p.gpu_block_stride;
  a.stride_dst = p.h2d ? p.gpu_block_stride : p.cpu_block_stride;
  a.chunk_bytes = p.chunk_size;
  a.num_blocks = p.num_blocks;
  a.lk = nl * p.kv_dim;
  a.vec = p.vec;
  a.nt_store = p.h2d ? 1 : 0;
  // Packed short chunks cost a wavefront more address arithmetic per request, so
  // such launches get half as many workgroups again.  Host->GPU, 2304-byte chunks:
  // 16 x 64 lanes reach 45 GB/s, 24 x 64 reach 55.8, 32 x 64 reach 56.2; GPU->host:
  // 48 x 64 lanes 50.7 GB/s, 72 x 64 52.5, 96 x 64 53.0.
  a.packed_grid_pct = 150; // replaced by the policy's when the launch is shaped
  a.xcd_mask = 0;
  a.claim = p.claims ? p.claims + l0 : nullptr; // a launch per first layer at most
  return a;
}

// Which XCDs, how many workgroups and how many ranges per workgroup a launch of
// `bytes` gets now; `a` is the (first) job of the launch.  Decided when a launch is
// made, not when its plan is built (a layerwise restore launches for tens of
// milliseconds after its plan was built): while the other direction is busy
// GPU->host keeps to its busy XCDs and host->GPU to its own; on an idle link large
// launches keep to their direction's home XCDs, so that a transfer of the other
// direction that starts while they run finds its own XCDs free.  On the home XCDs
// a launch gets no more workgroups than on all XCDs: what a copy costs the kernels
// next to it grows with their number (a 2048^3 GEMM takes 47 us next to 16 host->GPU
// workgroups, confined or not, and 67 us next to 24), and 16 on four XCDs already
// reach the link rate.
// Ranges per workgroup: next to a transfer in the other direction one each is best
// (finer ranges shift the balance towards GPU->host and lower the sum: two threads
// with 25 MB requests 88.9 against 87.5 GB/s).  On an idle link the neighbours are
// the engine's compute kernels, which slow down single workgroups of a copy, and
// with one range each the slowest one holds up the launch: a restore next to
// fused-attention calls moves 37 GB/s with one range per workgroup and 54 GB/s with
// two.
int shape_for_now(const KernelPlan &p, int64_t bytes, hipStream_t stream, CopyKernelArgs *a) {
  const fkv_launch_policy pol = p.no_alloc ? policy_peek(p.device) : policy_of(p.device);
  int workgroups = p.workgroups;
  const uint32_t all = pol.xcd_present_mask;
  const uint32_t busy_mask = p.h2d ? pol.h2d_busy_mask : pol.d2h_busy_mask;
  const uint32_t home_mask = p.h2d ? pol.h2d_home_mask : pol.d2h_home_mask;
  const int busy_workgroups =
      std::max(1, p.workgroups * (p.h2d ? pol.h2d_busy_pct : pol.d2h_busy_pct) / 100);
  a->xcd_present = all;
  a->safety_net_wait_us = pol.safety_net_wait_us;
  a->packed_grid_pct = pol.packed_grid_pct;
  a->xcd_mask = 0;
  a->claims_per_wg = pol.all_claims_per_wg;
  a->lane_runs = !p.h2d && pol.d2h_lane_runs != 0;
  if (pol.arbiter == 3) {
    // tests: a mask that names no XCD of the device, every workgroup but the
    // safety net leaves
    a->xcd_mask = (all + 1u) & ~all ? ((all + 1u) & ~all) : 0x8000u;
    a->claims_per_wg = 1;
  } else if (pol.arbiter == 2 ||
             (pol.arbiter == 1 && busy_mask != all && !p.recorded &&
              link_direction_busy(p.device, !p.h2d, stream))) {
    a->xcd_mask = busy_mask;
    workgroups = busy_workgroups;
    a->claims_per_wg = pol.busy_claims_per_wg;
    a->lane_runs = !p.h2d && pol.d2h_lane_runs == 2; // next to traffic the other way: see copy_slice
  } else if (pol.arbiter == 1 && home_mask != all && pol.home_min_kb >= 0 &&
             bytes >= (int64_t)pol.home_min_kb * 1024) {
    a->xcd_mask = home_mask;
    a->claims_per_wg = pol.home_claims_per_wg;
  }
  return workgroups;
}
} // namespace

int kernel_plan_launch(const KernelPlan &p, int layer_offset, int num_layers,
                       hipStream_t stream) {
  if (!p.host_visible)
    return fail(FKV_ERR_INVALID_ARG, "kernel transfer: the host pool is not device-visible "
                "(allocate it pinned or register it)");
  if (layer_offset < 0 || num_layers < 0 || layer_offset + num_layers > p.num_layers)
    return fail(FKV_ERR_RUNTIME, "kernel plan: layers [%d, %d) outside the plan's %d", layer_offset,
                layer_offset + num_layers, p.num_layers);
  // Layers go out in groups whose (layer, kv) base tables fit the kernel's LDS.
  const int layers_per_launch = kCopyMaxLK / p.kv_dim;
  if (layers_per_launch < 1)
    return fail(FKV_ERR_INVALID_ARG, "kv_dim %d too large", p.kv_dim);
  for (int l0 = layer_offset; l0 < layer_offset + num_layers; l0 += layers_per_launch) {
    const int nl = std::min(layers_per_launch, layer_offset + num_layers - l0);
    CopyKernelArgs a = plan_job(p, l0, nl);
    const int workgroups =
        shape_for_now(p, (int64_t)p.num_blocks * a.lk * p.chunk_size, stream, &a);
    FKV_TRY(launch_copy_kernel(a, workgroups, p.threads, stream));
  }
  if (!p.no_alloc) // the bookkeeping creates events on first use
    link_direction_mark(p.device, p.h2d, stream,
                        (int64_t)p.num_blocks * num_layers * p.kv_dim * p.chunk_size);
  return FKV_OK;
}

int kernel_plans_launch(const KernelPlan *const *plans, const int *layer_offsets,
                        const int *num_layers, int count, hipStream_t stream) {
  // One launch for all of them when they can share one: same direction, device,
  // vector width and launch shape, each range within one LDS table.
  const bool fuse = policy_of(plans[0]->device).fuse_launches != 0;
  bool together = fuse && count >= 2 && count <= kCopyMaxJobs;
  for (int i = 0; i < count; ++i)
    together = together && plans[i]->host_visible; // the single launches refuse the others
  for (int i = 0; i < count && together; ++i) {
    const KernelPlan &p = *plans[i], &q = *plans[0];
    together = p.h2d == q.h2d && p.device == q.device && p.vec == q.vec &&
               p.threads == q.threads && p.workgroups == q.workgroups &&
               layer_offsets[i] >= 0 && num_layers[i] > 0 &&
               layer_offsets[i] + num_layers[i] <= p.num_layers &&
               num_layers[i] * p.kv_dim <= kCopyMaxLK;
  }
  if (!together) {
    for (int i = 0; i < count; ++i)
      FKV_TRY(kernel_plan_launch(*plans[i], layer_offsets[i], num_layers[i], stream));
    return FKV_OK;
  }
  CopyKernelArgs jobs[kCopyMaxJobs];
  int64_t bytes = 0;
  for (int i = 0; i < count; ++i) {
    jobs[i] = plan_job(*plans[i], layer_offsets[i], num_layers[i]);
    bytes += (int64_t)plans[i]->num_blocks * jobs[i].lk * plans[i]->chunk_size;
  }
  const int workgroups = shape_for_now(*plans[0], bytes, stream, &jobs[0]);
  FKV_TRY(launch_copy_jobs(jobs, count, workgroups, plans[0]->threads, stream));
  link_direction_mark(plans[0]->device, plans[0]->h2d, stream, bytes);
  return FKV_OK;
}

void kernel_plan_release(KernelPlan *p, hipStream_t stream) {
  if (p->slot)
    plan_release(p->slot, stream, false);
  p->slot = nullptr;
}

int run_kernel_path(const fkv_transfer_desc &d, hipStream_t stream) {
  set_last_path(FKV_PATH_KERNEL);
  KernelPlan plan;
  FKV_TRY(kernel_plan_build(d, stream, &plan));
  KernelPlanHold hold{&plan, stream};
  return kernel_plan_launch(plan, 0, d.num_layers, stream);
}

int validate(const fkv_transfer_desc &d) {
  if (d.backend != FKV_BACKEND_VLLM && d.backend != FKV_BACKEND_TRTLLM &&
      d.backend != FKV_BACKEND_SGLANG)
    return fail(FKV_ERR_RUNTIME, "Unsupported gpu_block_type: %d", d.backend);
  if (d.num_blocks < 0 || d.num_layers < 0 || d.start_layer_id < 0 || d.kv_dim < 1)
    return fail(FKV_ERR_INVALID_ARG,
                "bad transfer extents: num_blocks=%d start_layer=%d num_layers=%d kv_dim=%d",
                d.num_blocks, d.start_layer_id, d.num_layers, d.kv_dim);
  if (d.chunk_size <= 0)
    return fail(FKV_ERR_INVALID_ARG, "chunk_size_in_bytes must be positive, got %lld",
                (long long)d.chunk_size);
  if (d.num_blocks == 0 || d.num_layers == 0)
    return FKV_OK;
  if (!d.gpu_tensor_ptrs || !d.cpu_ptr || !d.gpu_block_ids || !d.cpu_block_ids)
    return fail(FKV_ERR_INVALID_ARG, "null pointer in transfer descriptor");
  // highest tensor-pointer index the addressing mode will touch
  const int64_t last_layer = (int64_t)d.start_layer_id + d.num_layers - 1;
  int64_t need = 1;
  if (d.backend == FKV_BACKEND_VLLM)
    need = last_layer + 1;
  else if (d.backend == FKV_BACKEND_SGLANG)
    need = (int64_t)(d.kv_dim - 1) * d.num_layers_total + last_layer + 1;
  if (d.num_gpu_tensor_ptrs > 0 && need > d.num_gpu_tensor_ptrs)
    return fail(FKV_ERR_INVALID_ARG,
                "layer range [%d, %lld] with kv_dim %d needs %lld GPU tensor pointers, %d given",
                d.start_layer_id, (long long)last_layer, d.kv_dim, (long long)need,
                d.num_gpu_tensor_ptrs);
  for (int i = 0; i < d.num_blocks; ++i)
    if (d.gpu_block_ids[i] < 0 || d.cpu_block_ids[i] < 0)
      return fail(FKV_ERR_INVALID_ARG, "negative block id at position %d", i);
  return FKV_OK;
}

} // namespace fkv

extern "C" {

int fkv_abi_version(void) { return FKV_ABI_VERSION; }
const char *fkv_last_error(void) { return fkv::t_last_error.c_str(); }
int fkv_last_path(void) { return fkv::t_last_path; }

void fkv_ce_config_default(fkv_ce_config *cfg) {
  if (!cfg)
    return;
  std::memset(cfg, 0, sizeof(*cfg));
  cfg->segment_threshold = 8;
  cfg->path_opt_enabled = 1;
  cfg->force_path = -1;
  cfg->enable_memcpy2d = 0;
  cfg->is_blockfirst = 0;
  cfg->num_kv_heads = 1;
  cfg->gather_threads = 4;
  cfg->gather_nt = 1;
}

int fkv_choose_engine(const fkv_transfer_desc *desc, int32_t *use_ce, double *est_kernel_ms,
                      double *est_ce_ms) try {
  fkv::clear_error();
  if (!desc || !use_ce)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_choose_engine: null argument");
  FKV_TRY(fkv::validate(*desc));
  double tk = 0, tc = 0;
  int ce = 0;
  if (desc->num_blocks > 0 && desc->num_layers > 0)
    FKV_TRY(fkv::choose_engine(*desc, &ce, &tk, &tc));
  *use_ce = ce;
  if (est_kernel_ms)
    *est_kernel_ms = tk * 1e3;
  if (est_ce_ms)
    *est_ce_ms = tc * 1e3;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

void fkv_get_stats(fkv_stats *out) {
  if (!out)
    return;
  fkv::Stats &s = fkv::stats();
  out->calls = s.calls.load();
  out->bytes_h2d = s.bytes_h2d.load();
  out->bytes_d2h = s.bytes_d2h.load();
  out->kernel_launches = s.kernel_launches.load();
  out->dma_copies = s.dma_copies.load();
  out->staging_bytes_device = s.staging_bytes_device.load();
  out->staging_bytes_host = s.staging_bytes_host.load();
  out->confined_launches = s.confined_launches.load();
  // a device counter: only worth a device call once a confined launch has been made
  out->safety_net_ranges =
      out->confined_launches ? fkv::safety_net_ranges_of_current_device() : 0;
  out->staged_batches = s.staged_batches.load();
  out->gathered_batches = s.gathered_batches.load();
  out->second_stream_batches = s.second_stream_batches.load();
  int slots = 0, in_use = 0;
  fkv::plan_pool_counts(&slots, &in_use);
  out->plan_slots = (uint64_t)slots;
  out->plan_slots_in_use = (uint64_t)in_use;
  out->plan_slot_waits = s.plan_slot_waits.load();
  out->gather_busy_us = s.gather_busy_ns.load() / 1000;
}
void fkv_reset_stats(void) {
  fkv::Stats &s = fkv::stats();
  s.calls = 0;
  s.bytes_h2d = 0;
  s.bytes_d2h = 0;
  s.kernel_launches = 0;
  s.dma_copies = 0;
  s.staging_bytes_device = 0;
  s.staging_bytes_host = 0;
  s.confined_launches = 0;
  s.staged_batches = 0;
  s.gathered_batches = 0;
  s.second_stream_batches = 0;
  s.plan_slot_waits = 0;
  s.gather_busy_ns = 0;
}

} // extern "C"

namespace {
constexpr int kMaxDevices = 64;
struct PerThreadEvents { // events go when their thread ends
  hipEvent_t done[kMaxDevices][2] = {}; // blocking; [1] with the system-scope fence
  hipEvent_t order[kMaxDevices][2] = {}; // hand-over between a caller's stream and a lane
  ~PerThreadEvents() {
    for (auto *set : {done, order})
      for (int d = 0; d < kMaxDevices; ++d)
        for (hipEvent_t e : set[d])
          if (e && hipEventDestroy(e) != hipSuccess)
            (void)hipGetLastError();
  }
};
PerThreadEvents &my_events() {
  thread_local PerThreadEvents mine;
  return mine;
}

// Records, behind what is queued on `stream` so far, the event a synchronous call
// waits on (nullptr: devices beyond the table, synchronise the stream instead).
// Unlike hipStreamSynchronize, waiting on it does not wait for work that other
// threads queue behind it in the meantime: with 64 requests in flight over two streams
// the median request took 25 ms instead of 82 ms, the slowest percentile 55 ms instead of
// 113 ms.  (The event is made for blocking waits; the runtime keeps the waiting core busy
// all the same, which is why quiet_event_wait exists.)  One event per thread and device,
// reused.
// `host_reads_result`: the transfer wrote host memory that the caller will read
// (GPU->host): the event then keeps its system-scope fence.  A host->GPU transfer
// leaves nothing for the host to read, and its event goes without (see
// kBookkeepingEvent).
int record_completion(hipStream_t stream, bool host_reads_result, hipEvent_t *out) {
  *out = nullptr;
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return FKV_OK;
  hipEvent_t &ev = my_events().done[device][host_reads_result ? 1 : 0];
  if (!ev)
    FKV_HIP_TRY(hipEventCreateWithFlags(
        &ev, hipEventBlockingSync | (host_reads_result ? (unsigned)hipEventDisableTiming
                                                        : fkv::kBookkeepingEvent)));
  FKV_HIP_TRY(hipEventRecord(ev, stream));
  *out = ev;
  return FKV_OK;
}

// ---- lane streams ---------------------------------------------------------
// A process has few hardware queues (4 by default), and streams that share one
// run their kernels in turn.  A caller that issues puts and gets from many
// streams therefore ends up with both directions on every queue: 64 requests on
// 64 streams move 72 GB/s, the same requests on one put stream and one get stream
// 92-94 GB/s.  For such callers kernel transfers run on two streams of the
// library per device, one per direction and on different hardware queues,
// whatever stream the caller names; the caller's stream and the lane are ordered
// by events (the lane waits for what the caller's stream holds so far; an
// asynchronous call makes the caller's stream wait for the transfer).
struct Lane {
  std::mutex mu; // keeps the commands of one transfer together
  hipStream_t stream = nullptr;
};
struct DeviceLanes {
  std::mutex init;
  bool tried = false, ok = false;
  Lane dir[2]; // [0] GPU->host, [1] host->GPU
};
// lane_streams of the launch policy (FKV_LANE_STREAMS): 1 always, 0 never; -1: synchronous calls, once kernel
// transfers of a device have been issued on more than two different streams (a
// stream per request is then likely, and with it both directions on every
// hardware queue).  Asynchronous calls stay on the caller's stream unless asked:
// the hand-over to the lane and back is two more commands per transfer on each
// stream, and a caller that pipelines many small asynchronous transfers on one
// stream pays for them (125 transfers of 25 MB per direction: 76 instead of
// 89 GB/s).
bool lanes_wanted(int device, hipStream_t caller_stream, bool synchronous) {
  const int mode = fkv::policy_of(device).lane_streams;
  if (mode >= 0)
    return mode == 1;
  if (!synchronous)
    return false;
  static std::mutex mu;
  static std::map<int, std::vector<hipStream_t>> seen;
  std::lock_guard<std::mutex> lk(mu);
  std::vector<hipStream_t> &v = seen[device];
  if (v.size() > 2)
    return true;
  if (std::find(v.begin(), v.end(), caller_stream) == v.end())
    v.push_back(caller_stream);
  return v.size() > 2;
}
Lane *lane_of(int device, bool h2d) {
  static std::mutex mu;
  static std::map<int, DeviceLanes *> all; // live until the process ends
  DeviceLanes *dl;
  {
    std::lock_guard<std::mutex> lk(mu);
    DeviceLanes *&p = all[device];
    if (!p)
      p = new DeviceLanes();
    dl = p;
  }
  std::lock_guard<std::mutex> lk(dl->init);
  if (!dl->tried) {
    dl->tried = true;
    hipStream_t a = nullptr, b = nullptr;
    if (hipStreamCreateWithFlags(&a, hipStreamNonBlocking) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    // a partner on another hardware queue; streams that are not kept stay alive, so
    // that the next one lands on a different queue
    for (int attempt = 0; attempt < 8; ++attempt) {
      if (hipStreamCreateWithFlags(&b, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        b = nullptr;
        break;
      }
      int32_t concurrent = 0;
      if (fkv_streams_run_concurrently(device, a, b, &concurrent) == FKV_OK && concurrent)
        break;
    }
    if (b) {
      dl->dir[0].stream = a;
      dl->dir[1].stream = b;
      dl->ok = true;
    }
  }
  return dl->ok ? &dl->dir[h2d ? 1 : 0] : nullptr;
}
// A hand-over event of this thread, recorded on `from`, that `to` waits for.
int order_after(hipStream_t from, hipStream_t to, int device, int which) {
  if (device < 0 || device >= kMaxDevices) {
    FKV_HIP_TRY(hipStreamSynchronize(from));
    return FKV_OK;
  }
  hipEvent_t &ev = my_events().order[device][which];
  if (!ev)
    FKV_HIP_TRY(hipEventCreateWithFlags(&ev, fkv::kBookkeepingEvent));
  FKV_HIP_TRY(hipEventRecord(ev, from));
  FKV_HIP_TRY(hipStreamWaitEvent(to, ev, 0));
  return FKV_OK;
}

// Several descriptors of one direction on the kernel path: a plan each, one launch
// for all of them where they can share one.
int run_kernel_path_multi(const fkv_transfer_desc *descs, int count, hipStream_t stream) {
  fkv::set_last_path(FKV_PATH_KERNEL);
  std::vector<fkv::KernelPlan> plans(count);
  struct GiveBack { // also when a launch throws
    std::vector<fkv::KernelPlan> &plans;
    hipStream_t stream;
    ~GiveBack() {
      for (fkv::KernelPlan &p : plans)
        if (p.slot)
          fkv::kernel_plan_release(&p, stream);
    }
  } give_back{plans, stream};
  int rc = FKV_OK, built = 0;
  for (; built < count && rc == FKV_OK; ++built)
    rc = fkv::kernel_plan_build(descs[built], stream, &plans[built]);
  if (rc != FKV_OK)
    --built; // the one that failed holds nothing
  for (int k = 0; k < built && rc == FKV_OK; k += fkv::kCopyMaxJobs) {
    const int n = std::min(fkv::kCopyMaxJobs, built - k);
    const fkv::KernelPlan *group[fkv::kCopyMaxJobs];
    int first[fkv::kCopyMaxJobs], layers[fkv::kCopyMaxJobs];
    for (int j = 0; j < n; ++j) {
      group[j] = &plans[k + j];
      first[j] = 0;
      layers[j] = descs[k + j].num_layers;
    }
    rc = fkv::kernel_plans_launch(group, first, layers, n, stream);
  }
  return rc;
}

// The body of fkv_transfer_kv_blocks{,_multi}: `count` validated, non-empty
// descriptors of one direction and device; the last one says whether to wait.
int transfer_descs(const fkv_transfer_desc *descs, int count, hipStream_t stream) {
  using namespace fkv;
  const fkv_transfer_desc &d = descs[0];
  const bool sync = descs[count - 1].sync != 0, trace = descs[count - 1].enable_trace != 0;
  // what an earlier, unrelated call of this thread left in the runtime's error slot is not
  // this transfer's (the check at the end reads that slot)
  (void)hipGetLastError();
  DeviceGuard guard(d.device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", d.device);
  uint64_t bytes = 0;
  int64_t blocks = 0;
  for (int i = 0; i < count; ++i) {
    bytes += (uint64_t)descs[i].num_blocks * descs[i].num_layers * descs[i].kv_dim *
             (uint64_t)descs[i].chunk_size;
    blocks += descs[i].num_blocks;
  }
  Range range("fkv %s %d blocks x %d layers (%.2f MB)%s", d.is_host_to_device ? "H2D" : "D2H",
              d.num_blocks, d.num_layers, bytes / (1024.0 * 1024.0),
              count > 1 ? " and more groups" : "");
  // 0 kernel, 1 copy engine, 2 decide per transfer; FKV_TRANSFER_ENGINE overrides the caller.
  static const int forced_engine = [] {
    const char *v = std::getenv("FKV_TRANSFER_ENGINE");
    if (!v || !*v)
      return -1;
    return !std::strcmp(v, "kernel") ? 0 : !std::strcmp(v, "ce") ? 1 : !std::strcmp(v, "auto") ? 2 : -1;
  }();
  // the engine of every descriptor; the kernel path takes them together
  std::vector<int> engines(count);
  bool all_kernel = true;
  for (int i = 0; i < count; ++i) {
    engines[i] = forced_engine >= 0 ? forced_engine : descs[i].use_ce_transfer;
    if (engines[i] == 2) {
      // the model's link figures come from this device, measured once
      int dev = 0;
      if (hipGetDevice(&dev) == hipSuccess)
        (void)policy_of_seeded(dev);
      else
        (void)hipGetLastError();
      FKV_TRY(choose_engine(descs[i], &engines[i], nullptr, nullptr));
    }
    all_kernel = all_kernel && engines[i] == 0;
  }
  auto run_all = [&](hipStream_t on) -> int {
    if (all_kernel)
      return count == 1 ? run_kernel_path(d, on) : run_kernel_path_multi(descs, count, on);
    for (int i = 0; i < count; ++i)
      FKV_TRY(engines[i] ? run_ce_path(descs[i], on) : run_kernel_path(descs[i], on));
    return FKV_OK;
  };
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  Lane *lane = (all_kernel && lanes_wanted(device, stream, sync))
                   ? lane_of(device, d.is_host_to_device != 0)
                   : nullptr;
  hipEvent_t done = nullptr;
  if (lane) {
    std::lock_guard<std::mutex> lk(lane->mu);
    // the lane starts after what the caller's stream holds; an idle stream holds nothing
    if (hipStreamQuery(stream) != hipSuccess) {
      (void)hipGetLastError();
      FKV_TRY(order_after(stream, lane->stream, device, 0));
    }
    FKV_TRY(run_all(lane->stream));
    if (sync)
      FKV_TRY(record_completion(lane->stream, !d.is_host_to_device, &done));
    else
      FKV_TRY(order_after(lane->stream, stream, device, 1));
    stream = lane->stream;
  } else {
    FKV_TRY(run_all(stream));
    if (sync)
      FKV_TRY(record_completion(stream, /*host_reads_result=*/!d.is_host_to_device, &done));
  }
  (d.is_host_to_device ? stats().bytes_h2d : stats().bytes_d2h)
      .fetch_add(bytes, std::memory_order_relaxed);

  if (sync) {
    auto t0 = std::chrono::steady_clock::now();
    // alone on the link the transfer takes bytes / link rate (the policy's figure, re-based on
    // a measurement of the device where one has been made; 3 % taken off)
    const int64_t expected_ns =
        (int64_t)((double)bytes * 1000.0 / std::max(1, policy_peek(device).model_link_mbps) * 0.97);
    if (done)
      FKV_HIP_TRY(quiet_event_wait(done, device, expected_ns));
    else
      FKV_HIP_TRY(quiet_stream_wait(stream, device));
    if (trace) {
      double ms = std::chrono::duration<double, std::milli>(
                      std::chrono::steady_clock::now() - t0)
                      .count();
      // same fields as the reference's trace line, csrc/transfer.cu:304-311
      fprintf(stderr, "[XFER] type=%s blocks=%lld sync_ms=%.3f\n",
              d.is_host_to_device ? "H2D" : "D2H", (long long)blocks, ms);
    }
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(FKV_ERR_RUNTIME, "%s", hipGetErrorString(e));
  return FKV_OK;
}
} // namespace

extern "C" {

int fkv_transfer_kv_blocks(const fkv_transfer_desc *desc, void *stream_v) try {
  using namespace fkv;
  clear_error();
  if (!desc)
    return fail(FKV_ERR_INVALID_ARG, "null descriptor");
  FKV_TRY(validate(*desc));
  stats().calls.fetch_add(1, std::memory_order_relaxed);
  if (desc->num_blocks == 0 || desc->num_layers == 0)
    return FKV_OK;
  return transfer_descs(desc, 1, static_cast<hipStream_t>(stream_v));
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_transfer_kv_blocks_multi(const fkv_transfer_desc *descs, int32_t count, void *stream_v) try {
  using namespace fkv;
  clear_error();
  if (count < 0 || (count > 0 && !descs))
    return fail(FKV_ERR_INVALID_ARG, "fkv_transfer_kv_blocks_multi: bad descriptor array");
  std::vector<fkv_transfer_desc> work;
  for (int i = 0; i < count; ++i) {
    FKV_TRY(validate(descs[i]));
    stats().calls.fetch_add(1, std::memory_order_relaxed);
    if (descs[i].num_blocks == 0 || descs[i].num_layers == 0)
      continue;
    if (!work.empty() && ((descs[i].is_host_to_device != 0) != (work[0].is_host_to_device != 0) ||
                          descs[i].device != work[0].device))
      return fail(FKV_ERR_INVALID_ARG,
                  "fkv_transfer_kv_blocks_multi: descriptors differ in direction or device");
    work.push_back(descs[i]);
  }
  if (work.empty())
    return FKV_OK;
  work.back().sync = descs[count - 1].sync;
  work.back().enable_trace = descs[count - 1].enable_trace;
  return transfer_descs(work.data(), (int)work.size(), static_cast<hipStream_t>(stream_v));
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
