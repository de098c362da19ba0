// A HIP runtime made of host threads, for sanitizer builds of the library's host code.
//
// Test infrastructure only: it stands in for libamdhip64 and for the library's kernels so
// that the host side of the library (plans, rings, launching thread, gates, pollers, the
// copy-engine strategies) runs whole under AddressSanitizer / UndefinedBehaviorSanitizer /
// ThreadSanitizer on a machine without a GPU.
//
//  * "Device memory" and pinned host memory are aligned host allocations kept in a table,
//    so a kernel stand-in dereferences what the library hands it and the sanitizers see
//    every access.  hipPointerGetAttributes / hipHostGetDevicePointer answer from the table;
//    memory that is not in it is pageable.
//  * A stream is a thread with a queue: commands run in order and asynchronously to the
//    host, as on the device.  The null stream is one more such stream.
//  * An event is a pair of counters (recorded, completed) under a mutex: a stream waits for
//    the record that was current when the wait was enqueued, an event that was never
//    recorded reads as complete, as in HIP.  Every hand-over goes through that mutex, so
//    ThreadSanitizer sees exactly the ordering a HIP program may rely on: work that is not
//    ordered by stream order, an event or a synchronize shows up as a race.
//  * The copy kernel stand-ins do what the kernels do (rows of `chunk_bytes` between base
//    tables and block ids) with memcpy, on the stream's thread.  With
//    FKV_KERNELS_FROM_SOURCE there are no stand-ins: the library's kernel sources are
//    compiled for the CPU device model (cpu_device_model.h) and a launch runs the kernel
//    itself, workgroup by workgroup, every work-item on a host thread.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "fkv_internal.h"

// ---- streams ----------------------------------------------------------------------
struct ihipStream_t {
  std::mutex mu;
  std::condition_variable wake, idle;
  std::deque<std::function<void()>> queue;
  bool busy = false, quit = false;
  int hardware_queue = 0; // streams are dealt over four, the null stream sits on the first
  std::thread worker;
  ihipStream_t() : worker([this] { run(); }) {}
  ~ihipStream_t() {
    {
      std::unique_lock<std::mutex> lk(mu);
      idle.wait(lk, [this] { return queue.empty() && !busy; });
      quit = true;
    }
    wake.notify_all();
    worker.join();
  }
  void run() {
    for (;;) {
      std::function<void()> op;
      {
        std::unique_lock<std::mutex> lk(mu);
        wake.wait(lk, [this] { return quit || !queue.empty(); });
        if (queue.empty())
          return;
        op = std::move(queue.front());
        queue.pop_front();
        busy = true;
      }
      op();
      {
        std::lock_guard<std::mutex> lk(mu);
        busy = false;
        if (queue.empty())
          idle.notify_all();
      }
    }
  }
  void push(std::function<void()> op) {
    {
      std::lock_guard<std::mutex> lk(mu);
      queue.push_back(std::move(op));
    }
    wake.notify_one();
  }
  void drain() {
    std::unique_lock<std::mutex> lk(mu);
    idle.wait(lk, [this] { return queue.empty() && !busy; });
  }
  bool is_idle() {
    std::lock_guard<std::mutex> lk(mu);
    return queue.empty() && !busy;
  }
};

struct ihipEvent_t {
  std::mutex mu;
  std::condition_variable cv;
  uint64_t recorded = 0, completed = 0;
  std::chrono::steady_clock::time_point when{};
};

namespace {

thread_local int t_device = 0;
thread_local hipError_t t_last = hipSuccess;
constexpr int kDevices = 2;

hipError_t remember(hipError_t e) {
  if (e != hipSuccess)
    t_last = e;
  return e;
}

// Failures on request: after `after` more successful calls of a category the next `count`
// calls of it fail (fkv_emulated_fail below).  What a real runtime does when memory, streams
// or events run out, or a launch is refused.
enum Category { kDeviceAlloc, kPinnedAlloc, kStreamCreate, kEventCreate, kCopy, kLaunch, kEventRecord,
                kThrow, kCategories };
std::atomic<long> g_fail_after[kCategories];
std::atomic<long> g_fail_count[kCategories];
std::atomic<long> g_failed_calls{0};
std::atomic<long> g_host_waited_copies{0}; // hipMemcpy calls: the host waits for each
bool refused(Category c) {
  if (g_fail_count[c].load(std::memory_order_relaxed) <= 0)
    return false;
  if (g_fail_after[c].fetch_sub(1) > 0)
    return false;
  if (g_fail_count[c].fetch_sub(1) <= 0)
    return false;
  g_failed_calls.fetch_add(1);
  return true;
}

struct Runtime {
  std::mutex mu;
  // every live stream, the null stream first; shared, so that a device-wide wait can outlive
  // the destruction of a stream by another thread
  std::vector<std::shared_ptr<ihipStream_t>> streams;
  struct Block {
    size_t size;
    bool pinned;
    bool registered; // pinned by hipHostRegister: memory of the caller
  };
  std::map<uintptr_t, Block> memory;
  ihipStream_t *null_stream() {
    std::lock_guard<std::mutex> lk(mu);
    if (streams.empty())
      streams.push_back(std::make_shared<ihipStream_t>());
    return streams[0].get();
  }
  const std::pair<const uintptr_t, Block> *find(const void *p) {
    std::lock_guard<std::mutex> lk(mu);
    auto it = memory.upper_bound((uintptr_t)p);
    if (it == memory.begin())
      return nullptr;
    --it;
    return (uintptr_t)p < it->first + it->second.size ? &*it : nullptr;
  }
  void drain_all() {
    std::vector<std::shared_ptr<ihipStream_t>> all;
    {
      std::lock_guard<std::mutex> lk(mu);
      all = streams;
    }
    for (auto &s : all)
      s->drain();
  }
};
Runtime &rt() {
  static Runtime r;
  return r;
}
ihipStream_t *of(hipStream_t s) { return s ? s : rt().null_stream(); }

void *allocate(size_t size, bool pinned) {
  // 2 MiB alignment, as the runtime gives large allocations
  void *p = nullptr;
  if (posix_memalign(&p, (size_t)2 << 20, std::max<size_t>(size, 1)) != 0)
    return nullptr;
  std::lock_guard<std::mutex> lk(rt().mu);
  rt().memory[(uintptr_t)p] = Runtime::Block{std::max<size_t>(size, 64), pinned, false};
  return p;
}

hipError_t release(void *p, bool pinned) {
  if (!p)
    return hipSuccess;
  rt().drain_all(); // hipFree waits for the device
  {
    std::lock_guard<std::mutex> lk(rt().mu);
    auto it = rt().memory.find((uintptr_t)p);
    if (it == rt().memory.end() || it->second.pinned != pinned || it->second.registered)
      return remember(hipErrorInvalidValue);
    rt().memory.erase(it);
  }
  free(p);
  return hipSuccess;
}

void copy_2d(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t height) {
  for (size_t r = 0; r < height; ++r)
    std::memcpy(static_cast<char *>(dst) + r * dpitch, static_cast<const char *>(src) + r * spitch,
                width);
}

} // namespace

extern "C" {

hipError_t hipGetLastError(void) {
  hipError_t e = t_last;
  t_last = hipSuccess;
  return e;
}
const char *hipGetErrorString(hipError_t e) {
  switch (e) {
  case hipSuccess: return "no error";
  case hipErrorNotReady: return "device not ready";
  case hipErrorInvalidValue: return "invalid argument";
  case hipErrorOutOfMemory: return "out of memory";
  case hipErrorNotSupported: return "operation not supported";
  case hipErrorLaunchFailure: return "launch failure";
  case hipErrorInvalidHandle: return "invalid handle";
  default: return "emulated runtime error";
  }
}
hipError_t hipGetDevice(int *d) {
  *d = t_device;
  return hipSuccess;
}
hipError_t hipSetDevice(int d) {
  if (d < 0 || d >= kDevices)
    return remember(hipErrorInvalidDevice);
  t_device = d;
  return hipSuccess;
}
hipError_t hipGetDeviceCount(int *n) {
  *n = kDevices;
  return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) {
  rt().drain_all();
  return hipSuccess;
}
hipError_t hipDeviceGetPCIBusId(char *id, int len, int device) {
  snprintf(id, (size_t)len, "0000:%02x:00.0", device);
  return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned int) {
  if (refused(kStreamCreate))
    return remember(hipErrorOutOfMemory);
  auto made = std::make_shared<ihipStream_t>();
  *s = made.get();
  static std::atomic<int> dealt{0};
  made->hardware_queue = ++dealt % 4;
  std::lock_guard<std::mutex> lk(rt().mu);
  if (rt().streams.empty())
    rt().streams.push_back(std::make_shared<ihipStream_t>());
  rt().streams.push_back(std::move(made));
  return hipSuccess;
}
hipError_t hipStreamCreate(hipStream_t *s) { return hipStreamCreateWithFlags(s, 0); }
hipError_t hipStreamDestroy(hipStream_t s) {
  if (!s)
    return remember(hipErrorInvalidHandle);
  std::shared_ptr<ihipStream_t> mine;
  {
    std::lock_guard<std::mutex> lk(rt().mu);
    auto &v = rt().streams;
    for (size_t i = 1; i < v.size(); ++i)
      if (v[i].get() == s) {
        mine = std::move(v[i]);
        v.erase(v.begin() + (long)i);
        break;
      }
  }
  if (!mine)
    return remember(hipErrorInvalidHandle);
  mine->drain(); // finishes what is queued, as the runtime does; the thread ends with the last owner
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t s) {
  of(s)->drain();
  return hipSuccess;
}
hipError_t hipStreamQuery(hipStream_t s) { return of(s)->is_idle() ? hipSuccess : hipErrorNotReady; }

hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned int) {
  if (refused(kEventCreate))
    return remember(hipErrorOutOfMemory);
  *e = new ihipEvent_t();
  return hipSuccess;
}
hipError_t hipEventCreate(hipEvent_t *e) { return hipEventCreateWithFlags(e, 0); }
hipError_t hipEventDestroy(hipEvent_t e) {
  if (!e)
    return remember(hipErrorInvalidHandle);
  {
    // whoever completes a record of this event does so under its mutex
    std::unique_lock<std::mutex> lk(e->mu);
    e->cv.wait(lk, [e] { return e->completed >= e->recorded; });
  }
  delete e;
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) {
  if (!e)
    return remember(hipErrorInvalidHandle);
  if (refused(kEventRecord))
    return remember(hipErrorLaunchFailure);
  uint64_t gen;
  {
    std::lock_guard<std::mutex> lk(e->mu);
    gen = ++e->recorded;
  }
  of(s)->push([e, gen] {
    std::lock_guard<std::mutex> lk(e->mu);
    e->completed = std::max(e->completed, gen);
    e->when = std::chrono::steady_clock::now();
    e->cv.notify_all();
  });
  return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t e) {
  if (!e)
    return remember(hipErrorInvalidHandle);
  std::lock_guard<std::mutex> lk(e->mu);
  return e->completed >= e->recorded ? hipSuccess : hipErrorNotReady;
}
hipError_t hipEventSynchronize(hipEvent_t e) {
  if (!e)
    return remember(hipErrorInvalidHandle);
  std::unique_lock<std::mutex> lk(e->mu);
  const uint64_t gen = e->recorded;
  e->cv.wait(lk, [e, gen] { return e->completed >= gen; });
  return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t e, unsigned int) {
  if (!e)
    return remember(hipErrorInvalidHandle);
  uint64_t gen;
  {
    std::lock_guard<std::mutex> lk(e->mu);
    gen = e->recorded;
  }
  of(s)->push([e, gen] {
    std::unique_lock<std::mutex> lk(e->mu);
    e->cv.wait(lk, [e, gen] { return e->completed >= gen; });
  });
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b) {
  if (!a || !b)
    return remember(hipErrorInvalidHandle);
  std::chrono::steady_clock::time_point ta, tb;
  {
    std::lock_guard<std::mutex> lk(a->mu);
    if (a->recorded == 0)
      return remember(hipErrorInvalidHandle);
    if (a->completed < a->recorded)
      return remember(hipErrorNotReady);
    ta = a->when;
  }
  {
    std::lock_guard<std::mutex> lk(b->mu);
    if (b->recorded == 0)
      return remember(hipErrorInvalidHandle);
    if (b->completed < b->recorded)
      return remember(hipErrorNotReady);
    tb = b->when;
  }
  *ms = std::chrono::duration<float, std::milli>(tb - ta).count();
  return hipSuccess;
}

hipError_t hipMalloc(void **p, size_t size) {
  *p = refused(kDeviceAlloc) ? nullptr : allocate(size, false);
  return *p ? hipSuccess : remember(hipErrorOutOfMemory);
}
hipError_t hipFree(void *p) { return release(p, false); }
hipError_t hipHostMalloc(void **p, size_t size, unsigned int) {
  *p = refused(kPinnedAlloc) ? nullptr : allocate(size, true);
  return *p ? hipSuccess : remember(hipErrorOutOfMemory);
}
hipError_t hipHostFree(void *p) { return release(p, true); }
hipError_t hipHostRegister(void *p, size_t size, unsigned int) {
  if (!p || size == 0)
    return remember(hipErrorInvalidValue);
  std::lock_guard<std::mutex> lk(rt().mu);
  rt().memory[(uintptr_t)p] = Runtime::Block{size, true, true};
  return hipSuccess;
}
hipError_t hipHostUnregister(void *p) {
  rt().drain_all();
  std::lock_guard<std::mutex> lk(rt().mu);
  auto it = rt().memory.find((uintptr_t)p);
  if (it == rt().memory.end() || !it->second.registered)
    return remember(hipErrorHostMemoryNotRegistered);
  rt().memory.erase(it);
  return hipSuccess;
}
hipError_t hipHostGetDevicePointer(void **dev, void *host, unsigned int) {
  const auto *b = rt().find(host);
  if (!b || !b->second.pinned)
    return remember(hipErrorInvalidValue);
  *dev = host;
  return hipSuccess;
}
hipError_t hipPointerGetAttributes(hipPointerAttribute_t *at, const void *p) {
  const auto *b = rt().find(p);
  if (!b)
    return remember(hipErrorInvalidValue);
  std::memset(at, 0, sizeof(*at));
  at->type = b->second.pinned ? hipMemoryTypeHost : hipMemoryTypeDevice;
  at->device = 0;
  at->devicePointer = const_cast<void *>(p);
  at->hostPointer = b->second.pinned ? const_cast<void *>(p) : nullptr;
  return hipSuccess;
}
hipError_t hipMemGetAddressRange(hipDeviceptr_t *base, size_t *size, hipDeviceptr_t p) {
  const auto *b = rt().find(p);
  if (!b)
    return remember(hipErrorInvalidValue);
  if (base)
    *base = (hipDeviceptr_t)b->first;
  if (size)
    *size = b->second.size;
  return hipSuccess;
}

hipError_t hipMemcpyAsync(void *dst, const void *src, size_t n, hipMemcpyKind, hipStream_t s) {
  if (refused(kCopy))
    return remember(hipErrorLaunchFailure);
  of(s)->push([dst, src, n] { std::memcpy(dst, src, n); });
  return hipSuccess;
}
hipError_t hipMemcpy(void *dst, const void *src, size_t n, hipMemcpyKind) {
  g_host_waited_copies.fetch_add(1);
  rt().null_stream()->drain();
  std::memcpy(dst, src, n);
  return hipSuccess;
}
hipError_t hipMemcpy2DAsync(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width,
                            size_t height, hipMemcpyKind, hipStream_t s) {
  if (width > dpitch || width > spitch)
    return remember(hipErrorInvalidPitchValue);
  if (refused(kCopy))
    return remember(hipErrorLaunchFailure);
  of(s)->push([=] { copy_2d(dst, dpitch, src, spitch, width, height); });
  return hipSuccess;
}
hipError_t hipMemset(void *dst, int value, size_t n) {
  rt().null_stream()->drain();
  std::memset(dst, value, n);
  return hipSuccess;
}
hipError_t hipMemsetAsync(void *dst, int value, size_t n, hipStream_t s) {
  of(s)->push([dst, value, n] { std::memset(dst, value, n); });
  return hipSuccess;
}

hipError_t hipIpcGetMemHandle(hipIpcMemHandle_t *, void *) { return remember(hipErrorNotSupported); }
hipError_t hipIpcOpenMemHandle(void **, hipIpcMemHandle_t, unsigned int) {
  return remember(hipErrorNotSupported);
}
hipError_t hipIpcCloseMemHandle(void *) { return remember(hipErrorNotSupported); }

} // extern "C"

#ifdef FKV_KERNELS_FROM_SOURCE
// ---- the library's kernels, from their own sources (cpu_device_model.h) ---------------
#include "cpu_device_model.h"
namespace cpu_device_model {
thread_local Index thread_index, block_index;
thread_local Extent block_extent, grid_extent;

namespace {
// The work-items of the workgroup that is running: a crew of host threads that lives as
// long as the process and grows to the largest workgroup seen.
struct Crew {
  std::mutex mu;
  // members wait for work in sets of 64, so that a small workgroup does not wake the members
  // a large one once needed
  static constexpr unsigned kSet = 64, kSets = 1024 / kSet;
  std::condition_variable start[kSets], done, barrier_cv;
  uint64_t workgroups_run = 0;
  std::vector<std::thread> members;
  uint64_t round = 0;        // a new workgroup
  unsigned size = 0;         // work-items of that workgroup
  unsigned finished = 0;
  // the barrier: work-items that have left the kernel no longer take part
  unsigned waiting = 0, left = 0;
  uint64_t barrier_round = 0;
  const std::function<void()> *work_item = nullptr;
  Index block;
  Extent block_extent, grid_extent;
  bool quit = false;
  std::vector<unsigned char> lds;
  unsigned xcc = 0;

  ~Crew() {
    {
      std::lock_guard<std::mutex> lk(mu);
      quit = true;
    }
    for (auto &cv : start)
      cv.notify_all();
    for (auto &t : members)
      t.join();
  }
  void member(unsigned id) {
    uint64_t seen = 0;
    for (;;) {
      {
        std::unique_lock<std::mutex> lk(mu);
        start[id / kSet].wait(lk, [&] { return quit || (round != seen && id < size); });
        if (quit)
          return;
        seen = round;
        thread_index = Index{id % block_extent.x, id / block_extent.x % block_extent.y,
                             id / (block_extent.x * block_extent.y)};
        block_index = block;
        cpu_device_model::block_extent = block_extent;
        cpu_device_model::grid_extent = grid_extent;
      }
      (*work_item)();
      {
        std::lock_guard<std::mutex> lk(mu);
        ++left; // a barrier the others wait at may be complete now
        if (waiting > 0 && waiting + left == size) {
          waiting = 0;
          ++barrier_round;
          barrier_cv.notify_all();
        }
        if (++finished == size)
          done.notify_all();
      }
    }
  }
  void run_workgroup(const std::function<void()> &item, Index at, Extent block_ext, Extent grid_ext) {
    std::unique_lock<std::mutex> lk(mu);
    const unsigned n = block_ext.x * block_ext.y * block_ext.z;
    while (members.size() < n) {
      const unsigned id = (unsigned)members.size();
      members.emplace_back([this, id] { member(id); });
    }
    work_item = &item;
    block = at;
    block_extent = block_ext;
    grid_extent = grid_ext;
    size = n;
    finished = waiting = left = 0;
    ++round;
    ++workgroups_run;
    for (unsigned set = 0; set * kSet < n; ++set)
      start[set].notify_all();
    done.wait(lk, [&] { return finished == size; });
    size = 0;
  }
  void barrier() {
    std::unique_lock<std::mutex> lk(mu);
    if (++waiting + left == size) {
      waiting = 0;
      ++barrier_round;
      barrier_cv.notify_all();
      return;
    }
    const uint64_t mine = barrier_round;
    barrier_cv.wait(lk, [&] { return barrier_round != mine; });
  }
};
Crew &crew() {
  static Crew c;
  return c;
}
std::mutex g_device; // one launch at a time owns the crew and the kernels' __shared__ variables
std::atomic<unsigned> g_launch_number{0};
} // namespace

void sync_threads() { crew().barrier(); }
void *dynamic_lds() { return crew().lds.data(); }
unsigned xcc_id() { return crew().xcc; }
void nap() { std::this_thread::yield(); }

void launch(hipStream_t stream, dim3 grid, dim3 block, size_t lds_bytes, std::function<void()> work_item) {
  const uint64_t threads = (uint64_t)block.x * block.y * block.z;
  if (threads == 0 || threads > 1024 || grid.x == 0 || grid.y == 0 || grid.z == 0 ||
      lds_bytes > 160 * 1024) {
    remember(hipErrorInvalidConfiguration);
    return;
  }
  if (refused(kLaunch)) {
    remember(hipErrorLaunchFailure);
    return;
  }
  if (refused(kThrow)) // as if the library had run out of host memory at this point
    throw std::bad_alloc();
  const unsigned number = g_launch_number.fetch_add(1);
  of(stream)->push([=] {
    std::lock_guard<std::mutex> device(g_device);
    Crew &c = crew();
    // exactly as large as asked for: an access beyond it is one the device would not forgive either
    c.lds.assign(lds_bytes, 0xA5);
    c.lds.shrink_to_fit();
    const Extent block_ext{block.x, block.y, block.z}, grid_ext{grid.x, grid.y, grid.z};
    for (unsigned z = 0; z < grid.z; ++z)
      for (unsigned y = 0; y < grid.y; ++y)
        for (unsigned x = 0; x < grid.x; ++x) {
          c.xcc = (x + number * 3) % 8;
          c.run_workgroup(work_item, Index{x, y, z}, block_ext, grid_ext);
        }
  });
}
} // namespace cpu_device_model

// Workgroups of the library's kernels that have run from their sources in this process.
extern "C" unsigned long long fkv_emulated_workgroups_run() {
  auto &c = cpu_device_model::crew();
  std::lock_guard<std::mutex> lk(c.mu);
  return c.workgroups_run;
}

extern "C" {
// A __device__ variable of a kernel source is a variable of this process.
hipError_t hipGetSymbolAddress(void **out, const void *symbol) {
  if (!out || !symbol)
    return remember(hipErrorInvalidSymbol);
  *out = const_cast<void *>(symbol);
  return hipSuccess;
}
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus *status) { // no graphs here
  *status = hipStreamCaptureStatusNone;
  return hipSuccess;
}
hipError_t hipMemcpyFromSymbol(void *dst, const void *symbol, size_t bytes, size_t offset,
                               hipMemcpyKind) {
  rt().drain_all();
  std::memcpy(dst, static_cast<const unsigned char *>(symbol) + offset, bytes);
  return hipSuccess;
}
}
#else
// ---- the library's kernels, on the stream's thread ------------------------------------
namespace fkv {

namespace {
// What fkv_copy_chunks_kernel does: row (i, p) of `chunk_bytes` from
// base_src[i] + ids_src[p] * stride_src to base_dst[i] + ids_dst[p] * stride_dst; a null id
// list stands for 0, 1, 2, ...
void copy_rows(const CopyKernelArgs &a) {
  for (int i = 0; i < a.lk; ++i)
    for (int p = 0; p < a.num_blocks; ++p) {
      const int64_t s = a.ids_src ? a.ids_src[p] : p, d = a.ids_dst ? a.ids_dst[p] : p;
      std::memcpy(reinterpret_cast<void *>((uintptr_t)a.base_dst[i] + (uintptr_t)(d * a.stride_dst)),
                  reinterpret_cast<const void *>((uintptr_t)a.base_src[i] + (uintptr_t)(s * a.stride_src)),
                  (size_t)a.chunk_bytes);
    }
}
std::atomic<uint64_t> g_launches{0};
} // namespace

int launch_copy_kernel(CopyKernelArgs a, int num_workgroups, int threads_per_workgroup,
                       hipStream_t stream) {
  if (a.num_blocks < 0 || a.lk < 0 || a.lk > kCopyMaxLK || a.chunk_bytes < 0 || num_workgroups < 1 ||
      threads_per_workgroup < 1)
    return fail(FKV_ERR_RUNTIME, "emulated copy kernel: bad launch");
  if (refused(kLaunch))
    return fail(FKV_ERR_RUNTIME, "emulated copy kernel: launch refused");
  if (refused(kThrow)) // as if the library had run out of host memory at this point
    throw std::bad_alloc();
  g_launches.fetch_add(1);
  stats().kernel_launches.fetch_add(1, std::memory_order_relaxed);
  of(stream)->push([a] { copy_rows(a); });
  return FKV_OK;
}

int launch_copy_jobs(const CopyKernelArgs *jobs, int njobs, int num_workgroups,
                     int threads_per_workgroup, hipStream_t stream) {
  if (njobs < 1 || njobs > kCopyMaxJobs)
    return fail(FKV_ERR_RUNTIME, "copy kernel: %d jobs in one launch (1..%d)", njobs, kCopyMaxJobs);
  if (refused(kLaunch))
    return fail(FKV_ERR_RUNTIME, "emulated copy kernel: launch refused");
  std::vector<CopyKernelArgs> all(jobs, jobs + njobs);
  stats().kernel_launches.fetch_add(1, std::memory_order_relaxed);
  of(stream)->push([all] {
    for (const CopyKernelArgs &a : all)
      copy_rows(a);
  });
  return FKV_OK;
}

uint64_t safety_net_ranges_of_current_device() { return 0; }

int launch_plan_upload(void *device_dst, const void *pinned_src, size_t bytes, hipStream_t stream) {
  if (refused(kLaunch))
    return fail(FKV_ERR_RUNTIME, "emulated plan upload: launch refused");
  of(stream)->push([=] { std::memcpy(device_dst, pinned_src, bytes); });
  return FKV_OK;
}

int probe_xcds(uint32_t *present_mask) {
  *present_mask = 0xffu;
  return FKV_OK;
}

int common_vector_width(const uint64_t *vals, int n) {
  uint64_t acc = 0;
  for (int i = 0; i < n; ++i)
    acc |= vals[i];
  for (int w = 16; w > 1; w >>= 1)
    if (acc % (uint64_t)w == 0)
      return w;
  return 1;
}

} // namespace fkv

#endif // FKV_KERNELS_FROM_SOURCE

#ifndef FKV_KERNELS_FROM_SOURCE
extern "C" unsigned long long fkv_emulated_workgroups_run() { return 0; }
#endif

// Copies the host has waited for since the process started (hipMemcpy): a library that
// makes one per request under load holds every thread up for as long as the device is busy.
extern "C" long fkv_emulated_host_waited_copies() { return g_host_waited_copies.load(); }

// Test hook: the next `count` calls of `category` (0 device allocation, 1 pinned allocation,
// 2 stream creation, 3 event creation, 4 copy, 5 kernel launch, 6 event record; 7: a kernel
// launch throws std::bad_alloc, as an allocation of the library's own might) fail once `after`
// more of them have succeeded; count 0 switches it off.  Returns the calls refused so far.
extern "C" long fkv_emulated_fail(int category, long after, long count) {
  if (category >= 0 && category < kCategories) {
    g_fail_after[category].store(after);
    g_fail_count[category].store(count);
  }
  return g_failed_calls.load();
}

// Entry points of the library that live beside its kernels: not part of what runs here.
extern "C" {
int fkv_measure_hbm_rate(int32_t, size_t, int32_t, int32_t, double *, double *) {
  return fkv::fail(FKV_ERR_UNSUPPORTED, "emulated runtime: no HBM to measure");
}
int fkv_streams_run_concurrently(int32_t, void *a, void *b, int32_t *concurrent) {
  if (!concurrent)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_streams_run_concurrently: null result pointer");
  *concurrent = of(static_cast<hipStream_t>(a))->hardware_queue !=
                of(static_cast<hipStream_t>(b))->hardware_queue;
  return FKV_OK;
}
int fkv_streams_hand_over_us(int32_t, void *, void *, double *round_trip_us) {
  if (!round_trip_us)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_streams_hand_over_us: null result pointer");
  *round_trip_us = 25.0; // every pair of the emulated device hands over alike
  return FKV_OK;
}
#ifndef FKV_KERNELS_FROM_SOURCE
int fkv_transfer_kv_blocks_noalloc(const fkv_transfer_desc *, void *) {
  return fkv::fail(FKV_ERR_UNSUPPORTED, "emulated runtime: the entry point lives beside the kernels");
}
int fkv_build_gpu_chunk_ptrs(const fkv_chunk_ptrs_desc *, void *) {
  return fkv::fail(FKV_ERR_UNSUPPORTED, "emulated runtime: the entry point lives beside the kernels");
}
int fkv_staging_transfer(const fkv_staging_transfer_desc *, void *) {
  return fkv::fail(FKV_ERR_UNSUPPORTED, "emulated runtime: the entry point lives beside the kernels");
}
#endif
}
