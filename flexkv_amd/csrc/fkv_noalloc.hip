// fkv_transfer_kv_blocks_noalloc: the kernel path of fkv_transfer_kv_blocks for
// callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc).
//
// The regular entry point keeps the plan of a launch (two tables of base
// addresses, the two block-id lists) and the claim counters of confined launches
// in memory it allocates on demand.  Here both live in a fixed array in device
// memory that is part of the library's code object:
//
//   scratch = [ kNoAllocCounters claim counters | plan of the call in flight ]
//
// Every GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends.  The array's name is a host-side stand-in; the
// device address is looked up once per device with hipGetSymbolAddress and only
// that address is ever handed to the runtime or to a kernel.
//
// Everything the call enqueues is a kernel launch on the caller's stream, so it is
// ordered like any other work of that stream and can be recorded into a graph:
//   * the plan reaches the array inside the arguments of a small fill kernel, 3.5 KiB
//     per launch (arguments are copied when the launch is made, and a graph node keeps
//     its copy: a replay writes the same plan again).  No copy from host memory, no
//     host buffer that has to outlive the call;
//   * block-id lists that the device can read where they are (pinned, registered or
//     device memory) are not copied at all: the copy kernel reads them in place, as
//     the reference's kernel reads its id tensors (csrc/transfer.cu:121-122).  Only
//     id lists in pageable memory travel with the fill kernels;
//   * the claim counters need no clearing: a launch takes a counter over whatever it
//     holds (see Shares::adopt in fkv_kernels.hip).
// The call waits for nothing on the host (unless desc->sync asks for it) and keeps no
// stream handle.  All calls on a GPU share the one array: calls on one stream follow
// each other; calls that are in flight at the same time on different streams of one
// GPU race for it and must be ordered by the caller.
#include "fkv_internal.h"

#include <cstring>
#include <mutex>

namespace {

constexpr size_t kNoAllocCounters = 1024;                     // uint64 each
constexpr size_t kNoAllocPlanBytes = FKV_NOALLOC_MAX_PLAN_BYTES;
constexpr size_t kScratchBytes = kNoAllocCounters * 8 + kNoAllocPlanBytes;
constexpr int kNoAllocMaxDevices = 16;
constexpr int kFillWords = 448; // 64-bit words a fill launch carries: 3.5 KiB of the 4 KiB
                                // a launch has for its arguments

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

struct FillWords {
  uint64_t w[kFillWords];
};

// dst[i] = words.w[i] for i < n: the payload arrives in the kernel arguments.
__global__ void fkv_noalloc_fill_kernel(uint64_t *dst, FillWords words, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    dst[i] = words.w[i];
}

struct PerDevice {
  std::mutex mu;                 // one call at a time prepares a plan for this GPU
  unsigned char *ptr = nullptr;  // device address of this GPU's copy of `scratch`
};
PerDevice g_dev[kNoAllocMaxDevices];
// Where the tables of a plan are put together before they go into launch arguments
// (read only while the call runs; one per GPU: calls on different GPUs do not wait
// for each other).
unsigned char g_host_plan[kNoAllocMaxDevices][kNoAllocPlanBytes];

// Once per device, with that device current.
int setup(int device, PerDevice &pd) {
  if (pd.ptr)
    return FKV_OK;
  void *p = nullptr;
  hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    (void)hipGetLastError();
    return fkv::fail(FKV_ERR_RUNTIME, "no-alloc transfer: hipGetSymbolAddress on device %d: %s",
                     device, hipGetErrorString(e));
  }
  pd.ptr = static_cast<unsigned char *>(p);
  return FKV_OK;
}

// `bytes` (a multiple of 8) from host memory into the device array at `dst`, carried by
// the arguments of as many fill launches as it takes.
int upload_in_arguments(unsigned char *dst, const unsigned char *src, size_t bytes,
                        hipStream_t stream) {
  const size_t words = bytes / 8;
  for (size_t at = 0; at < words; at += kFillWords) {
    const int n = (int)std::min<size_t>(kFillWords, words - at);
    FillWords payload;
    std::memcpy(payload.w, src + at * 8, (size_t)n * 8);
    hipLaunchKernelGGL(fkv_noalloc_fill_kernel, dim3((n + 63) / 64), dim3(64), 0, stream,
                       reinterpret_cast<uint64_t *>(dst) + at, payload, n);
    FKV_HIP_TRY(hipGetLastError());
  }
  return FKV_OK;
}

// The address under which the device reads `n` ids at host pointer `p`, or nullptr
// when `p` is ordinary pageable memory.
const int64_t *device_view_of(const int64_t *p) {
  hipPointerAttribute_t attr;
  std::memset(&attr, 0, sizeof(attr));
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError(); // not known to the runtime: pageable
    return nullptr;
  }
  if (attr.type == hipMemoryTypeHost)
    return static_cast<const int64_t *>(attr.devicePointer);
  if (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged)
    return p;
  return nullptr;
}

} // namespace

extern "C" int fkv_transfer_kv_blocks_noalloc(const fkv_transfer_desc *desc, void *stream_v) try {
  using namespace fkv;
  clear_error();
  if (!desc)
    return fail(FKV_ERR_INVALID_ARG, "null descriptor");
  FKV_TRY(validate(*desc));
  const fkv_transfer_desc &d = *desc;
  if (d.use_ce_transfer != 0)
    return fail(FKV_ERR_UNSUPPORTED,
                "fkv_transfer_kv_blocks_noalloc runs the kernel path only (use_ce_transfer must "
                "be 0): the copy-engine strategies allocate staging buffers");
  stats().calls.fetch_add(1, std::memory_order_relaxed);
  if (d.num_blocks == 0 || d.num_layers == 0)
    return FKV_OK;
  const size_t plan_bytes = kernel_plan_bytes(d);
  if (plan_bytes > kNoAllocPlanBytes)
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_transfer_kv_blocks_noalloc: the plan of %d blocks x %d layers x kv_dim %d "
                "takes %zu bytes, the fixed scratch holds %zu (16 bytes per block + 16 per "
                "(layer, kv) pair): split the call or use fkv_transfer_kv_blocks",
                d.num_blocks, d.num_layers, d.kv_dim, plan_bytes, kNoAllocPlanBytes);
  if ((size_t)d.num_layers > kNoAllocCounters)
    return fail(FKV_ERR_INVALID_ARG,
                "fkv_transfer_kv_blocks_noalloc: %d layers in one call, at most %zu", d.num_layers,
                kNoAllocCounters);
  DeviceGuard guard(d.device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", d.device);
  int device = 0;
  FKV_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kNoAllocMaxDevices)
    return fail(FKV_ERR_UNSUPPORTED, "fkv_transfer_kv_blocks_noalloc: device %d beyond the %d "
                "the fixed host buffers cover", device, kNoAllocMaxDevices);
  hipStream_t stream = static_cast<hipStream_t>(stream_v);
  PerDevice &pd = g_dev[device];
  std::lock_guard<std::mutex> lk(pd.mu);
  FKV_TRY(setup(device, pd));
  unsigned char *host_plan = g_host_plan[device];
  unsigned char *dev_counters = pd.ptr;
  unsigned char *dev_plan = pd.ptr + kNoAllocCounters * 8;
  KernelPlan plan;
  FKV_TRY(kernel_plan_fill(d, host_plan, /*may_probe_device=*/false, &plan));
  set_last_path(FKV_PATH_KERNEL);
  // A launch that is being recorded into a graph is shaped once, for every replay: it
  // does not look at what the link is doing at the moment of the capture.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    capture = hipStreamCaptureStatusNone;
  }
  plan.recorded = capture != hipStreamCaptureStatusNone;
  const size_t tab_bytes = 2 * (size_t)d.num_layers * d.kv_dim * 8;
  const int64_t *gpu_ids = device_view_of(d.gpu_block_ids);
  const int64_t *cpu_ids = device_view_of(d.cpu_block_ids);
  const bool ids_in_place = gpu_ids && cpu_ids;
  FKV_TRY(upload_in_arguments(dev_plan, host_plan, ids_in_place ? tab_bytes : plan_bytes, stream));
  kernel_plan_point(&plan, dev_plan, reinterpret_cast<uint64_t *>(dev_counters));
  if (ids_in_place) {
    plan.gpu_ids = gpu_ids;
    plan.cpu_ids = cpu_ids;
  }
  FKV_TRY(kernel_plan_launch(plan, 0, d.num_layers, stream));
  (d.is_host_to_device ? stats().bytes_h2d : stats().bytes_d2h)
      .fetch_add((uint64_t)d.num_blocks * d.num_layers * d.kv_dim * (uint64_t)d.chunk_size,
                 std::memory_order_relaxed);
  if (d.sync)
    FKV_HIP_TRY(hipStreamSynchronize(stream));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}
