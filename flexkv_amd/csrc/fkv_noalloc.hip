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
// The plan is written into a fixed host buffer and copied up with hipMemcpyAsync
// on the caller's stream, so calls on one stream are ordered like any other work
// of that stream.  All calls on a GPU share the one array: a call waits (on the
// host) until the stream of the previous call on that GPU has drained before it
// reuses the host buffer, but two calls that are in flight on different streams
// of one GPU at the same time race for the device array.  The claim counters
// need no clearing: a launch takes a counter over whatever it holds (see
// Shares::adopt in fkv_kernels.hip).
#include "fkv_internal.h"

#include <cstring>
#include <mutex>

namespace {

constexpr size_t kNoAllocCounters = 1024;                     // uint64 each
constexpr size_t kNoAllocPlanBytes = FKV_NOALLOC_MAX_PLAN_BYTES;
constexpr size_t kScratchBytes = kNoAllocCounters * 8 + kNoAllocPlanBytes;
constexpr int kNoAllocMaxDevices = 16;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

struct PerDevice {
  std::mutex mu;                 // one call at a time prepares a plan for this GPU
  unsigned char *ptr = nullptr;  // device address of this GPU's copy of `scratch`
  hipStream_t last_stream = nullptr;
  bool in_flight = false;        // a call was enqueued on last_stream and not waited for
};
PerDevice g_dev[kNoAllocMaxDevices];
// Where a plan is put together before it is copied up (one per GPU: calls on
// different GPUs do not wait for each other).
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

} // namespace

extern "C" int fkv_transfer_kv_blocks_noalloc(const fkv_transfer_desc *desc, void *stream_v) {
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
  // The host buffer and the device array still belong to the previous call on
  // this GPU until its stream has run the copy and the kernels behind it.
  if (pd.in_flight) {
    if (hipStreamSynchronize(pd.last_stream) != hipSuccess) {
      // the caller has destroyed that stream in the meantime; what it held may still run
      (void)hipGetLastError();
      FKV_HIP_TRY(hipDeviceSynchronize());
    }
    pd.in_flight = false;
  }
  unsigned char *host_plan = g_host_plan[device];
  unsigned char *dev_counters = pd.ptr;
  unsigned char *dev_plan = pd.ptr + kNoAllocCounters * 8;
  KernelPlan plan;
  FKV_TRY(kernel_plan_fill(d, host_plan, /*may_probe_device=*/false, &plan));
  set_last_path(FKV_PATH_KERNEL);
  FKV_HIP_TRY(hipMemcpyAsync(dev_plan, host_plan, plan_bytes, hipMemcpyHostToDevice, stream));
  pd.last_stream = stream;
  pd.in_flight = true;
  kernel_plan_point(&plan, dev_plan, reinterpret_cast<uint64_t *>(dev_counters));
  FKV_TRY(kernel_plan_launch(plan, 0, d.num_layers, stream));
  (d.is_host_to_device ? stats().bytes_h2d : stats().bytes_d2h)
      .fetch_add((uint64_t)d.num_blocks * d.num_layers * d.kv_dim * (uint64_t)d.chunk_size,
                 std::memory_order_relaxed);
  if (d.sync) {
    FKV_HIP_TRY(hipStreamSynchronize(stream));
    pd.in_flight = false;
  }
  return FKV_OK;
}
