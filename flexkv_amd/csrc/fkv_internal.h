// Internal declarations shared by the translation units of libfkv_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "fkv_transfer.h"

namespace fkv {

// ---- errors -------------------------------------------------------------
// Records the message for fkv_last_error() on this thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Streams of the library's groups (layerwise restore, thread group): taken from a pool per
// device and kind and given back, idle, when the group ends.  A process that makes and ends
// groups by the hundred (a test session, an engine that re-creates its connectors) creates a
// handful of streams instead of thousands; pooled streams are never destroyed, like plan
// memory (tearing runtime objects down from a static destructor is unsafe).  The device must
// be current.
hipError_t pooled_stream_acquire(int device, bool non_blocking, hipStream_t *out);
void pooled_stream_release(int device, bool non_blocking, hipStream_t stream);
// Waits of the host for device work.  The runtime's own (hipEventSynchronize,
// hipStreamSynchronize, also on events made for blocking waits) keep a core busy for as long
// as they last; these poll instead when quiet_wait_us of the device's launch policy says so
// and two threads of the process are already waiting the runtime's way:
// a spin of 30 us for work that is nearly done, then sleeps that double from 20 us up to
// that limit; with `expected_ns` (how long the work takes when nothing else holds it up, 0 =
// unknown) the thread sleeps towards that moment first, a millisecond at a time at most, and
// spins for the 80 us either side of it.  `event` must have been recorded.  The stream form records an event of the calling
// thread behind what the stream holds and waits for that.
hipError_t quiet_event_wait(hipEvent_t event, int device, int64_t expected_ns = 0);
hipError_t quiet_stream_wait(hipStream_t stream, int device);
// For the catch-all handler of an entry point: turns the exception in flight into a status
// and an error text.  No C++ exception crosses the C ABI.
int caught(const char *where) noexcept;
void clear_error();

#define FKV_HIP_TRY(expr)                                                      \
  do {                                                                         \
    hipError_t fkv_e_ = (expr);                                                \
    if (fkv_e_ != hipSuccess) {                                                \
      (void)hipGetLastError();                                                 \
      return ::fkv::fail(FKV_ERR_RUNTIME, "%s: %s", #expr,                     \
                         hipGetErrorString(fkv_e_));                           \
    }                                                                          \
  } while (0)

#define FKV_TRY(expr)                                                          \
  do {                                                                         \
    int fkv_rc_ = (expr);                                                      \
    if (fkv_rc_ != FKV_OK)                                                     \
      return fkv_rc_;                                                          \
  } while (0)

// ---- profiler ranges ------------------------------------------------------
// Pushes a named range for its lifetime when FKV_ROCTX=1 (see fkv_range_push).
class Range {
public:
  explicit Range(const char *fmt, ...) __attribute__((format(printf, 2, 3)));
  ~Range();
  Range(const Range &) = delete;
  Range &operator=(const Range &) = delete;

private:
  bool pushed_ = false;
};

// ---- events ---------------------------------------------------------------
// Flags for events that only order or time work and never publish bytes the GPU
// wrote to *host* memory.  An event recorded with the default flags carries a
// system-scope fence; behind a host->GPU kernel that fence does not retire while
// another stream keeps posted writes to host memory in flight, and the stream
// stands idle for ~0.77 ms after every such kernel (measured: 12 back-to-back
// 2 ms host->GPU kernels next to a GPU->host kernel, 770 us between them with a
// default event after each, 20 us with these flags or with no event).
constexpr unsigned kBookkeepingEvent = hipEventDisableTiming | hipEventDisableSystemFence;
constexpr unsigned kTimingEventNoFence = hipEventDisableSystemFence;

// ---- counters -----------------------------------------------------------
struct Stats {
  std::atomic<uint64_t> calls{0}, bytes_h2d{0}, bytes_d2h{0}, kernel_launches{0},
      dma_copies{0}, staging_bytes_device{0}, staging_bytes_host{0}, confined_launches{0},
      staged_batches{0}, gathered_batches{0}, gather_busy_ns{0}, second_stream_batches{0},
      plan_slot_waits{0};
};
Stats &stats();

void set_last_path(int path);

// Makes `device` current for the lifetime of the object (no-op for -1) and
// restores the previous device afterwards.
class DeviceGuard {
public:
  explicit DeviceGuard(int device);
  ~DeviceGuard();
  int device() const { return device_; }
  bool ok() const { return ok_; }

private:
  int prev_ = -1;
  int device_ = -1;
  bool switched_ = false;
  bool ok_ = true;
};

// ---- GPU chunk addressing ----------------------------------------------
// Device address of chunk (layer, kv, block) before the in-chunk offset.
// Restates ptr_at<> of the reference (csrc/gtensor_handler.cuh:43-67) in bytes.
inline uint64_t gpu_chunk_addr(int backend, const uint64_t *ptrs,
                               int64_t num_layers_total, int64_t kv_stride,
                               int64_t block_stride, int64_t layer_stride,
                               int64_t layer, int64_t kv, int64_t block) {
  switch (backend) {
  case FKV_BACKEND_VLLM:
    return ptrs[layer] + (uint64_t)(kv * kv_stride) + (uint64_t)(block * block_stride);
  case FKV_BACKEND_TRTLLM:
    return ptrs[0] + (uint64_t)(block * block_stride) +
           (uint64_t)(layer * layer_stride) + (uint64_t)(kv * kv_stride);
  default: // FKV_BACKEND_SGLANG
    return ptrs[kv * num_layers_total + layer] + (uint64_t)(block * block_stride);
  }
}
inline uint64_t gpu_chunk_addr(const fkv_transfer_desc &d, int64_t layer, int64_t kv,
                               int64_t block) {
  return gpu_chunk_addr(d.backend, d.gpu_tensor_ptrs, d.num_layers_total,
                        d.gpu_kv_stride, d.gpu_block_stride, d.gpu_layer_stride, layer,
                        kv, block) +
         (uint64_t)d.gpu_startoff_inside_chunks;
}
// Host address of chunk (layer, kv, block) including the in-chunk offset
// (csrc/transfer.cu:124-130).
inline uint8_t *cpu_chunk_ptr(const fkv_transfer_desc &d, int64_t layer, int64_t kv,
                              int64_t block) {
  return static_cast<uint8_t *>(d.cpu_ptr) + layer * d.cpu_layer_stride +
         kv * d.cpu_kv_stride + block * d.cpu_block_stride +
         d.cpu_startoff_inside_chunks;
}

// ---- the gather/scatter kernel -----------------------------------------
// One launch copies `num_blocks * lk` chunks of `chunk_bytes`:
//   for pos, i:  src = base_src[i] + ids_src[pos]*stride_src
//                dst = base_dst[i] + ids_dst[pos]*stride_dst
// (ids == nullptr means ids[pos] == pos).  All four arrays live in memory the
// device can read.  `lk` = layers-in-call * kv_dim.
struct CopyKernelArgs {
  const uint64_t *base_src;
  const uint64_t *base_dst;
  const int64_t *ids_src;
  const int64_t *ids_dst;
  int64_t stride_src;
  int64_t stride_dst;
  int64_t chunk_bytes;
  int32_t num_blocks;
  int32_t lk;
  int32_t slices_per_chunk;
  int32_t vec;      // 16, 8, 4, 2 or 1: widest access all addresses allow
  int32_t nt_store; // 1: nontemporal stores (destination in HBM), 0: plain (pinned host)
  int32_t unroll;   // vector accesses in flight per lane: kCopyUnroll (also for 0), or
                    // kCopyUnrollDeep where launch_copy_kernel finds the launch fit for it
  int32_t packed;   // set by launch_copy_kernel: chunks shorter than a slice, see the kernel
  int32_t lane_runs; // stores into pinned host memory: a lane moves adjacent vectors (see copy_slice)
  int32_t packed_grid_pct; // workgroups to launch in packed mode, percent of the request (0 = 100)
  uint32_t xcd_mask; // bit k: workgroups that run on XCD k take part; 0 = all
  uint32_t xcd_present;        // host side: the XCDs of the device (0 = eight, ids 0-7)
  int32_t safety_net_wait_us;  // confined launches, see the kernel (0 = 50)
  // Launches whose workgroups claim their work: a 64-bit counter in device memory
  // (high half: `epoch` of the launch that owns the count, low half: ranges handed
  // out of `num_claims`, set by launch_copy_kernel).  The counter need not be clean:
  // the first workgroup that finds another epoch in it starts it at zero.  Without
  // a counter the mask is ignored.
  uint64_t *claim;
  uint32_t num_claims;
  uint32_t epoch; // set by launch_copy_kernel: a number no other launch in flight has
  int32_t claims_per_wg; // ranges per working workgroup: confined launches (0 = 1), and
                         // launches on all XCDs that have counters (0 = fixed shares)
};
constexpr int kCopyBlockThreads = 1024;  // largest workgroup the kernel is built for
constexpr int kCopyUnroll = 8;           // vector accesses in flight per lane
constexpr int kCopyUnrollDeep = 16;      // the same for launches that HBM bounds
constexpr int kCopyMaxLK = 1024;         // base-table entries staged in LDS
constexpr int kCopyIdTile = 1024;        // block positions staged in LDS at a time
int launch_copy_kernel(CopyKernelArgs args, int num_workgroups, int threads_per_workgroup,
                       hipStream_t stream);
// Up to kCopyMaxJobs jobs of one direction and vector width in one launch: the work
// of all of them is shared out among the workgroups by bytes.  Mask, counters and
// ranges per workgroup are taken from jobs[0].
constexpr int kCopyMaxJobs = 4;
struct CopyJobs {
  int32_t njobs;
  uint32_t weight[kCopyMaxJobs]; // length of each job on the line the shares are cut from
  CopyKernelArgs job[kCopyMaxJobs];
};
int launch_copy_jobs(const CopyKernelArgs *jobs, int njobs, int num_workgroups,
                     int threads_per_workgroup, hipStream_t stream);
// Ranges of work that safety-net workgroups (see the kernel) have copied on the
// current device since the process started; reads a device counter.
uint64_t safety_net_ranges_of_current_device();
// Copies `bytes` (rounded up to 16) from a pinned, device-mapped host buffer to
// device memory with a small kernel on `stream`.
int launch_plan_upload(void *device_dst, const void *pinned_src, size_t bytes, hipStream_t stream);
// The XCDs of the current device, by a probe kernel on the null stream (blocking).
int probe_xcds(uint32_t *present_mask);
// The launch policy of `device` (a copy; built on first use, see fkv_policy.cpp).
fkv_launch_policy policy_of(int device);
// The same with the link-dependent figures of the cost model re-based on a measurement
// of the device (once per device, a few tens of milliseconds; see fkv_policy.cpp).
fkv_launch_policy policy_of_seeded(int device);
// The same without the probe: the table of a device that has none yet is the one
// of a device of unknown shape (nothing is confined).
fkv_launch_policy policy_peek(int device);
// `p` with every field brought into its allowed range (what fkv_launch_policy_set
// would store), for callers that bring a table of their own.
fkv_launch_policy policy_sanitized(const fkv_launch_policy &p);
// Widest vector width (bytes) that divides every value in `vals`.
int common_vector_width(const uint64_t *vals, int n);

// ---- plan memory ---------------------------------------------------------
// A plan is the small table (base addresses + block ids) one launch reads.
// Slots are pinned host buffers with a device mirror, recycled once the event
// recorded behind their last user has completed.
struct PlanSlot;
// Returns nullptr (and sets the error) on allocation failure.
PlanSlot *plan_acquire(int device, size_t bytes);
// Slots the pool holds, and how many of them are handed out at the moment (acquired and not
// yet released): after every user has finished, none.
void plan_pool_counts(int *slots, int *handed_out);
uint8_t *plan_host(PlanSlot *s);
// `count` claim counters in device memory that belong to the slot
// (CopyKernelArgs::claim), or nullptr when a slot holds fewer.
uint64_t *plan_counters(PlanSlot *s, int count);
// Publishes the first `bytes` of the slot to the device on `stream` and returns
// the address kernels must use (the device mirror, or the pinned buffer itself
// when `mirror` is false).
int plan_publish(PlanSlot *s, size_t bytes, bool mirror, hipStream_t stream,
                 uint8_t **device_visible);
// `drained`: the stream has been synchronised, the slot is reusable at once.
void plan_release(PlanSlot *s, hipStream_t stream, bool drained);

// ---- paths ----------------------------------------------------------------
// The kernel path in two steps, so that a caller that launches layer by layer
// (the layerwise restore) uploads the id lists and base tables once.
struct KernelPlan {
  PlanSlot *slot = nullptr;
  const uint64_t *gpu_base = nullptr; // device-visible, [num_layers * kv_dim]
  const uint64_t *cpu_base = nullptr;
  const int64_t *gpu_ids = nullptr;   // device-visible, [num_blocks]
  const int64_t *cpu_ids = nullptr;
  int vec = 1;
  bool h2d = false;
  int kv_dim = 1, num_layers = 0, num_blocks = 0;
  int64_t chunk_size = 0, gpu_block_stride = 0, cpu_block_stride = 0;
  int workgroups = 1, threads = 64;
  int device = 0;
  bool no_alloc = false; // built by the entry point that allocates nothing: launches of this
                         // plan create no events and do not probe the device
  bool host_visible = true; // false: the host pool is ordinary pageable memory, the plan has no
                            // host addresses and serves only as the device side of a restore
                            // whose rows host threads gather (kernel_plan_launch refuses it)
  bool recorded = false; // the launches are being recorded into a graph: shaped once for every
                         // replay, without a look at what the link is doing right now
  uint64_t *claims = nullptr; // a claim counter per layer of the plan, device memory
};
void kernel_plan_release(KernelPlan *p, hipStream_t stream);
// Give plan memory back when the scope ends, by whichever way it ends.
struct KernelPlanHold {
  KernelPlan *plan;
  hipStream_t stream;
  ~KernelPlanHold() {
    if (plan && plan->slot)
      kernel_plan_release(plan, stream);
  }
};
struct PlanSlotHold {
  PlanSlot *slot;
  hipStream_t stream;
  ~PlanSlotHold() {
    if (slot)
      plan_release(slot, stream, false);
  }
};
// Link-bound launches of the last while, per device and direction (see fkv_core.cpp).
bool link_direction_busy(int device, bool h2d, hipStream_t launching_stream);
void link_direction_mark(int device, bool h2d, hipStream_t stream, int64_t bytes);
// The same across processes (fkv_linkboard.cpp): post that this process keeps the
// link busy in one direction for about `expected_ns` more, and ask whether another
// process has posted activity that ends less than `window_ns` ago or later.
void link_board_post(int device, bool h2d, int64_t expected_ns);
bool link_board_busy_elsewhere(int device, bool h2d, int64_t window_ns);
// The two halves of kernel_plan_build, for a caller that brings its own plan
// memory: bytes a plan of `d` takes; fill them into host memory `h` (and every
// field of `out` but the addresses); point `out` at the device-visible copy `dv`
// and at `claims` (num_layers counters, or nullptr).
size_t kernel_plan_bytes(const fkv_transfer_desc &d);
int kernel_plan_fill(const fkv_transfer_desc &d, uint8_t *h, bool may_probe_device,
                     KernelPlan *out, bool host_optional = false);
void kernel_plan_point(KernelPlan *out, const uint8_t *dv, uint64_t *claims);
// Builds and uploads (on `stream`) the plan for all layers of `d`.  With `host_optional` a
// host pool the device cannot read is no error: the plan then has host_visible == false.
int kernel_plan_build(const fkv_transfer_desc &d, hipStream_t stream, KernelPlan *out,
                      bool host_optional = false);
// Enqueues the copy of layers [layer_offset, layer_offset + num_layers) of the plan.
int kernel_plan_launch(const KernelPlan &p, int layer_offset, int num_layers,
                       hipStream_t stream);
// The same for layer ranges of several plans of one direction in one launch (the
// members of one original layer of a multi-group restore); falls back to one launch
// per plan where the plans cannot share one.
int kernel_plans_launch(const KernelPlan *const *plans, const int *layer_offsets,
                        const int *num_layers, int count, hipStream_t stream);
// The plan memory is recycled once everything enqueued on `stream` so far has run.
void kernel_plan_release(KernelPlan *p, hipStream_t stream);
int run_kernel_path(const fkv_transfer_desc &d, hipStream_t stream);
int run_ce_path(const fkv_transfer_desc &d, hipStream_t stream);
// Cost-model choice between the two paths for this transfer (no device call).
int choose_engine(const fkv_transfer_desc &d, int *use_ce, double *kernel_s, double *ce_s);
// Device-side compaction between the engine's KV tensors and a packed device
// buffer; see fkv_ce.cpp.
int device_staging_copy(const fkv_transfer_desc &d, int it0, int nit, int p0, int np,
                        uint8_t *staging, bool blockfirst, bool to_staging,
                        hipStream_t stream);

// ---- restore through the copy engines (fkv_staged_restore.cpp) ---------------
// Staging buffers of one (layer group, GPU); they outlive the calls.
struct StagedRing {
  std::vector<uint8_t *> buf;
  size_t cap = 0;
  std::vector<hipEvent_t> copied, freed; // per buffer: copies landed / scatter done
  std::vector<bool> used;
  int next = 0;
  int idle_calls = 0;   // restores of the group in a row that did not use the buffers
  bool touched = false; // used by the restore that is being set up
  void release(); // frees everything; the device must have finished with the buffers
};
// Pinned host buffers of one (layer group, GPU) for restores whose rows host threads
// gather first; they outlive the calls like the staging buffers.
struct GatherRing {
  std::vector<uint8_t *> buf;
  size_t cap = 0;
  std::vector<hipEvent_t> read; // per buffer: the copy engine has read it
  std::vector<bool> used;
  int next = 0;
  int idle_calls = 0;
  bool touched = false;
  void release(); // the device must have finished with the buffers
};
class HostCrew;
// Routes of a layerwise batch other than the kernel path.
enum : int { kRouteKernel = 0, kRouteRuns = 1, kRouteGathered = 2 };
// What one call derives for one (layer group, GPU).
struct StagedPlan {
  struct Seg {
    int64_t first_id; // first host block of the run
    int32_t rows;     // host blocks it spans (holes read along included)
    int32_t row0;     // staging row of the first
  };
  bool usable = false;
  int route = kRouteKernel; // kRouteRuns: a copy command per run of host blocks; kRouteGathered:
                            // host threads gather the rows, one copy command per batch
  bool first_by_kernel = false;  // kRouteGathered: the first batch of the restore goes the kernel way
  std::vector<int64_t> host_ids; // kRouteGathered: the call's host block ids (the launching
                                 // thread may outlive the caller's list)
  std::vector<Seg> segs;
  int32_t total_rows = 0;
  int kind = 0; // chunks of a host block that are adjacent: 0 all of a batch, 1 K and V of a layer, 2 none
  int max_lk = 0, batch_layers = 0, kv_dim = 1, num_blocks = 0;
  int64_t chunk = 0, cpu_kv_stride = 0, cpu_layer_stride = 0, cpu_block_stride = 0;
  const uint8_t *host0 = nullptr;
  PlanSlot *slot = nullptr;
  const uint64_t *base_tables = nullptr; // device-visible, [ring buffers][max_lk]
  const int64_t *stage_rows = nullptr;   // device-visible, [num_blocks]
};
// Decides whether the restore described by `d` (all its layers, in batches of
// `batch_layers`) goes through the copy engines on the current device and, if so,
// sizes the ring and uploads the tables on `scatter_stream`.  FKV_OK with
// out->usable == false: use the kernel path.
// `host_visible`: the device can read the host pool (else only the gathered route is open);
// `kernel_allowed`: the caller lets batches go by kernel (the first batch of a gathered restore).
int staged_plan_build(const fkv_transfer_desc &d, int batch_layers, StagedRing &ring,
                      GatherRing &pinned, hipStream_t scatter_stream, StagedPlan *out,
                      bool host_visible = true, bool kernel_allowed = true,
                      bool several_gpus = false);
// The choice alone (no device): kRouteKernel, kRouteRuns (fills `segs` and `total_rows`)
// or kRouteGathered.
// `free_commands`: up to so many copy commands a batch are taken whatever the batch's size.
int staged_route(const int64_t *cpu_ids, int num_blocks, int64_t row_bytes, int pieces,
                 const fkv_launch_policy &pol, std::vector<StagedPlan::Seg> *segs,
                 int64_t *total_rows, int free_commands = 0);
// Host threads a gathered restore uses under `pol` on this machine (>= 1).
int gather_threads_of(const fkv_launch_policy &pol);
// Layers [l0, l0 + nl) of a kRouteGathered plan: gathers the rows on the calling thread
// and `crew` (blocks for that long, and before that until a pinned buffer is free),
// then enqueues one copy and the scatter.
int gathered_launch(const StagedPlan &sp, StagedRing &ring, GatherRing &pinned, HostCrew &crew,
                    const KernelPlan &kp, int l0, int nl, hipStream_t dma_stream,
                    hipStream_t scatter_stream);
// Layers [l0, l0 + nl) of the plan: copies on `dma_stream`, scatter on `scatter_stream`.
int staged_launch(const StagedPlan &sp, StagedRing &ring, const KernelPlan &kp, int l0, int nl,
                  hipStream_t dma_stream, hipStream_t scatter_stream);
void staged_plan_release(StagedPlan *sp, hipStream_t scatter_stream);

int default_num_cta(bool is_h2d);
int validate(const fkv_transfer_desc &d);

} // namespace fkv
