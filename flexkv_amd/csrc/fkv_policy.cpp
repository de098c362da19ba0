// The launch policy: every tunable of the kernel path in one table per device.
//
// Defaults are derived from the device.  The XCDs a device exposes are found by a
// probe kernel (each workgroup reports the id of the XCD it runs on), so the masks
// that keep the two directions of the host link apart follow the device instead of
// being literals: with the XCD ids sorted, host->GPU launches own the upper half,
// GPU->host launches the ids [1, n/4] while gets are running and [1, n/2) on an
// idle link (the first XCD is left out: a writer to host memory that includes it
// measured 4 GB/s slower).  Devices with fewer than four XCDs are not split.
// A few fields can be preset from the environment (kEnv below); everything can be
// changed at run time through fkv_launch_policy_set.
#include "fkv_internal.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

namespace fkv {
namespace {

struct EnvField {
  const char *name;
  size_t offset; // of an int32_t / uint32_t field of fkv_launch_policy
};
#define FKV_FIELD(env, field) {env, offsetof(fkv_launch_policy, field)}
// The environment variables that preset a field (read once per device table).
const EnvField kEnv[] = {
    FKV_FIELD("FKV_LINK_ARBITER", arbiter),
    FKV_FIELD("FKV_LINK_ARBITER_WINDOW_MS", busy_window_ms),
    FKV_FIELD("FKV_HOME_MIN_KB", home_min_kb),
    FKV_FIELD("FKV_CLAIMS_PER_WORKGROUP", all_claims_per_wg),
    FKV_FIELD("FKV_LANE_STREAMS", lane_streams),
    FKV_FIELD("FKV_PLAN_MIRROR", plan_mirror),
    FKV_FIELD("FKV_STAGED_RESTORE", staged_restore),
    FKV_FIELD("FKV_CE_STAGING_MB", ce_staging_mb),
    FKV_FIELD("FKV_CE_TWO_STREAMS", ce_two_streams),
    FKV_FIELD("FKV_D2H_LANE_RUNS", d2h_lane_runs),
    FKV_FIELD("FKV_STAGED_GATHER", staged_gather),
    FKV_FIELD("FKV_GATHER_THREADS", gather_threads),
    FKV_FIELD("FKV_MODEL_SEED", model_seed),
    FKV_FIELD("FKV_QUIET_WAIT_US", quiet_wait_us),
};
#undef FKV_FIELD

struct DevicePolicy {
  bool built = false;
  fkv_launch_policy derived{}; // from the device and the environment
  fkv_launch_policy current{};
};
std::mutex g_mu;
std::map<int, DevicePolicy> &tables() {
  static auto *t = new std::map<int, DevicePolicy>(); // lives until the process ends
  return *t;
}

int clampi(int v, int lo, int hi) { return v < lo ? lo : v > hi ? hi : v; }

// The figures of the cost model that depend on the host link of the box, as compiled in
// (an MI355X on PCIe Gen5 x16).  A table is re-based on a measurement of the device it
// belongs to the first time the model is needed (seed_from_measurement below); a field
// that no longer holds the compiled-in figure was set by the caller or the environment
// and is left alone.
struct LinkFigures {
  int link_mbps = 57200, kernel_d2h_mbps = 57000, kernel_h2d_mbps = 57200;
  int link_gbps_estimate = 45; // what other processes are told: 79 % of the link
  int copy_overhead_us = 10;
};
constexpr LinkFigures kCompiled{};

void seed_from_measurement(fkv_launch_policy &p, double d2h_gbps, double h2d_gbps,
                           double copy_overhead_us) {
  const bool rates_ok = d2h_gbps > 1.0 && d2h_gbps < 2000.0 && h2d_gbps > 1.0 && h2d_gbps < 2000.0;
  if (rates_ok) {
    const double mean = (d2h_gbps + h2d_gbps) / 2;
    if (p.model_link_mbps == kCompiled.link_mbps)
      p.model_link_mbps = (int)(mean * 1000 + 0.5);
    if (p.model_kernel_d2h_mbps == kCompiled.kernel_d2h_mbps)
      p.model_kernel_d2h_mbps = (int)(d2h_gbps * 1000 + 0.5);
    if (p.model_kernel_h2d_mbps == kCompiled.kernel_h2d_mbps)
      p.model_kernel_h2d_mbps = (int)(h2d_gbps * 1000 + 0.5);
    if (p.link_gbps_estimate == kCompiled.link_gbps_estimate)
      p.link_gbps_estimate = std::max(
          1, (int)(mean * kCompiled.link_gbps_estimate * 1000.0 / kCompiled.link_mbps + 0.5));
  }
  if (copy_overhead_us > 0.05 && copy_overhead_us < 1000.0 &&
      p.staged_copy_overhead_us == kCompiled.copy_overhead_us)
    p.staged_copy_overhead_us = std::max(1, (int)(copy_overhead_us + 0.5));
  if (rates_ok)
    p.model_seeded = 1;
}

// Masks from the sorted XCD ids of the device.
void derive_masks(fkv_launch_policy &p) {
  int ids[16], n = 0;
  for (int k = 0; k < 16; ++k)
    if ((p.xcd_present_mask >> k) & 1u)
      ids[n++] = k;
  const uint32_t all = p.xcd_present_mask;
  p.d2h_busy_mask = p.h2d_busy_mask = p.d2h_home_mask = p.h2d_home_mask = all;
  if (n < 4)
    return;
  uint32_t upper = 0, busy = 0, home = 0;
  for (int k = n / 2; k < n; ++k)
    upper |= 1u << ids[k];
  for (int k = 1; k <= n / 4; ++k)
    busy |= 1u << ids[k];
  for (int k = 1; k < n / 2; ++k)
    home |= 1u << ids[k];
  p.h2d_busy_mask = p.h2d_home_mask = upper;
  p.d2h_busy_mask = busy;
  p.d2h_home_mask = home;
}

void sanitize(fkv_launch_policy &p, const fkv_launch_policy &derived) {
  p.xcd_count = derived.xcd_count;
  p.xcd_present_mask = derived.xcd_present_mask;
  p.arbiter = clampi(p.arbiter, 0, 3);
  const uint32_t all = p.xcd_present_mask;
  for (uint32_t *m : {&p.d2h_busy_mask, &p.h2d_busy_mask, &p.d2h_home_mask, &p.h2d_home_mask}) {
    *m &= all;
    if (*m == 0)
      *m = all;
  }
  p.busy_window_ms = clampi(p.busy_window_ms, 0, 10000);
  p.d2h_busy_pct = clampi(p.d2h_busy_pct, 5, 1000);
  p.h2d_busy_pct = clampi(p.h2d_busy_pct, 5, 1000);
  p.busy_claims_per_wg = clampi(p.busy_claims_per_wg, 1, 64);
  p.home_claims_per_wg = clampi(p.home_claims_per_wg, 1, 64);
  p.all_claims_per_wg = clampi(p.all_claims_per_wg, 0, 64);
  p.safety_net_wait_us = clampi(p.safety_net_wait_us, 1, 100000);
  p.link_gbps_estimate = clampi(p.link_gbps_estimate, 1, 1000);
  p.d2h_wg_per_cta = clampi(p.d2h_wg_per_cta, 1, 256);
  p.h2d_wg_per_cta = clampi(p.h2d_wg_per_cta, 1, 256);
  p.d2h_wg_threads = clampi(p.d2h_wg_threads, 64, kCopyBlockThreads);
  p.h2d_wg_threads = clampi(p.h2d_wg_threads, 64, kCopyBlockThreads);
  p.packed_grid_pct = clampi(p.packed_grid_pct, 100, 400);
  p.plan_mirror = clampi(p.plan_mirror, -1, 1);
  p.fuse_launches = p.fuse_launches != 0;
  p.lane_streams = clampi(p.lane_streams, -1, 1);
  p.staged_restore = clampi(p.staged_restore, 0, 2);
  p.staged_ring = clampi(p.staged_ring, 2, 8);
  p.staged_copy_overhead_us = clampi(p.staged_copy_overhead_us, 0, 1000);
  p.staged_overhead_pct = clampi(p.staged_overhead_pct, 0, 100);
  p.staged_bridge_kb = clampi(p.staged_bridge_kb, 0, 1 << 20);
  p.staged_max_mb = clampi(p.staged_max_mb, 1, 1 << 16);
  p.hbm_workgroups = clampi(p.hbm_workgroups, 1, 1 << 16);
  p.hbm_wg_threads = clampi(p.hbm_wg_threads, 64, kCopyBlockThreads);
  p.hbm_unroll = p.hbm_unroll >= kCopyUnrollDeep ? kCopyUnrollDeep : kCopyUnroll;
  p.ce_staging_mb = clampi(p.ce_staging_mb, 1, 1 << 18);
  p.ce_two_streams = clampi(p.ce_two_streams, 0, 2);
  p.ce_rect_min_kb = clampi(p.ce_rect_min_kb, -1, 1 << 24);
  p.model_link_mbps = clampi(p.model_link_mbps, 100, 10000000);
  p.model_kernel_d2h_mbps = clampi(p.model_kernel_d2h_mbps, 100, 10000000);
  p.model_kernel_h2d_mbps = clampi(p.model_kernel_h2d_mbps, 100, 10000000);
  p.model_dma_ns = clampi(p.model_dma_ns, 0, 10000000);
  p.model_compaction_gbps = clampi(p.model_compaction_gbps, 1, 100000);
  p.model_host_pass_mbps = clampi(p.model_host_pass_mbps, 100, 10000000);
  p.model_launch_ns = clampi(p.model_launch_ns, 0, 10000000);
  p.model_prefer_ce_pct = clampi(p.model_prefer_ce_pct, 1, 1000);
  p.d2h_lane_runs = clampi(p.d2h_lane_runs, 0, 2);
  p.staged_gather = clampi(p.staged_gather, 0, 3);
  p.gather_threads = clampi(p.gather_threads, 1, 64);
  p.gather_ring = clampi(p.gather_ring, 2, 8);
  p.gather_first_by_kernel = p.gather_first_by_kernel != 0;
  p.model_gather_thread_mbps = clampi(p.model_gather_thread_mbps, 100, 10000000);
  p.model_seed = p.model_seed != 0;
  p.model_seeded = derived.model_seeded;
  p.staged_scatter_threads = clampi(p.staged_scatter_threads, 64, kCopyBlockThreads);
  p.test_fail_restore_batch = clampi(p.test_fail_restore_batch, 0, 1 << 20);
  p.staged_dma_streams = clampi(p.staged_dma_streams, 1, 2);
  p.kernel_alt_stream_kb = clampi(p.kernel_alt_stream_kb, 0, 1 << 20);
  p.quiet_wait_us = clampi(p.quiet_wait_us, -10000, 10000);
}

// The table of a device with the XCDs `present`, environment applied.
fkv_launch_policy defaults_for(uint32_t present) {
  fkv_launch_policy p{};
  p.xcd_present_mask = present;
  p.xcd_count = __builtin_popcount(present);
  derive_masks(p);
  p.arbiter = p.xcd_count >= 4 ? 1 : 0;
  p.busy_window_ms = 20;
  p.home_min_kb = 8192;
  p.d2h_busy_pct = 100;
  p.h2d_busy_pct = 150;
  p.busy_claims_per_wg = 1;
  p.home_claims_per_wg = 2;
  p.all_claims_per_wg = 0;
  p.safety_net_wait_us = 50;
  p.link_gbps_estimate = kCompiled.link_gbps_estimate;
  p.d2h_wg_per_cta = 12;
  p.h2d_wg_per_cta = 4;
  p.d2h_wg_threads = p.h2d_wg_threads = 64;
  p.packed_grid_pct = 150;
  p.plan_mirror = -1;
  p.fuse_launches = 1;
  p.lane_streams = -1;
  p.staged_restore = 1;
  p.staged_ring = 3;
  p.staged_copy_overhead_us = kCompiled.copy_overhead_us;
  p.staged_overhead_pct = 10;
  p.staged_bridge_kb = 512;
  p.staged_max_mb = 512;
  p.hbm_workgroups = 8192;
  p.hbm_wg_threads = 1024;
  p.hbm_unroll = kCopyUnrollDeep;
  p.ce_staging_mb = 1024;
  p.ce_two_streams = 1;
  p.ce_rect_min_kb = 32768; // 32 MiB and more: the same rate either way (3 GiB in copies of 32 MiB:
                            // 54.7 against 54.8 GB/s; of 128 MiB and of 1.5 GiB: equal), and the
                            // compute units stay free; 5 MiB copies: 51 against 56 GB/s
  // Measured on MI355X: a DMA command costs about 2.5 us beyond its bytes when copies
  // alternate over two streams (256 x 2 MiB: 50-54 GB/s; 2048 x 5 MiB: 56.2 GB/s); the
  // compaction pass stages 2.8 TB/s (512 MiB in 0.19 ms); a host scatter/gather pass
  // runs at about 20 GB/s with four threads; the gather/scatter kernel reaches
  // 57.0 GB/s GPU->host and 57.2 GB/s and more host->GPU.
  p.model_link_mbps = kCompiled.link_mbps;
  p.model_kernel_d2h_mbps = kCompiled.kernel_d2h_mbps;
  p.model_kernel_h2d_mbps = kCompiled.kernel_h2d_mbps;
  p.model_dma_ns = 2500;
  p.model_compaction_gbps = 2800;
  p.model_host_pass_mbps = 20000;
  p.model_launch_ns = 15000;
  p.model_prefer_ce_pct = 103;
  p.d2h_lane_runs = 1;
  // Host gather of scattered rows (72 KiB each, 16-core host of an MI355X box): one thread
  // 25-34 GB/s, four threads 79-96 GB/s, eight 120-125 GB/s; next to the copy engine reading
  // the previous buffer four threads still gather 36 MiB in 0.31-0.41 ms (0.67 ms on the
  // link), though once, in the first process on a fresh box, in 0.79 ms: six threads by
  // default, for the same thread time in sum.  20 GB/s a thread is the figure the choice
  // assumes.
  p.staged_gather = 1;
  p.gather_threads = 6;
  p.gather_ring = 4;
  p.gather_first_by_kernel = 1;
  p.model_gather_thread_mbps = 20000;
  p.model_seed = 1;
  p.model_seeded = 0;
  p.staged_scatter_threads = 256;
  p.staged_dma_streams = 2;
  p.kernel_alt_stream_kb = 4096;
  p.quiet_wait_us = 100;
  for (const EnvField &f : kEnv) {
    const char *v = std::getenv(f.name);
    if (v && *v) // decimal, 0x.. or 0.. as written
      *reinterpret_cast<int32_t *>(reinterpret_cast<char *>(&p) + f.offset) =
          (int32_t)std::strtol(v, nullptr, 0);
  }
  fkv_launch_policy derived = p;
  sanitize(p, derived);
  return p;
}

void build(int device, DevicePolicy &t) {
  uint32_t present = 0;
  {
    DeviceGuard guard(device);
    if (!guard.ok() || probe_xcds(&present) != FKV_OK || present == 0) {
      (void)hipGetLastError();
      present = 1; // one XCD as far as anybody can tell: nothing is split
    }
  }
  t.derived = t.current = defaults_for(present);
  t.built = true;
}

int resolve(int device, int *out) {
  if (device < 0)
    FKV_HIP_TRY(hipGetDevice(&device));
  *out = device;
  return FKV_OK;
}

} // namespace

fkv_launch_policy policy_of(int device) {
  std::lock_guard<std::mutex> lk(g_mu);
  DevicePolicy &t = tables()[device];
  if (!t.built)
    build(device, t);
  return t.current;
}

namespace {

// Cost of one more small copy command on the copy engines: a burst of 32 one-row 2-D
// copies of 2 KiB, host -> device, per copy, best of two bursts after a warm-up.
double measure_copy_overhead_us() {
  constexpr int kCopies = 32;
  constexpr size_t kBytes = 2048;
  void *h = nullptr, *d = nullptr;
  hipStream_t st = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  double best = 0;
  bool ok = hipHostMalloc(&h, kCopies * kBytes, hipHostMallocDefault) == hipSuccess &&
            hipMalloc(&d, kCopies * kBytes) == hipSuccess &&
            hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess &&
            hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
  if (ok)
    std::memset(h, 0x3c, kCopies * kBytes);
  for (int burst = 0; ok && burst < 3; ++burst) {
    ok = hipEventRecord(e0, st) == hipSuccess;
    for (int i = 0; ok && i < kCopies; ++i)
      ok = hipMemcpy2DAsync(static_cast<char *>(d) + i * kBytes, kBytes,
                            static_cast<char *>(h) + i * kBytes, kBytes, kBytes, 1,
                            hipMemcpyHostToDevice, st) == hipSuccess;
    float ms = 0;
    ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
         hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    if (ok && burst > 0 && ms > 0) {
      const double us = ms * 1e3 / kCopies;
      best = best == 0 ? us : std::min(best, us);
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (st) (void)hipStreamDestroy(st);
  if (d) (void)hipFree(d);
  if (h) (void)hipHostFree(h);
  (void)hipGetLastError();
  return ok ? best : 0;
}

std::mutex g_seed_mu; // one measurement at a time

} // namespace

fkv_launch_policy policy_of_seeded(int device) {
  fkv_launch_policy p = policy_of(device);
  if (!p.model_seed || p.model_seeded)
    return p;
  std::lock_guard<std::mutex> seeding(g_seed_mu);
  p = policy_of(device);
  if (!p.model_seed || p.model_seeded) // another thread was faster
    return p;
  double d2h = 0, h2d = 0, overhead_us = 0;
  {
    DeviceGuard guard(device);
    const std::string keep = fkv_last_error(); // a failed measurement is no error of the caller
    if (guard.ok() && fkv_measure_link_peak(device, (size_t)64 << 20, 3, 0, &d2h, nullptr) == FKV_OK &&
        fkv_measure_link_peak(device, (size_t)64 << 20, 3, 1, &h2d, nullptr) == FKV_OK)
      overhead_us = measure_copy_overhead_us();
    else
      d2h = h2d = 0;
    clear_error();
    if (!keep.empty())
      (void)fail(FKV_ERR_RUNTIME, "%s", keep.c_str());
  }
  std::lock_guard<std::mutex> lk(g_mu);
  DevicePolicy &t = tables()[device];
  seed_from_measurement(t.derived, d2h, h2d, overhead_us);
  seed_from_measurement(t.current, d2h, h2d, overhead_us);
  if (!t.current.model_seeded) // nothing usable came out: do not try again on every call
    t.derived.model_seed = t.current.model_seed = 0;
  return t.current;
}

fkv_launch_policy policy_sanitized(const fkv_launch_policy &in) {
  fkv_launch_policy p = in;
  fkv_launch_policy shape = in; // keeps the caller's XCD fields: no device is asked
  if (shape.xcd_present_mask == 0) {
    shape.xcd_present_mask = 1u;
    shape.xcd_count = 1;
  }
  sanitize(p, shape);
  return p;
}

fkv_launch_policy policy_peek(int device) {
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = tables().find(device);
  if (it != tables().end() && it->second.built)
    return it->second.current;
  return defaults_for(1u);
}

} // namespace fkv

extern "C" {

int fkv_launch_policy_get(int32_t device, fkv_launch_policy *out) try {
  using namespace fkv;
  clear_error();
  if (!out)
    return fail(FKV_ERR_INVALID_ARG, "fkv_launch_policy_get: null result pointer");
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  *out = policy_of(dev);
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_launch_policy_set(int32_t device, const fkv_launch_policy *in) try {
  using namespace fkv;
  clear_error();
  if (!in)
    return fail(FKV_ERR_INVALID_ARG, "fkv_launch_policy_set: null policy");
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  (void)policy_of(dev); // builds the table of the device
  std::lock_guard<std::mutex> lk(g_mu);
  DevicePolicy &t = tables()[dev];
  fkv_launch_policy p = *in;
  sanitize(p, t.derived);
  t.current = p;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_launch_policy_seed(int32_t device) try {
  using namespace fkv;
  clear_error();
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  (void)policy_of_seeded(dev);
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_launch_policy_seeded(const fkv_launch_policy *in, double d2h_gbps, double h2d_gbps,
                             double copy_overhead_us, fkv_launch_policy *out) try {
  using namespace fkv;
  clear_error();
  if (!in || !out)
    return fail(FKV_ERR_INVALID_ARG, "fkv_launch_policy_seeded: null argument");
  fkv_launch_policy p = *in;
  p.model_seeded = 0;
  seed_from_measurement(p, d2h_gbps, h2d_gbps, copy_overhead_us);
  *out = p;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_launch_policy_reset(int32_t device) try {
  using namespace fkv;
  clear_error();
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  (void)policy_of(dev);
  std::lock_guard<std::mutex> lk(g_mu);
  DevicePolicy &t = tables()[dev];
  t.current = t.derived;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
