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
  p.staged_gather = clampi(p.staged_gather, 0, 2);
  p.gather_threads = clampi(p.gather_threads, 1, 64);
  p.gather_ring = clampi(p.gather_ring, 2, 8);
  p.gather_first_by_kernel = p.gather_first_by_kernel != 0;
  p.model_gather_thread_mbps = clampi(p.model_gather_thread_mbps, 100, 10000000);
  p.model_seed = p.model_seed != 0;
  p.model_seeded = derived.model_seeded;
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
  p.link_gbps_estimate = 45;
  p.d2h_wg_per_cta = 12;
  p.h2d_wg_per_cta = 4;
  p.d2h_wg_threads = p.h2d_wg_threads = 64;
  p.packed_grid_pct = 150;
  p.plan_mirror = -1;
  p.fuse_launches = 1;
  p.lane_streams = -1;
  p.staged_restore = 1;
  p.staged_ring = 3;
  p.staged_copy_overhead_us = 10;
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
  p.model_link_mbps = 57200;
  p.model_kernel_d2h_mbps = 57000;
  p.model_kernel_h2d_mbps = 57200;
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

int fkv_launch_policy_get(int32_t device, fkv_launch_policy *out) {
  using namespace fkv;
  clear_error();
  if (!out)
    return fail(FKV_ERR_INVALID_ARG, "fkv_launch_policy_get: null result pointer");
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  *out = policy_of(dev);
  return FKV_OK;
}

int fkv_launch_policy_set(int32_t device, const fkv_launch_policy *in) {
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
}

int fkv_launch_policy_reset(int32_t device) {
  using namespace fkv;
  clear_error();
  int dev = 0;
  FKV_TRY(resolve(device, &dev));
  (void)policy_of(dev);
  std::lock_guard<std::mutex> lk(g_mu);
  DevicePolicy &t = tables()[dev];
  t.current = t.derived;
  return FKV_OK;
}

} // extern "C"
