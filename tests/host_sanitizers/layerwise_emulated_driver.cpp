// The library's whole host side over the emulated HIP runtime (emulated_hip_runtime.cpp),
// for sanitizer builds: layerwise restores with several ranks on every route (kernel, one
// copy per run of host blocks, rows gathered by host threads), asked for on the kernel and
// on the copy engine, from pinned and pageable host pools, in both notify modes with
// eventfds, consumer streams gated per layer, restores made to give up part-way; and plain
// puts and gets on the kernel path and through every copy-engine strategy.  Every result is
// compared with a plain model of the addressing (vLLM-style tensors per layer).
#include <hip/hip_runtime_api.h>
#include <sys/eventfd.h>
#include <unistd.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "fkv_transfer.h"

namespace fkv {
void plan_pool_counts(int *slots, int *handed_out); // fkv_core.cpp: the pool of plan memory
}

// the CPU restatement of the reference's rank placement and byte loop (oracle/fkv_oracle.c)
extern "C" {
typedef struct {
  int32_t active;
  int32_t start_layer;
  int32_t num_layers;
  int32_t reserved;
  int64_t cpu_startoff;
  int64_t gpu_startoff;
  int64_t chunk_size;
} fkv_oracle_rank_plan;
int fkv_oracle_tp_rank_plan(int rank, int num_gpus, int num_kv_heads, int is_host_to_device,
                            const char *mode_in, int designated_rank, int rotate_counter,
                            int layer_id, int layer_granularity, int num_blocks,
                            int64_t gpu_chunk_size, int64_t cpu_block_stride, int64_t cpu_tp_stride,
                            fkv_oracle_rank_plan *out);
long fkv_emulated_fail(int category, long after, long count); // emulated_hip_runtime.cpp
unsigned long long fkv_emulated_workgroups_run();             // 0: the kernels are stand-ins
long fkv_emulated_host_waited_copies();                        // hipMemcpy calls so far
int fkv_oracle_transfer(int backend, const uint64_t *tensor_ptrs, int64_t num_layers_total,
                        int64_t gpu_kv_stride, int64_t gpu_block_stride, int64_t gpu_layer_stride,
                        int64_t gpu_off, uint8_t *cpu_ptr, int64_t cpu_kv_stride,
                        int64_t cpu_layer_stride, int64_t cpu_block_stride, int64_t cpu_off,
                        int64_t chunk, int start_layer, int num_layers, int kv_dim, int num_blocks,
                        const int64_t *gpu_ids, const int64_t *cpu_ids, int is_host_to_device);
}

#define REQUIRE(cond, ...)                                                                          \
  do {                                                                                              \
    if (!(cond)) {                                                                                  \
      fprintf(stderr, "FAILED %s:%d: %s\n  ", __FILE__, __LINE__, #cond);                           \
      fprintf(stderr, __VA_ARGS__);                                                                 \
      fprintf(stderr, "\n  last error: %s\n", fkv_last_error());                                    \
      exit(1);                                                                                      \
    }                                                                                               \
  } while (0)

namespace {

struct Shape {
  int ranks, L, kv, NG, NC;
  int64_t chunk;
  bool blockfirst;
  // engine tensors: per rank and layer [kv, NG, chunk]
  int64_t gpu_kv_stride() const { return (int64_t)NG * chunk; }
  int64_t gpu_block_stride() const { return chunk; }
  int64_t layer_bytes() const { return (int64_t)kv * NG * chunk; }
  // host pool: block-first [NC, L, kv, chunk] or layer-first [L, kv, NC, chunk]
  int64_t cpu_kv_stride() const { return blockfirst ? chunk : (int64_t)NC * chunk; }
  int64_t cpu_layer_stride() const { return blockfirst ? kv * chunk : (int64_t)kv * NC * chunk; }
  int64_t cpu_block_stride() const { return blockfirst ? (int64_t)L * kv * chunk : chunk; }
  int64_t host_bytes() const { return (int64_t)NC * L * kv * chunk; }
};

struct Tensors {
  std::vector<std::vector<uint8_t *>> dev; // [rank][layer], "device" memory
  std::vector<std::vector<std::vector<uint8_t>>> model; // the same, as the model sees it
  uint8_t *host = nullptr;
  bool host_pinned = true;
};

void fill(std::mt19937_64 &rng, uint8_t *p, size_t n) {
  for (size_t i = 0; i < n; i += 8) {
    const uint64_t v = rng();
    std::memcpy(p + i, &v, std::min<size_t>(8, n - i));
  }
}

void set_policy(const std::vector<std::pair<std::string, int>> &fields) {
  fkv_launch_policy p{};
  REQUIRE(fkv_launch_policy_reset(0) == FKV_OK, "policy reset");
  REQUIRE(fkv_launch_policy_get(0, &p) == FKV_OK, "policy get");
  for (const auto &f : fields) {
    if (f.first == "staged_restore") p.staged_restore = f.second;
    else if (f.first == "staged_gather") p.staged_gather = f.second;
    else if (f.first == "gather_threads") p.gather_threads = f.second;
    else if (f.first == "gather_ring") p.gather_ring = f.second;
    else if (f.first == "staged_ring") p.staged_ring = f.second;
    else if (f.first == "gather_first_by_kernel") p.gather_first_by_kernel = f.second;
    else if (f.first == "staged_dma_streams") p.staged_dma_streams = f.second;
    else if (f.first == "kernel_alt_stream_kb") p.kernel_alt_stream_kb = f.second;
    else if (f.first == "test_fail_restore_batch") p.test_fail_restore_batch = f.second;
    else if (f.first == "model_seed") p.model_seed = f.second;
    else REQUIRE(false, "unknown policy field %s", f.first.c_str());
  }
  REQUIRE(fkv_launch_policy_set(0, &p) == FKV_OK, "policy set");
}

int drain(int fd) {
  uint64_t v = 0;
  int units = 0;
  while (read(fd, &v, 8) == 8)
    units += (int)v;
  return units;
}

// What a case is drawn from; a field >= 0 pins the choice.
struct Pinned {
  int ranks = -1, L = -1, kv = -1, NG = -1, NC = -1, chunk16 = -1, blockfirst = -1, mode = -1,
      pageable = -1, route = -1, use_ce = -1, with_fds = -1;
};

// One group, a few restores, everything compared.
void layerwise_case(uint64_t seed, const Pinned &fix = Pinned()) {
  std::mt19937_64 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  auto pinned = [](int drawn, int fixed) { return fixed >= 0 ? fixed : drawn; };
  Shape s{};
  s.ranks = pinned(std::vector<int>{1, 2, 4}[pick(0, 2)], fix.ranks);
  s.L = pinned(pick(1, 18), fix.L);
  s.kv = pinned(pick(1, 2), fix.kv);
  s.NG = pinned(pick(6, 40), fix.NG);
  s.NC = pinned(pick(6, 48), fix.NC);
  s.chunk = 16 * pinned(pick(1, 96), fix.chunk16);
  s.blockfirst = pinned((int)(rng() & 1), fix.blockfirst);
  const std::string mode =
      std::vector<std::string>{"sharded", "all_write", "rank0_only"}[pinned(pick(0, 2), fix.mode)];
  const int copies = mode == "all_write" ? s.ranks : 1;
  const int pool_blocks = s.NC;
  s.NC *= copies; // rank r of an all_write restore reads n blocks further on, see below
  const bool pageable = pinned((rng() % 5) == 0, fix.pageable);
  const int route = pinned(pick(0, 3), fix.route); // 0 the library's choice, 1 kernel, 2 copy per run, 3 gathered
  const bool use_ce = pinned((rng() % 3) == 0, fix.use_ce);
  const bool with_fds = pinned((int)(rng() & 1), fix.with_fds);
  const int counters = 2;

  Tensors t;
  t.host_pinned = !pageable;
  if (pageable)
    t.host = static_cast<uint8_t *>(malloc((size_t)s.host_bytes()));
  else
    REQUIRE(hipHostMalloc((void **)&t.host, (size_t)s.host_bytes(), 0) == hipSuccess, "host pool");
  t.dev.resize(s.ranks);
  t.model.resize(s.ranks);
  std::vector<uint64_t> ptrs;
  for (int r = 0; r < s.ranks; ++r)
    for (int l = 0; l < s.L; ++l) {
      uint8_t *d = nullptr;
      REQUIRE(hipMalloc((void **)&d, (size_t)s.layer_bytes()) == hipSuccess, "engine tensor");
      std::vector<uint8_t> init((size_t)s.layer_bytes());
      fill(rng, init.data(), init.size());
      std::memcpy(d, init.data(), init.size());
      t.dev[r].push_back(d);
      t.model[r].push_back(std::move(init));
      ptrs.push_back((uint64_t)(uintptr_t)d);
    }
  std::vector<int32_t> fds;
  if (with_fds)
    for (int i = 0; i < counters * s.ranks * s.L; ++i)
      fds.push_back(eventfd(0, EFD_NONBLOCK));
  std::vector<int64_t> kvs(s.ranks, s.gpu_kv_stride()), bs(s.ranks, s.gpu_block_stride()),
      ls(s.ranks, s.layer_bytes()), cs(s.ranks, s.chunk), devs(s.ranks, 0);
  fkv_layerwise_params p{};
  p.num_gpus = s.ranks;
  p.num_tensors_per_gpu = s.L;
  p.gpu_block_ptrs_flat = ptrs.data();
  p.cpu_blocks_ptr = t.host;
  p.num_layers = s.L;
  p.tp_size = s.ranks;
  p.gpu_kv_strides = kvs.data();
  p.gpu_block_strides = bs.data();
  p.gpu_layer_strides = ls.data();
  p.gpu_chunk_sizes = cs.data();
  p.gpu_device_ids = devs.data();
  p.layer_eventfds = fds.empty() ? nullptr : fds.data();
  p.num_layer_eventfds = (int32_t)fds.size();
  fkv_ce_config_default(&p.ce);
  p.ce.is_blockfirst = s.blockfirst;
  p.ce.num_kv_heads = 1;
  p.ce.gather_threads = pick(0, 3);
  p.ce.enable_memcpy2d = rng() & 1;
  fkv_layerwise *g = nullptr;
  REQUIRE(fkv_layerwise_create(&p, &g) == FKV_OK, "create");

  std::vector<std::pair<std::string, int>> pol = {
      {"model_seed", 0}, {"gather_threads", pick(2, 4)}, {"gather_ring", pick(2, 4)},
      {"staged_ring", pick(2, 4)}, {"gather_first_by_kernel", pick(0, 1)},
      {"staged_dma_streams", pick(1, 2)}, {"kernel_alt_stream_kb", (rng() & 1) ? 4096 : 0}};
  if (route == 1) { pol.push_back({"staged_restore", 0}); pol.push_back({"staged_gather", 0}); }
  if (route == 2) { pol.push_back({"staged_restore", 2}); pol.push_back({"staged_gather", 0}); }
  // 3: also in groups of several GPUs, where the library does not take the route by itself
  if (route == 3) { pol.push_back({"staged_restore", 0}); pol.push_back({"staged_gather", 3}); }
  set_policy(pol);

  hipStream_t consumer = nullptr;
  REQUIRE(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking) == hipSuccess, "stream");
  std::vector<uint8_t> seen((size_t)s.layer_bytes()); // what the consumer copies out of layer l
  for (int rep = 0; rep < 3; ++rep) {
    // the engine names its stream: at set-up, or between two restores
    if (rng() % 3 == 0) {
      int32_t sharing = -1;
      const int named = fkv_layerwise_set_compute_stream(g, pick(0, s.ranks - 1),
                                                         (rng() & 1) ? consumer : nullptr, &sharing);
      REQUIRE(named == FKV_OK && sharing == 0,
              "seed %llu rep %d: set_compute_stream rc %d, %d streams share the queue",
              (unsigned long long)seed, rep, named, sharing);
    }
    fill(rng, t.host, (size_t)s.host_bytes());
    const int n = pick(0, std::min(s.NG, pool_blocks));
    std::vector<int64_t> gids(s.NG), cids(pool_blocks);
    std::iota(gids.begin(), gids.end(), 0);
    std::iota(cids.begin(), cids.end(), 0);
    std::shuffle(gids.begin(), gids.end(), rng);
    if (rng() & 1)
      std::shuffle(cids.begin(), cids.end(), rng);
    else
      std::rotate(cids.begin(), cids.begin() + pick(0, pool_blocks - 1), cids.end());
    gids.resize(n);
    cids.resize(n);
    if (mode == "all_write") // rank r reads blocks [r*n, (r+1)*n) further on: ids stay below n
      for (int i = 0; i < n; ++i)
        cids[i] = i;
    const int layers = pick(1, s.L), gran = pick(1, s.L);
    const int notify = (rng() & 1) ? FKV_NOTIFY_POLLING : FKV_NOTIFY_HOSTFUNC;
    const int counter = pick(0, counters - 1);
    const int give_up = (rng() % 6) == 0 ? pick(1, (layers + gran - 1) / gran) : 0;
    if (give_up) {
      auto q = pol;
      q.push_back({"test_fail_restore_batch", give_up});
      set_policy(q);
    }
    const bool kernel_only = route == 1 || (pageable && route != 3 && route != 0);
    const int rc = fkv_layerwise_transfer(
        g, gids.data(), cids.data(), n, s.cpu_block_stride(), s.cpu_kv_stride(),
        s.cpu_layer_stride(), s.cpu_block_stride(), 4, use_ce, layers, gran, s.kv, 1, counter,
        mode.c_str(), notify, 0);
    // a pageable pool has no kernel route: refused unless the copy engine was asked for or
    // rows can be gathered
    const bool refused_ok = pageable && !use_ce && n > 0;
    if (rc != FKV_OK && !give_up) {
      REQUIRE(refused_ok && (kernel_only || route == 0 || route == 2),
              "seed %llu rep %d: restore refused", (unsigned long long)seed, rep);
      REQUIRE(fkv_layerwise_synchronize(g) == FKV_OK, "synchronize after a refusal");
      continue;
    }
    // a consumer gated on a layer sees that layer whole
    const int watch = pick(0, layers - 1);
    if (rc == FKV_OK) {
      if (!give_up && n > 0) {
        REQUIRE(fkv_layerwise_wait_layer(g, 0, watch, consumer) == FKV_OK, "wait_layer");
        REQUIRE(hipMemcpyAsync(seen.data(), t.dev[0][watch], seen.size(), hipMemcpyDeviceToHost,
                               consumer) == hipSuccess, "consumer copy");
      }
    }
    const int src = fkv_layerwise_synchronize(g);
    REQUIRE(hipStreamSynchronize(consumer) == hipSuccess, "consumer");
    if (give_up) {
      // the call or the synchronize reports it; what landed is a prefix of the batches
      REQUIRE(rc != FKV_OK || src != FKV_OK || n == 0 || give_up > (layers + gran - 1) / gran,
              "seed %llu: a restore that gave up went unreported", (unsigned long long)seed);
      set_policy(pol);
      // re-base the model on what is there: the next restore must be whole again
      for (int r = 0; r < s.ranks; ++r)
        for (int l = 0; l < s.L; ++l)
          std::memcpy(t.model[r][l].data(), t.dev[r][l], (size_t)s.layer_bytes());
      for (int fd : fds)
        drain(fd);
      continue;
    }
    REQUIRE(src == FKV_OK, "seed %llu rep %d: synchronize", (unsigned long long)seed, rep);
    // the model: rank r, layer l < layers, kv, position p
    for (int r = 0; r < s.ranks; ++r) {
      const int64_t off = mode == "all_write" ? (int64_t)r * n * s.cpu_block_stride() : 0;
      for (int l = 0; l < layers; ++l)
        for (int k = 0; k < s.kv; ++k)
          for (int q = 0; q < n; ++q)
            std::memcpy(t.model[r][l].data() + k * s.gpu_kv_stride() + gids[q] * s.chunk,
                        t.host + off + cids[q] * s.cpu_block_stride() + l * s.cpu_layer_stride() +
                            k * s.cpu_kv_stride(),
                        (size_t)s.chunk);
    }
    for (int r = 0; r < s.ranks; ++r)
      for (int l = 0; l < s.L; ++l)
        REQUIRE(std::memcmp(t.dev[r][l], t.model[r][l].data(), (size_t)s.layer_bytes()) == 0,
                "seed %llu rep %d: rank %d layer %d differs (route %d use_ce %d pageable %d mode %s "
                "gran %d layers %d n %d)", (unsigned long long)seed, rep, r, l, route, (int)use_ce,
                (int)pageable, mode.c_str(), gran, layers, n);
    if (n > 0)
      REQUIRE(std::memcmp(seen.data(), t.model[0][watch].data(), seen.size()) == 0,
              "seed %llu rep %d: the consumer gated on layer %d saw other bytes",
              (unsigned long long)seed, rep, watch);
    if (with_fds) {
      for (int c = 0; c < counters; ++c)
        for (int r = 0; r < s.ranks; ++r)
          for (int l = 0; l < s.L; ++l) {
            const int units = drain(fds[((size_t)c * s.ranks + r) * s.L + l]);
            REQUIRE(units == (c == counter && l < layers ? 1 : 0),
                    "seed %llu rep %d: eventfd counter %d rank %d layer %d has %d units",
                    (unsigned long long)seed, rep, c, r, l, units);
          }
    }
  }
  REQUIRE(hipStreamDestroy(consumer) == hipSuccess, "stream destroy");
  fkv_layerwise_destroy(g);
  for (int fd : fds)
    close(fd);
  for (auto &rank : t.dev)
    for (uint8_t *d : rank)
      REQUIRE(hipFree(d) == hipSuccess, "free");
  if (pageable)
    free(t.host);
  else
    REQUIRE(hipHostFree(t.host) == hipSuccess, "host free");
}

// Plain puts and gets: kernel path and every copy-engine strategy the ids lead to.
void transfer_case(uint64_t seed) {
  std::mt19937_64 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  Shape s{};
  s.ranks = 1;
  s.L = pick(1, 6);
  s.kv = pick(1, 2);
  s.NG = pick(4, 40);
  s.NC = pick(4, 40);
  s.chunk = 8 * pick(1, 300);
  s.blockfirst = rng() & 1;
  std::vector<uint8_t *> dev;
  std::vector<std::vector<uint8_t>> model;
  std::vector<uint64_t> ptrs;
  for (int l = 0; l < s.L; ++l) {
    uint8_t *d = nullptr;
    REQUIRE(hipMalloc((void **)&d, (size_t)s.layer_bytes()) == hipSuccess, "engine tensor");
    std::vector<uint8_t> init((size_t)s.layer_bytes());
    fill(rng, init.data(), init.size());
    std::memcpy(d, init.data(), init.size());
    dev.push_back(d);
    model.push_back(std::move(init));
    ptrs.push_back((uint64_t)(uintptr_t)d);
  }
  uint8_t *host = nullptr;
  REQUIRE(hipHostMalloc((void **)&host, (size_t)s.host_bytes(), 0) == hipSuccess, "host pool");
  std::vector<uint8_t> host_model((size_t)s.host_bytes());
  fill(rng, host_model.data(), host_model.size());
  std::memcpy(host, host_model.data(), host_model.size());
  hipStream_t st = nullptr;
  REQUIRE(hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess, "stream");
  set_policy({{"model_seed", 0}});
  for (int rep = 0; rep < 8; ++rep) {
    const int n = pick(0, std::min(s.NG, s.NC));
    std::vector<int64_t> gids(s.NG), cids(s.NC);
    std::iota(gids.begin(), gids.end(), 0);
    std::iota(cids.begin(), cids.end(), 0);
    const int pattern = pick(0, 2); // scattered, one run on both sides, runs on the host side
    if (pattern == 0) {
      std::shuffle(gids.begin(), gids.end(), rng);
      std::shuffle(cids.begin(), cids.end(), rng);
    } else if (pattern == 2) {
      std::shuffle(gids.begin(), gids.end(), rng);
    }
    gids.resize(n);
    cids.resize(n);
    fkv_transfer_desc d{};
    d.backend = FKV_BACKEND_VLLM;
    d.num_layers_total = s.L;
    d.gpu_tensor_ptrs = ptrs.data();
    d.num_gpu_tensor_ptrs = s.L;
    d.device = -1;
    d.gpu_kv_stride = s.gpu_kv_stride();
    d.gpu_block_stride = s.gpu_block_stride();
    d.gpu_layer_stride = s.layer_bytes();
    d.cpu_ptr = host;
    d.cpu_kv_stride = s.cpu_kv_stride();
    d.cpu_layer_stride = s.cpu_layer_stride();
    d.cpu_block_stride = s.cpu_block_stride();
    d.chunk_size = s.chunk;
    d.start_layer_id = pick(0, s.L - 1);
    d.num_layers = pick(1, s.L - d.start_layer_id);
    d.kv_dim = s.kv;
    d.num_blocks = n;
    d.gpu_block_ids = gids.data();
    d.cpu_block_ids = cids.data();
    d.is_host_to_device = rng() & 1;
    d.use_ce_transfer = pick(0, 2);
    d.transfer_num_cta = pick(1, 8);
    d.sync = rng() & 1;
    fkv_ce_config_default(&d.ce);
    d.ce.is_blockfirst = s.blockfirst;
    d.ce.num_kv_heads = (rng() & 1) ? 1 : 8;
    d.ce.segment_threshold = (rng() & 1) ? 8 : 2;
    d.ce.path_opt_enabled = (rng() % 4) != 0;
    d.ce.enable_memcpy2d = rng() & 1;
    d.ce.gather_threads = pick(0, 4);
    d.ce.gather_nt = rng() & 1;
    // every third transfer with the runtime refusing something part-way: it may fail, and what
    // it leaves behind is the starting point of the next one
    const bool inject = rep % 3 == 2;
    if (inject)
      fkv_emulated_fail(pick(0, 7), pick(0, 6), pick(1, 2));
    const int rc = fkv_transfer_kv_blocks(&d, st);
    REQUIRE(hipStreamSynchronize(st) == hipSuccess, "sync");
    for (int c = 0; c < 8; ++c)
      fkv_emulated_fail(c, 0, 0);
    REQUIRE(rc == FKV_OK || inject, "seed %llu rep %d: transfer", (unsigned long long)seed, rep);
    if (rc != FKV_OK) {
      { // the library's own streams included
        void *probe = nullptr;
        REQUIRE(hipMalloc(&probe, 64) == hipSuccess && hipFree(probe) == hipSuccess, "drain");
      }
      for (int l = 0; l < s.L; ++l)
        std::memcpy(model[l].data(), dev[l], (size_t)s.layer_bytes());
      std::memcpy(host_model.data(), host, host_model.size());
      continue;
    }
    for (int l = d.start_layer_id; l < d.start_layer_id + d.num_layers; ++l)
      for (int k = 0; k < s.kv; ++k)
        for (int q = 0; q < n; ++q) {
          uint8_t *gm = model[l].data() + k * s.gpu_kv_stride() + gids[q] * s.chunk;
          uint8_t *hm = host_model.data() + cids[q] * s.cpu_block_stride() +
                        l * s.cpu_layer_stride() + k * s.cpu_kv_stride();
          if (d.is_host_to_device)
            std::memcpy(gm, hm, (size_t)s.chunk);
          else
            std::memcpy(hm, gm, (size_t)s.chunk);
        }
    for (int l = 0; l < s.L; ++l)
      REQUIRE(std::memcmp(dev[l], model[l].data(), (size_t)s.layer_bytes()) == 0,
              "seed %llu rep %d: layer %d differs (path %d)", (unsigned long long)seed, rep, l,
              fkv_last_path());
    REQUIRE(std::memcmp(host, host_model.data(), host_model.size()) == 0,
            "seed %llu rep %d: host pool differs (path %d)", (unsigned long long)seed, rep,
            fkv_last_path());
  }
  REQUIRE(hipStreamDestroy(st) == hipSuccess, "stream destroy");
  for (uint8_t *d : dev)
    REQUIRE(hipFree(d) == hipSuccess, "free");
  REQUIRE(hipHostFree(host) == hipSuccess, "host free");
}

// The thread group of a tensor-parallel engine: a thread per rank inside the library, every
// shared-KV mode and head slices of multi-head KV, against the oracle's rank plan and byte loop.
void tp_case(uint64_t seed) {
  std::mt19937_64 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  const int n = std::vector<int>{1, 2, 4}[pick(0, 2)];
  const bool shared = rng() & 1;             // KV identical on all ranks (one KV head)
  const int heads = shared ? 1 : n * pick(1, 2);
  Shape s{};
  s.ranks = n;
  s.L = pick(1, 7);
  s.kv = pick(1, 2);
  s.NG = pick(4, 24);
  s.chunk = 16 * n * pick(1, 24);            // what one rank holds of a block and layer
  s.blockfirst = rng() & 1;
  const std::string mode = std::vector<std::string>{"sharded", "all_write", "rank0_only",
                                                    "layer_parallel", "rank_rotate", "bogus"}[pick(0, 5)];
  const int copies = shared && mode == "all_write" ? n : 1;
  const int pool_blocks = pick(4, 24);
  const int64_t host_chunk = shared ? s.chunk : s.chunk * n; // multi-head: every rank's slice side by side
  // host pool [NC, L, kv, host_chunk] or [L, kv, NC, host_chunk]
  const int NC = pool_blocks * copies;
  const int64_t cpu_block_stride = s.blockfirst ? (int64_t)s.L * s.kv * host_chunk : host_chunk;
  const int64_t host_bytes = (int64_t)NC * s.L * s.kv * host_chunk;
  // strides a rank uses inside its share: the per-rank layout of the reference's workers
  // (flexkv/transfer/worker.py:1199-1204): block-first, a rank's chunks of a block lie together
  int64_t cpu_kv_stride, cpu_layer_stride, cpu_tp_stride;
  if (shared) {
    cpu_kv_stride = s.blockfirst ? host_chunk : (int64_t)NC * host_chunk;
    cpu_layer_stride = s.blockfirst ? s.kv * host_chunk : (int64_t)s.kv * NC * host_chunk;
    cpu_tp_stride = cpu_block_stride;
  } else {
    cpu_kv_stride = s.blockfirst ? s.chunk : (int64_t)NC * host_chunk;
    cpu_layer_stride = s.blockfirst ? s.kv * s.chunk : (int64_t)s.kv * NC * host_chunk;
    cpu_tp_stride = cpu_block_stride / n;
  }
  uint8_t *host = nullptr;
  REQUIRE(hipHostMalloc((void **)&host, (size_t)host_bytes, 0) == hipSuccess, "host pool");
  std::vector<uint8_t> host_model((size_t)host_bytes);
  fill(rng, host_model.data(), host_model.size());
  std::memcpy(host, host_model.data(), host_model.size());
  std::vector<std::vector<uint8_t *>> dev(n);
  std::vector<std::vector<std::vector<uint8_t>>> model(n);
  std::vector<uint64_t> ptrs;
  for (int r = 0; r < n; ++r)
    for (int l = 0; l < s.L; ++l) {
      uint8_t *d = nullptr;
      REQUIRE(hipMalloc((void **)&d, (size_t)s.layer_bytes()) == hipSuccess, "engine tensor");
      std::vector<uint8_t> init((size_t)s.layer_bytes());
      fill(rng, init.data(), init.size());
      std::memcpy(d, init.data(), init.size());
      dev[r].push_back(d);
      model[r].push_back(std::move(init));
      ptrs.push_back((uint64_t)(uintptr_t)d);
    }
  std::vector<int64_t> kvs(n, s.gpu_kv_stride()), bs(n, s.gpu_block_stride()), ls(n, s.layer_bytes()),
      cs(n, s.chunk), devs(n, 0);
  fkv_tp_group_params p{};
  p.num_gpus = n;
  p.num_tensors_per_gpu = s.L;
  p.gpu_block_ptrs_flat = ptrs.data();
  p.cpu_blocks_ptr = host;
  p.num_layers = s.L;
  p.gpu_kv_strides = kvs.data();
  p.gpu_block_strides = bs.data();
  p.gpu_layer_strides = ls.data();
  p.gpu_chunk_sizes = cs.data();
  p.gpu_device_ids = devs.data();
  fkv_ce_config_default(&p.ce);
  p.ce.is_blockfirst = s.blockfirst;
  p.ce.num_kv_heads = heads;
  p.ce.gather_threads = pick(0, 3);
  fkv_tp_group *g = nullptr;
  REQUIRE(fkv_tp_group_create(&p, &g) == FKV_OK, "tp group");
  set_policy({{"model_seed", 0}});
  int puts = 0; // rank_rotate moves on with every put
  for (int rep = 0; rep < 6; ++rep) {
    const int nb = pick(0, std::min(s.NG, pool_blocks));
    std::vector<int64_t> gids(s.NG), cids(pool_blocks);
    std::iota(gids.begin(), gids.end(), 0);
    std::iota(cids.begin(), cids.end(), 0);
    std::shuffle(gids.begin(), gids.end(), rng);
    if (rng() & 1)
      std::shuffle(cids.begin(), cids.end(), rng);
    gids.resize(nb);
    cids.resize(nb);
    if (copies > 1) // rank r's region starts r * nb blocks further on
      for (int i = 0; i < nb; ++i)
        cids[i] = i;
    const bool valid_get = !shared || mode == "sharded" || mode == "all_write" || mode == "rank0_only";
    const int h2d = valid_get ? (int)(rng() & 1) : 0;
    const int layer_id = pick(0, s.L - 1), gran = pick(1, s.L - layer_id);
    const int use_ce = s.chunk % 8 == 0 ? pick(0, 1) : 0;
    const int designated = pick(0, n - 1);
    // every third call with the runtime refusing something in one of the rank threads
    const bool inject = rep % 3 == 2;
    if (inject)
      fkv_emulated_fail(pick(0, 7), pick(0, 4), pick(1, 2));
    const int rc = fkv_tp_group_transfer(g, gids.data(), cids.data(), nb, cpu_kv_stride,
                                         cpu_layer_stride, cpu_block_stride, cpu_tp_stride, 4, h2d,
                                         use_ce, layer_id, gran, s.kv, heads, mode.c_str(), designated);
    for (int c = 0; c < 8; ++c)
      fkv_emulated_fail(c, 0, 0);
    REQUIRE(rc == FKV_OK || inject, "seed %llu rep %d: tp transfer (mode %s h2d %d ce %d)",
            (unsigned long long)seed, rep, mode.c_str(), h2d, use_ce);
    if (rc != FKV_OK) {
      { // whatever the ranks left in flight
        void *probe = nullptr;
        REQUIRE(hipMalloc(&probe, 64) == hipSuccess && hipFree(probe) == hipSuccess, "drain");
      }
      for (int r = 0; r < n; ++r)
        for (int l = 0; l < s.L; ++l)
          std::memcpy(model[r][l].data(), dev[r][l], (size_t)s.layer_bytes());
      std::memcpy(host_model.data(), host, host_model.size());
      if (!h2d && shared && mode == "rank_rotate")
        ++puts; // the writer moves on with every put that was asked for
      continue;
    }
    for (int r = 0; r < n; ++r) {
      fkv_oracle_rank_plan plan{};
      REQUIRE(fkv_oracle_tp_rank_plan(r, n, heads, h2d, mode.c_str(), designated, puts % n, layer_id,
                                      gran, nb, s.chunk, cpu_block_stride, cpu_tp_stride, &plan) == 0,
              "rank plan");
      if (!plan.active)
        continue;
      std::vector<uint64_t> mp;
      for (int l = 0; l < s.L; ++l)
        mp.push_back((uint64_t)(uintptr_t)model[r][l].data());
      REQUIRE(fkv_oracle_transfer(0, mp.data(), s.L, s.gpu_kv_stride(), s.gpu_block_stride(),
                                  s.layer_bytes(), plan.gpu_startoff, host_model.data(), cpu_kv_stride,
                                  cpu_layer_stride, cpu_block_stride, plan.cpu_startoff,
                                  plan.chunk_size, plan.start_layer, plan.num_layers, s.kv, nb,
                                  gids.data(), cids.data(), h2d) == 0, "oracle transfer");
    }
    if (!h2d)
      ++puts;
    for (int r = 0; r < n; ++r)
      for (int l = 0; l < s.L; ++l)
        REQUIRE(std::memcmp(dev[r][l], model[r][l].data(), (size_t)s.layer_bytes()) == 0,
                "seed %llu rep %d: rank %d layer %d differs (mode %s h2d %d ce %d heads %d)",
                (unsigned long long)seed, rep, r, l, mode.c_str(), h2d, use_ce, heads);
    REQUIRE(std::memcmp(host, host_model.data(), host_model.size()) == 0,
            "seed %llu rep %d: host pool differs (mode %s h2d %d ce %d heads %d ranks %d)",
            (unsigned long long)seed, rep, mode.c_str(), h2d, use_ce, heads, n);
  }
  fkv_tp_group_destroy(g);
  for (auto &rank : dev)
    for (uint8_t *d : rank)
      REQUIRE(hipFree(d) == hipSuccess, "free");
  REQUIRE(hipHostFree(host) == hipSuccess, "host free");
}

// Puts and gets from several threads at once, a stream each, on blocks of their own: plan
// memory, claim counters, the arbiter's view of the link and the library's lane streams under
// concurrent calls.
void concurrent_case(uint64_t seed) {
  std::mt19937_64 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  const int threads = pick(2, 5), per = pick(3, 10);
  Shape s{};
  s.ranks = 1;
  s.L = pick(1, 5);
  s.kv = pick(1, 2);
  s.NG = threads * per;
  s.NC = threads * per;
  s.chunk = 16 * pick(1, 64);
  s.blockfirst = rng() & 1;
  std::vector<uint8_t *> dev;
  std::vector<std::vector<uint8_t>> model;
  std::vector<uint64_t> ptrs;
  for (int l = 0; l < s.L; ++l) {
    uint8_t *d = nullptr;
    REQUIRE(hipMalloc((void **)&d, (size_t)s.layer_bytes()) == hipSuccess, "engine tensor");
    std::vector<uint8_t> init((size_t)s.layer_bytes());
    fill(rng, init.data(), init.size());
    std::memcpy(d, init.data(), init.size());
    dev.push_back(d);
    model.push_back(std::move(init));
    ptrs.push_back((uint64_t)(uintptr_t)d);
  }
  uint8_t *host = nullptr;
  REQUIRE(hipHostMalloc((void **)&host, (size_t)s.host_bytes(), 0) == hipSuccess, "host pool");
  std::vector<uint8_t> host_model((size_t)s.host_bytes());
  fill(rng, host_model.data(), host_model.size());
  std::memcpy(host, host_model.data(), host_model.size());
  set_policy({{"model_seed", 0}});
  struct Op {
    std::vector<int64_t> gids, cids;
    int h2d, sync, use_ce;
  };
  std::vector<std::vector<Op>> script(threads);
  for (int t = 0; t < threads; ++t)
    for (int k = 0; k < 6; ++k) {
      Op op;
      const int n = pick(1, per);
      std::vector<int64_t> mine(per);
      std::iota(mine.begin(), mine.end(), (int64_t)t * per);
      std::shuffle(mine.begin(), mine.end(), rng);
      op.gids.assign(mine.begin(), mine.begin() + n);
      std::shuffle(mine.begin(), mine.end(), rng);
      op.cids.assign(mine.begin(), mine.begin() + n);
      op.h2d = rng() & 1;
      op.sync = rng() & 1;
      op.use_ce = (rng() % 4) == 0;
      script[t].push_back(std::move(op));
    }
  std::vector<std::thread> pool;
  std::atomic<int> failures{0};
  const long waited_before = fkv_emulated_host_waited_copies();
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&, t] {
      hipStream_t st = nullptr;
      if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) {
        failures.fetch_add(1);
        return;
      }
      for (const Op &op : script[t]) {
        fkv_transfer_desc d{};
        d.backend = FKV_BACKEND_VLLM;
        d.num_layers_total = s.L;
        d.gpu_tensor_ptrs = ptrs.data();
        d.num_gpu_tensor_ptrs = s.L;
        d.device = -1;
        d.gpu_kv_stride = s.gpu_kv_stride();
        d.gpu_block_stride = s.gpu_block_stride();
        d.gpu_layer_stride = s.layer_bytes();
        d.cpu_ptr = host;
        d.cpu_kv_stride = s.cpu_kv_stride();
        d.cpu_layer_stride = s.cpu_layer_stride();
        d.cpu_block_stride = s.cpu_block_stride();
        d.chunk_size = s.chunk;
        d.num_layers = s.L;
        d.kv_dim = s.kv;
        d.num_blocks = (int32_t)op.gids.size();
        d.gpu_block_ids = op.gids.data();
        d.cpu_block_ids = op.cids.data();
        d.is_host_to_device = op.h2d;
        d.use_ce_transfer = op.use_ce;
        d.transfer_num_cta = 4;
        d.sync = op.sync;
        fkv_ce_config_default(&d.ce);
        d.ce.is_blockfirst = s.blockfirst;
        if (fkv_transfer_kv_blocks(&d, st) != FKV_OK) {
          fprintf(stderr, "thread %d: %s\n", t, fkv_last_error());
          failures.fetch_add(1);
        }
      }
      if (hipStreamSynchronize(st) != hipSuccess || hipStreamDestroy(st) != hipSuccess)
        failures.fetch_add(1);
    });
  for (auto &th : pool)
    th.join();
  REQUIRE(failures.load() == 0, "seed %llu: %d calls failed", (unsigned long long)seed, failures.load());
  // Plan memory, counters and staging were set up by the transfers before this case: with
  // requests in flight the library makes no copy that the host waits for (it would wait for
  // the device's queue, with locks held that every other request needs).
  REQUIRE(fkv_emulated_host_waited_copies() == waited_before,
          "seed %llu: %ld host-waited copies during concurrent requests", (unsigned long long)seed,
          fkv_emulated_host_waited_copies() - waited_before);
  for (int t = 0; t < threads; ++t)
    for (const Op &op : script[t])
      for (int l = 0; l < s.L; ++l)
        for (int k = 0; k < s.kv; ++k)
          for (size_t q = 0; q < op.gids.size(); ++q) {
            uint8_t *gm = model[l].data() + k * s.gpu_kv_stride() + op.gids[q] * s.chunk;
            uint8_t *hm = host_model.data() + op.cids[q] * s.cpu_block_stride() +
                          l * s.cpu_layer_stride() + k * s.cpu_kv_stride();
            if (op.h2d)
              std::memcpy(gm, hm, (size_t)s.chunk);
            else
              std::memcpy(hm, gm, (size_t)s.chunk);
          }
  { // a device-wide wait: the library's lane streams included
    void *probe = nullptr;
    REQUIRE(hipMalloc(&probe, 64) == hipSuccess && hipFree(probe) == hipSuccess, "drain");
  }
  for (int l = 0; l < s.L; ++l)
    REQUIRE(std::memcmp(dev[l], model[l].data(), (size_t)s.layer_bytes()) == 0,
            "seed %llu: layer %d differs after %d threads", (unsigned long long)seed, l, threads);
  REQUIRE(std::memcmp(host, host_model.data(), host_model.size()) == 0,
          "seed %llu: host pool differs after %d threads", (unsigned long long)seed, threads);
  for (uint8_t *d : dev)
    REQUIRE(hipFree(d) == hipSuccess, "free");
  REQUIRE(hipHostFree(host) == hipSuccess, "host free");
}

// The runtime runs out of something part-way: allocations, streams, events, copies, launches
// and event records are refused at seeded points during layerwise restores on every route.
// A refused call either is made up for (the kernel path needs no staging memory) or fails the
// restore; it never hangs, corrupts or leaks into the next restore, which must be whole.
void failure_case(uint64_t seed) {
  std::mt19937_64 rng(seed);
  auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); };
  Shape s{};
  s.ranks = pick(1, 2);
  s.L = pick(2, 10);
  s.kv = pick(1, 2);
  s.NG = pick(6, 24);
  s.NC = pick(6, 24);
  s.chunk = 16 * pick(1, 64);
  s.blockfirst = rng() & 1;
  uint8_t *host = nullptr;
  REQUIRE(hipHostMalloc((void **)&host, (size_t)s.host_bytes(), 0) == hipSuccess, "host pool");
  std::vector<std::vector<uint8_t *>> dev(s.ranks);
  std::vector<uint64_t> ptrs;
  for (int r = 0; r < s.ranks; ++r)
    for (int l = 0; l < s.L; ++l) {
      uint8_t *d = nullptr;
      REQUIRE(hipMalloc((void **)&d, (size_t)s.layer_bytes()) == hipSuccess, "engine tensor");
      fill(rng, d, (size_t)s.layer_bytes());
      dev[r].push_back(d);
      ptrs.push_back((uint64_t)(uintptr_t)d);
    }
  std::vector<int32_t> fds;
  for (int i = 0; i < s.ranks * s.L; ++i)
    fds.push_back(eventfd(0, EFD_NONBLOCK));
  std::vector<int64_t> kvs(s.ranks, s.gpu_kv_stride()), bs(s.ranks, s.gpu_block_stride()),
      ls(s.ranks, s.layer_bytes()), cs(s.ranks, s.chunk), devs(s.ranks, 0);
  fkv_layerwise_params p{};
  p.num_gpus = s.ranks;
  p.num_tensors_per_gpu = s.L;
  p.gpu_block_ptrs_flat = ptrs.data();
  p.cpu_blocks_ptr = host;
  p.num_layers = s.L;
  p.tp_size = s.ranks;
  p.gpu_kv_strides = kvs.data();
  p.gpu_block_strides = bs.data();
  p.gpu_layer_strides = ls.data();
  p.gpu_chunk_sizes = cs.data();
  p.gpu_device_ids = devs.data();
  p.layer_eventfds = fds.data();
  p.num_layer_eventfds = (int32_t)fds.size();
  fkv_ce_config_default(&p.ce);
  p.ce.is_blockfirst = s.blockfirst;
  fkv_layerwise *g = nullptr;
  REQUIRE(fkv_layerwise_create(&p, &g) == FKV_OK, "create");
  for (int rep = 0; rep < 6; ++rep) {
    const int route = pick(1, 3);
    std::vector<std::pair<std::string, int>> pol = {
        {"model_seed", 0}, {"gather_threads", 3}, {"gather_first_by_kernel", pick(0, 1)},
        {"kernel_alt_stream_kb", 4096}};
    if (route == 1) { pol.push_back({"staged_restore", 0}); pol.push_back({"staged_gather", 0}); }
    if (route == 2) { pol.push_back({"staged_restore", 2}); pol.push_back({"staged_gather", 0}); }
    if (route == 3) { pol.push_back({"staged_restore", 0}); pol.push_back({"staged_gather", 3}); }
    set_policy(pol);
    const int n = pick(1, std::min(s.NG, s.NC));
    std::vector<int64_t> gids(s.NG), cids(s.NC);
    std::iota(gids.begin(), gids.end(), 0);
    std::iota(cids.begin(), cids.end(), 0);
    std::shuffle(gids.begin(), gids.end(), rng);
    std::shuffle(cids.begin(), cids.end(), rng);
    gids.resize(n);
    cids.resize(n);
    const int gran = pick(1, 3), use_ce = (rng() % 4) == 0;
    const int notify = (rng() & 1) ? FKV_NOTIFY_POLLING : FKV_NOTIFY_HOSTFUNC;
    const bool inject = rep % 2 == 0;
    fill(rng, host, (size_t)s.host_bytes());
    if (inject)
      fkv_emulated_fail(pick(0, 7), pick(0, 12), pick(1, 3));
    if (rng() % 4 == 0) // may be refused part-way; the group keeps a stream per GPU either way
      (void)fkv_layerwise_set_compute_stream(g, pick(0, s.ranks - 1), nullptr, nullptr);
    const int rc = fkv_layerwise_transfer(g, gids.data(), cids.data(), n, s.cpu_block_stride(),
                                          s.cpu_kv_stride(), s.cpu_layer_stride(),
                                          s.cpu_block_stride(), 4, use_ce, s.L, gran, s.kv, 1, 0,
                                          "sharded", notify, 0);
    const int src = fkv_layerwise_synchronize(g);
    for (int c = 0; c < 8; ++c)
      fkv_emulated_fail(c, 0, 0);
    if (!inject)
      REQUIRE(rc == FKV_OK && src == FKV_OK, "seed %llu rep %d: a clean restore failed (route %d)",
              (unsigned long long)seed, rep, route);
    if (rc == FKV_OK && src == FKV_OK) {
      // whole: every rank has every block of every layer, and every layer was announced once
      for (int r = 0; r < s.ranks; ++r)
        for (int l = 0; l < s.L; ++l)
          for (int k = 0; k < s.kv; ++k)
            for (int q = 0; q < n; ++q)
              REQUIRE(std::memcmp(dev[r][l] + k * s.gpu_kv_stride() + gids[q] * s.chunk,
                                  host + cids[q] * s.cpu_block_stride() + l * s.cpu_layer_stride() +
                                      k * s.cpu_kv_stride(), (size_t)s.chunk) == 0,
                      "seed %llu rep %d: rank %d layer %d block %d differs after a restore that "
                      "reported success (route %d, injected %d)", (unsigned long long)seed, rep, r, l,
                      q, route, (int)inject);
      for (int fd : fds)
        REQUIRE(drain(fd) == 1, "seed %llu rep %d: a layer was not announced exactly once",
                (unsigned long long)seed, rep);
    } else {
      for (int fd : fds)
        REQUIRE(drain(fd) <= 1, "seed %llu rep %d: a layer was announced twice",
                (unsigned long long)seed, rep);
    }
  }
  fkv_layerwise_destroy(g);
  for (int fd : fds)
    close(fd);
  for (auto &rank : dev)
    for (uint8_t *d : rank)
      REQUIRE(hipFree(d) == hipSuccess, "free");
  REQUIRE(hipHostFree(host) == hipSuccess, "host free");
}

} // namespace

int main(int argc, char **argv) {
  const int restores = argc > 1 ? atoi(argv[1]) : 120, transfers = argc > 2 ? atoi(argv[2]) : 60;
  for (int i = 0; i < transfers; ++i)
    transfer_case(7000 + i);
  for (int i = 0; i < transfers; ++i)
    tp_case(8000 + i);
  for (int i = 0; i < transfers; ++i)
    concurrent_case(10000 + i);
  for (int i = 0; i < restores; ++i)
    failure_case(12000 + i);
  const long refused_calls = fkv_emulated_fail(-1, 0, 0);
  for (int i = 0; i < restores; ++i)
    layerwise_case(9000 + i);
  // four ranks that share their KV, rows gathered by host threads, asked for on the copy
  // engine: the launching thread serves four staging rings and eight copy streams
  Pinned four;
  four.ranks = 4, four.L = 5, four.kv = 1, four.NG = 12, four.NC = 12, four.chunk16 = 128;
  four.blockfirst = 1, four.mode = 0, four.pageable = 0, four.route = 3, four.use_ce = 1;
  for (int i = 0; i < restores / 2; ++i)
    layerwise_case(11000 + i, four);
  printf("ok: %d groups of layerwise restores, %d sets of transfers, %d thread groups and %d bursts "
         "of concurrent calls over the emulated runtime; %ld runtime calls refused on request\n",
         restores, transfers, transfers, transfers, refused_calls);
  int plan_slots = 0, plan_slots_out = 0;
  fkv::plan_pool_counts(&plan_slots, &plan_slots_out);
  REQUIRE(plan_slots_out == 0, "%d of %d plan slots were never given back", plan_slots_out, plan_slots);
  printf("plan pool: %d slots, all given back\n", plan_slots);
  if (fkv_emulated_workgroups_run())
    printf("kernels from their sources: %llu workgroups\n", fkv_emulated_workgroups_run());
  return 0;
}
