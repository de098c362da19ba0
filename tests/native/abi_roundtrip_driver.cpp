// A consumer of libfkv_hip.so that knows nothing but include/fkv_transfer.h and
// the HIP runtime: no Python, no torch.  Moves blocks of a vLLM-shaped cache
// through every engine of the library and checks each byte against a plain
// host model.
#include <hip/hip_runtime.h>
#include <sys/eventfd.h>
#include <unistd.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "fkv_transfer.h"

#define HIP_OK(x)                                                                          \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_));    \
      return 1;                                                                            \
    }                                                                                      \
  } while (0)
#define FKV_OK_OR_DIE(x)                                                                   \
  do {                                                                                     \
    int rc_ = (x);                                                                         \
    if (rc_ != FKV_OK) {                                                                   \
      fprintf(stderr, "%s:%d %s -> %d: %s\n", __FILE__, __LINE__, #x, rc_, fkv_last_error()); \
      return 1;                                                                            \
    }                                                                                      \
  } while (0)

namespace {
constexpr int L = 6, KV = 2, N = 96, NH = 80;
constexpr int64_t CHUNK = 4096 + 512; // not a power of two
constexpr int64_t GKS = N * CHUNK, GBS = CHUNK, GLS = KV * N * CHUNK;           // per layer [kv, N, chunk]
constexpr int64_t CKS = CHUNK, CLS = KV * CHUNK, CBS = (int64_t)L * KV * CHUNK; // [NH, L, kv, chunk]

struct Model {
  std::vector<std::vector<uint8_t>> gpu; // L tensors
  std::vector<uint8_t> host;
  void put(const std::vector<int64_t> &g, const std::vector<int64_t> &c, bool h2d) {
    for (size_t i = 0; i < g.size(); ++i)
      for (int l = 0; l < L; ++l)
        for (int kv = 0; kv < KV; ++kv) {
          uint8_t *gp = gpu[l].data() + kv * GKS + g[i] * GBS;
          uint8_t *cp = host.data() + c[i] * CBS + l * CLS + kv * CKS;
          if (h2d)
            memcpy(gp, cp, CHUNK);
          else
            memcpy(cp, gp, CHUNK);
        }
  }
};

std::vector<int64_t> pick(std::mt19937_64 &rng, int pool, int n) {
  std::vector<int64_t> v(pool);
  std::iota(v.begin(), v.end(), 0);
  std::shuffle(v.begin(), v.end(), rng);
  v.resize(n);
  return v;
}
} // namespace

int main() {
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev < 1) {
    fprintf(stderr, "no GPU\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  std::mt19937_64 rng(11);
  Model m;
  m.gpu.assign(L, std::vector<uint8_t>(GLS));
  m.host.assign((size_t)NH * CBS, 0);
  std::vector<void *> dev(L);
  std::vector<uint64_t> ptrs(L);
  for (int l = 0; l < L; ++l) {
    for (auto &b : m.gpu[l])
      b = (uint8_t)rng();
    HIP_OK(hipMalloc(&dev[l], GLS));
    HIP_OK(hipMemcpy(dev[l], m.gpu[l].data(), GLS, hipMemcpyHostToDevice));
    ptrs[l] = (uint64_t)(uintptr_t)dev[l];
  }
  void *host = nullptr;
  FKV_OK_OR_DIE(fkv_host_alloc((size_t)NH * CBS, &host));
  memset(host, 0, (size_t)NH * CBS);
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  auto check = [&](const char *what) -> int {
    HIP_OK(hipDeviceSynchronize());
    if (memcmp(host, m.host.data(), m.host.size())) {
      fprintf(stderr, "%s: host pool differs\n", what);
      return 1;
    }
    std::vector<uint8_t> back(GLS);
    for (int l = 0; l < L; ++l) {
      HIP_OK(hipMemcpy(back.data(), dev[l], GLS, hipMemcpyDeviceToHost));
      if (back != m.gpu[l]) {
        fprintf(stderr, "%s: device layer %d differs\n", what, l);
        return 1;
      }
    }
    return 0;
  };

  int cases = 0, refused = 0;
  // ---- fkv_transfer_kv_blocks: kernel, copy engine (chosen and each forced strategy) ----
  struct Mode { int use_ce, force; const char *name; };
  const Mode modes[] = {{0, -1, "kernel"}, {1, -1, "ce"}, {2, -1, "auto"}, {1, 0, "ce0"},
                        {1, 1, "ce1"}, {1, 2, "ce2"}, {1, 3, "ce3"}, {1, 4, "ce4"}};
  for (const Mode &mode : modes)
    for (int pattern = 0; pattern < 3; ++pattern) {
      const int n = pattern == 0 ? 40 : pattern == 1 ? 1 : 17;
      std::vector<int64_t> g = pick(rng, N, n), c = pick(rng, NH, n);
      if (pattern == 0) { // runs of consecutive ids on both sides
        std::iota(g.begin(), g.end(), 8);
        std::iota(c.begin(), c.end(), 3);
      }
      fkv_transfer_desc d;
      memset(&d, 0, sizeof(d));
      d.backend = FKV_BACKEND_VLLM;
      d.num_layers_total = L;
      d.gpu_tensor_ptrs = ptrs.data();
      d.num_gpu_tensor_ptrs = L;
      d.device = -1;
      d.gpu_kv_stride = GKS, d.gpu_block_stride = GBS, d.gpu_layer_stride = GLS;
      d.cpu_ptr = host;
      d.cpu_kv_stride = CKS, d.cpu_layer_stride = CLS, d.cpu_block_stride = CBS;
      d.chunk_size = CHUNK;
      d.start_layer_id = 0, d.num_layers = L, d.kv_dim = KV, d.num_blocks = n;
      d.gpu_block_ids = g.data(), d.cpu_block_ids = c.data();
      d.use_ce_transfer = mode.use_ce;
      d.transfer_num_cta = 4;
      d.sync = 1;
      fkv_ce_config_default(&d.ce);
      d.ce.is_blockfirst = 1;
      d.ce.force_path = mode.force;
      d.ce.path_opt_enabled = 1;
      d.is_host_to_device = 0;
      if (mode.force >= 0) { // a forced strategy that does not fit the ids is refused, not run
        const int rc = fkv_transfer_kv_blocks(&d, stream);
        if (rc == FKV_ERR_INVALID_ARG && strstr(fkv_last_error(), "does not fit")) {
          ++refused;
          continue;
        }
        FKV_OK_OR_DIE(rc);
      } else {
        FKV_OK_OR_DIE(fkv_transfer_kv_blocks(&d, stream));
      }
      m.put(g, c, false);
      if (check(mode.name))
        return 1;
      std::vector<int64_t> g2 = pick(rng, N, n);
      d.gpu_block_ids = g2.data();
      d.is_host_to_device = 1;
      FKV_OK_OR_DIE(fkv_transfer_kv_blocks(&d, stream));
      m.put(g2, c, true);
      if (check(mode.name))
        return 1;
      ++cases;
    }

  // ---- fkv_transfer_kv_blocks_multi: the layers in three descriptors, one call ----
  for (int h2d = 0; h2d < 2; ++h2d) {
    std::vector<int64_t> g = pick(rng, N, 29), c = pick(rng, NH, 29);
    const int first[3] = {0, 2, 5}, count[3] = {2, 3, 1};
    fkv_transfer_desc ds[3];
    memset(ds, 0, sizeof(ds));
    for (int k = 0; k < 3; ++k) {
      fkv_transfer_desc &d = ds[k];
      d.backend = FKV_BACKEND_VLLM;
      d.num_layers_total = L;
      d.gpu_tensor_ptrs = ptrs.data();
      d.num_gpu_tensor_ptrs = L;
      d.device = -1;
      d.gpu_kv_stride = GKS, d.gpu_block_stride = GBS, d.gpu_layer_stride = GLS;
      d.cpu_ptr = host;
      d.cpu_kv_stride = CKS, d.cpu_layer_stride = CLS, d.cpu_block_stride = CBS;
      d.chunk_size = CHUNK;
      d.start_layer_id = first[k], d.num_layers = count[k], d.kv_dim = KV, d.num_blocks = 29;
      d.gpu_block_ids = g.data(), d.cpu_block_ids = c.data();
      d.transfer_num_cta = 4;
      d.sync = k == 2;
      d.is_host_to_device = h2d;
      fkv_ce_config_default(&d.ce);
      d.ce.is_blockfirst = 1;
    }
    FKV_OK_OR_DIE(fkv_transfer_kv_blocks_multi(ds, 3, stream));
    m.put(g, c, h2d != 0);
    if (check("multi"))
      return 1;
    ds[1].is_host_to_device = !h2d; // one call has one direction
    if (fkv_transfer_kv_blocks_multi(ds, 3, stream) != FKV_ERR_INVALID_ARG ||
        !strstr(fkv_last_error(), "direction")) {
      fprintf(stderr, "mixed directions were not refused\n");
      return 1;
    }
    ++cases;
  }

  // ---- TP group with one rank ----
  {
    const int64_t ks = GKS, bs = GBS, ls = GLS, cs = CHUNK, did = 0;
    fkv_tp_group_params p;
    memset(&p, 0, sizeof(p));
    p.num_gpus = 1, p.num_tensors_per_gpu = L;
    p.gpu_block_ptrs_flat = ptrs.data();
    p.cpu_blocks_ptr = host;
    p.num_layers = L;
    p.gpu_kv_strides = &ks, p.gpu_block_strides = &bs, p.gpu_layer_strides = &ls;
    p.gpu_chunk_sizes = &cs, p.gpu_device_ids = &did;
    fkv_ce_config_default(&p.ce);
    p.ce.is_blockfirst = 1;
    fkv_tp_group *grp = nullptr;
    FKV_OK_OR_DIE(fkv_tp_group_create(&p, &grp));
    for (int use_ce = 0; use_ce < 2; ++use_ce) {
      std::vector<int64_t> g = pick(rng, N, 23), c = pick(rng, NH, 23);
      FKV_OK_OR_DIE(fkv_tp_group_transfer(grp, g.data(), c.data(), 23, CKS, CLS, CBS, CBS, 4, 0,
                                          use_ce, 0, L, KV, 8, "sharded", 0));
      m.put(g, c, false);
      if (check("tp d2h"))
        return 1;
      std::vector<int64_t> g2 = pick(rng, N, 23);
      FKV_OK_OR_DIE(fkv_tp_group_transfer(grp, g2.data(), c.data(), 23, CKS, CLS, CBS, CBS, 4, 1,
                                          use_ce, 0, L, KV, 8, "sharded", 0));
      m.put(g2, c, true);
      if (check("tp h2d"))
        return 1;
      ++cases;
    }
    if (fkv_tp_group_transfer(grp, nullptr, nullptr, 3, CKS, CLS, CBS, CBS, 4, 1, 0, 0, L, KV, 8,
                              "sharded", 0) == FKV_OK) {
      fprintf(stderr, "null id arrays were accepted\n");
      return 1;
    }
    fkv_tp_group_destroy(grp);
  }

  // ---- layerwise restore, both notification modes, eventfds read back ----
  {
    const int64_t ks = GKS, bs = GBS, ls = GLS, cs = CHUNK, did = 0;
    std::vector<int32_t> fds(2 * L);
    for (auto &fd : fds)
      fd = eventfd(0, EFD_SEMAPHORE | EFD_NONBLOCK);
    fkv_layerwise_params p;
    memset(&p, 0, sizeof(p));
    p.num_gpus = 1, p.num_tensors_per_gpu = L;
    p.gpu_block_ptrs_flat = ptrs.data();
    p.cpu_blocks_ptr = host;
    p.num_layers = L, p.tp_size = 1;
    p.gpu_kv_strides = &ks, p.gpu_block_strides = &bs, p.gpu_layer_strides = &ls;
    p.gpu_chunk_sizes = &cs, p.gpu_device_ids = &did;
    p.layer_eventfds = fds.data(), p.num_layer_eventfds = (int32_t)fds.size();
    fkv_ce_config_default(&p.ce);
    p.ce.is_blockfirst = 1;
    fkv_layerwise *lw = nullptr;
    FKV_OK_OR_DIE(fkv_layerwise_create(&p, &lw));
    for (int notify = 0; notify < 2; ++notify)
      for (int use_ce = 0; use_ce < 2; ++use_ce) {
        std::vector<int64_t> g = pick(rng, N, 31), c = pick(rng, NH, 31);
        const int gran = 1 + (notify + use_ce) % 3;
        FKV_OK_OR_DIE(fkv_layerwise_transfer(lw, g.data(), c.data(), 31, CBS, CKS, CLS, CBS, 4,
                                             use_ce, L, gran, KV, 8, notify, "sharded", notify, 0));
        FKV_OK_OR_DIE(fkv_layerwise_synchronize(lw));
        m.put(g, c, true);
        if (check("layerwise"))
          return 1;
        for (int l = 0; l < L; ++l) { // one unit per layer on the chosen counter set
          uint64_t v = 0;
          if (read(fds[notify * L + l], &v, 8) != 8 || v != 1) {
            fprintf(stderr, "layer %d was not announced\n", l);
            return 1;
          }
        }
        ++cases;
      }
    // the same restore on every route the library has, forced through the launch policy:
    // kernel, one copy-engine command per run of host blocks, rows gathered by host threads
    // (batches launched one by one from the library's own thread), the latter also with
    // the cost model re-based on this device first
    fkv_launch_policy saved, pol;
    FKV_OK_OR_DIE(fkv_launch_policy_seed(-1));
    FKV_OK_OR_DIE(fkv_launch_policy_get(-1, &saved));
#ifndef FKV_EMULATED_RUNTIME // an emulated link has no rate worth re-basing on
    if (!saved.model_seeded || saved.model_link_mbps < 1000 || saved.staged_copy_overhead_us < 1) {
      fprintf(stderr, "launch policy: the cost model was not re-based on the device\n");
      return 1;
    }
#endif
    const int routes[3][2] = {{0, 0}, {2, 0}, {0, 2}}; // staged_restore, staged_gather
    for (int route = 0; route < 3; ++route)
      for (int notify = 0; notify < 2; ++notify) {
        pol = saved;
        pol.staged_restore = routes[route][0], pol.staged_gather = routes[route][1];
        pol.gather_threads = 3, pol.gather_ring = 2, pol.gather_first_by_kernel = notify;
        FKV_OK_OR_DIE(fkv_launch_policy_set(-1, &pol));
        fkv_stats before, after;
        fkv_get_stats(&before);
        std::vector<int64_t> g = pick(rng, N, 29), c = pick(rng, NH, 29);
        std::vector<int64_t> g_arg = g, c_arg = c;
        FKV_OK_OR_DIE(fkv_layerwise_transfer(lw, g_arg.data(), c_arg.data(), 29, CBS, CKS, CLS, CBS, 4,
                                             0, L, 1, KV, 8, notify, "sharded", notify, 0));
        // the lists belong to the caller again as soon as the call returns
        std::fill(g_arg.begin(), g_arg.end(), 0);
        std::fill(c_arg.begin(), c_arg.end(), 0);
        FKV_OK_OR_DIE(fkv_layerwise_synchronize(lw));
        fkv_get_stats(&after);
        m.put(g, c, true);
        if (check("layerwise restore, forced route"))
          return 1;
        const uint64_t staged = after.staged_batches - before.staged_batches;
        const uint64_t gathered = after.gathered_batches - before.gathered_batches;
        const uint64_t want_staged = route == 0 ? 0 : route == 2 && notify ? L - 1 : L;
        const uint64_t want_gathered = route == 2 ? want_staged : 0;
        if (staged != want_staged || gathered != want_gathered) {
          fprintf(stderr, "route %d: %llu staged and %llu gathered batches, expected %llu and %llu\n",
                  route, (unsigned long long)staged, (unsigned long long)gathered,
                  (unsigned long long)want_staged, (unsigned long long)want_gathered);
          return 1;
        }
        for (int l = 0; l < L; ++l) {
          uint64_t v = 0;
          if (read(fds[notify * L + l], &v, 8) != 8 || v != 1) {
            fprintf(stderr, "route %d: layer %d was not announced\n", route, l);
            return 1;
          }
        }
      }
    FKV_OK_OR_DIE(fkv_launch_policy_reset(-1));
    ++cases;
    // an engine in the same process: it names the stream of its forward pass once, then gates
    // every layer's work on that stream with fkv_layerwise_wait_layer
    {
      hipStream_t forward = nullptr;
      HIP_OK(hipStreamCreateWithFlags(&forward, hipStreamNonBlocking));
      int32_t sharing = -1;
      double round_trip_us = -1;
      FKV_OK_OR_DIE(fkv_layerwise_set_compute_stream(lw, 0, forward, &sharing));
      FKV_OK_OR_DIE(fkv_streams_hand_over_us(-1, forward, stream, &round_trip_us));
      if (sharing != 0 || round_trip_us <= 0 ||
          fkv_layerwise_set_compute_stream(lw, 1, forward, nullptr) == FKV_OK ||
          fkv_layerwise_set_compute_stream(nullptr, 0, forward, nullptr) == FKV_OK) {
        fprintf(stderr, "set_compute_stream: %d streams share the queue, round trip %.1f us\n", sharing,
                round_trip_us);
        return 1;
      }
      std::vector<int64_t> g = pick(rng, N, 27), c = pick(rng, NH, 27);
      FKV_OK_OR_DIE(fkv_layerwise_transfer(lw, g.data(), c.data(), 27, CBS, CKS, CLS, CBS, 4, 0, L, 1,
                                           KV, 8, 0, "sharded", 0, 0));
      std::vector<std::vector<uint8_t>> seen(L, std::vector<uint8_t>((size_t)KV * GKS));
      for (int l = 0; l < L; ++l) { // layer l as the forward stream sees it once it may go on
        FKV_OK_OR_DIE(fkv_layerwise_wait_layer(lw, 0, l, forward));
        HIP_OK(hipMemcpyAsync(seen[l].data(), dev[l], seen[l].size(), hipMemcpyDeviceToHost, forward));
      }
      HIP_OK(hipStreamSynchronize(forward));
      FKV_OK_OR_DIE(fkv_layerwise_synchronize(lw));
      m.put(g, c, true);
      for (int l = 0; l < L; ++l)
        if (memcmp(seen[l].data(), m.gpu[l].data(), seen[l].size()) != 0) {
          fprintf(stderr, "layer %d was not whole when the forward stream went on\n", l);
          return 1;
        }
      if (check("layerwise restore next to a named forward stream"))
        return 1;
      for (int l = 0; l < L; ++l) {
        uint64_t v = 0;
        if (read(fds[l], &v, 8) != 8 || v != 1) {
          fprintf(stderr, "named forward stream: layer %d was not announced\n", l);
          return 1;
        }
      }
      HIP_OK(hipStreamDestroy(forward));
      ++cases;
    }
    fkv_layerwise_destroy(lw);
    for (int fd : fds)
      close(fd);
  }

  // ---- multi-group restore with a uniform sliding-window sidecar ----
  {
    constexpr int OL = 4, NB = 24, NHB = 20, NS = 10, NHS = 12; // original layers, pool sizes
    constexpr int64_t C0 = 512, C1 = 256, CS = 1024;           // chunk of main, indexer, sidecar
    constexpr int64_t BLK = 4 * C0 + 3 * C1, OFF1 = 4 * C0;    // byte-flat host block
    const int group_layers[2] = {4, 3};
    const int64_t group_chunk[2] = {C0, C1};
    std::vector<std::vector<uint8_t>> gmodel[2];
    std::vector<void *> gdev[2];
    std::vector<uint64_t> gptrs[2];
    for (int g = 0; g < 2; ++g)
      for (int l = 0; l < group_layers[g]; ++l) {
        gmodel[g].emplace_back((size_t)NB * group_chunk[g], 0);
        void *p = nullptr;
        HIP_OK(hipMalloc(&p, NB * group_chunk[g]));
        HIP_OK(hipMemset(p, 0, NB * group_chunk[g]));
        gdev[g].push_back(p);
        gptrs[g].push_back((uint64_t)(uintptr_t)p);
      }
    std::vector<std::vector<uint8_t>> smodel(OL, std::vector<uint8_t>((size_t)NS * CS, 0));
    std::vector<void *> sdev(OL);
    std::vector<uint64_t> sptrs(OL);
    for (int l = 0; l < OL; ++l) {
      HIP_OK(hipMalloc(&sdev[l], NS * CS));
      HIP_OK(hipMemset(sdev[l], 0, NS * CS));
      sptrs[l] = (uint64_t)(uintptr_t)sdev[l];
    }
    void *mhost = nullptr, *shost = nullptr;
    FKV_OK_OR_DIE(fkv_host_alloc((size_t)NHB * BLK, &mhost));
    FKV_OK_OR_DIE(fkv_host_alloc((size_t)OL * NHS * CS, &shost)); // [layer, 1, block, chunk]
    uint8_t *mh = static_cast<uint8_t *>(mhost), *sh = static_cast<uint8_t *>(shost);
    for (size_t i = 0; i < (size_t)NHB * BLK; ++i)
      mh[i] = (uint8_t)rng();
    for (size_t i = 0; i < (size_t)OL * NHS * CS; ++i)
      sh[i] = (uint8_t)rng();

    fkv_layer_group groups[2], swa;
    int64_t kvs[2], bls[2], lys[2], chs[2];
    for (int g = 0; g < 2; ++g) {
      memset(&groups[g], 0, sizeof(groups[g]));
      kvs[g] = NB * group_chunk[g], bls[g] = group_chunk[g], lys[g] = NB * group_chunk[g];
      chs[g] = group_chunk[g];
      groups[g].num_layers = group_layers[g];
      groups[g].num_tensors_per_gpu = group_layers[g];
      groups[g].gpu_block_ptrs_flat = gptrs[g].data();
      groups[g].cpu_offset_bytes = g ? OFF1 : 0;
      groups[g].h2d_cpu_kv_stride = group_chunk[g];
      groups[g].h2d_cpu_layer_stride = group_chunk[g];
      groups[g].cpu_block_stride = BLK;
      groups[g].cpu_tp_stride = BLK;
      groups[g].gpu_kv_strides = &kvs[g], groups[g].gpu_block_strides = &bls[g];
      groups[g].gpu_layer_strides = &lys[g], groups[g].gpu_chunk_sizes = &chs[g];
    }
    const int32_t member_offsets[OL + 1] = {0, 1, 3, 5, 7};
    const fkv_layer_member members[7] = {{0, 0}, {0, 1}, {1, 0}, {0, 2}, {1, 1}, {0, 3}, {1, 2}};
    const int64_t did = 0;
    std::vector<int32_t> fds(OL);
    for (auto &fd : fds)
      fd = eventfd(0, EFD_SEMAPHORE | EFD_NONBLOCK);
    fkv_layerwise_mg_params p;
    memset(&p, 0, sizeof(p));
    p.num_gpus = 1, p.num_original_layers = OL, p.tp_size = 1, p.num_groups = 2;
    p.groups = groups, p.member_offsets = member_offsets, p.members = members;
    p.cpu_blocks_ptr = mhost, p.gpu_device_ids = &did;
    p.layer_eventfds = fds.data(), p.num_layer_eventfds = OL;
    fkv_ce_config_default(&p.ce);
    p.ce.is_blockfirst = 1;
    fkv_layerwise *lw = nullptr;
    FKV_OK_OR_DIE(fkv_layerwise_create_multi_group(&p, &lw));
    const int64_t sks = NS * CS, sbs = CS, sls = NS * CS, scs = CS;
    memset(&swa, 0, sizeof(swa));
    swa.num_layers = OL, swa.num_tensors_per_gpu = OL, swa.gpu_block_ptrs_flat = sptrs.data();
    swa.gpu_kv_strides = &sks, swa.gpu_block_strides = &sbs, swa.gpu_layer_strides = &sls;
    swa.gpu_chunk_sizes = &scs;
    FKV_OK_OR_DIE(fkv_layerwise_init_swa(lw, &swa, shost));
    for (int round = 0; round < 4; ++round) {
      const int n = 9, ns = 4;
      std::vector<int64_t> g = pick(rng, NB, n), c = pick(rng, NHB, n);
      std::vector<int64_t> sg = pick(rng, NS, ns), sc = pick(rng, NHS, ns);
      fkv_layerwise_call call;
      memset(&call, 0, sizeof(call));
      call.gpu_block_ids = g.data(), call.cpu_block_ids = c.data(), call.num_blocks = n;
      call.multi_group = 1;
      call.transfer_cta_num = 4, call.use_ce_transfer = round & 1, call.kv_dim = 1;
      call.num_kv_heads = 1, call.counter_id = 0, call.notify_mode = round >> 1;
      call.kv_shared_across_ranks_mode = "sharded";
      call.swa_num_blocks = ns, call.swa_gpu_block_ids = sg.data(), call.swa_cpu_block_ids = sc.data();
      call.swa_h2d_cpu_kv_stride = NHS * CS, call.swa_h2d_cpu_layer_stride = NHS * CS;
      call.swa_cpu_block_stride = CS;
      FKV_OK_OR_DIE(fkv_layerwise_transfer_call(lw, &call));
      FKV_OK_OR_DIE(fkv_layerwise_synchronize(lw));
      for (int i = 0; i < n; ++i)
        for (int gi = 0; gi < 2; ++gi)
          for (int l = 0; l < group_layers[gi]; ++l)
            memcpy(gmodel[gi][l].data() + g[i] * group_chunk[gi],
                   mh + c[i] * BLK + (gi ? OFF1 : 0) + l * group_chunk[gi], group_chunk[gi]);
      for (int i = 0; i < ns; ++i)
        for (int l = 0; l < OL; ++l)
          memcpy(smodel[l].data() + sg[i] * CS, sh + (size_t)l * NHS * CS + sc[i] * CS, CS);
      HIP_OK(hipDeviceSynchronize());
      std::vector<uint8_t> back;
      for (int gi = 0; gi < 2; ++gi)
        for (int l = 0; l < group_layers[gi]; ++l) {
          back.resize(gmodel[gi][l].size());
          HIP_OK(hipMemcpy(back.data(), gdev[gi][l], back.size(), hipMemcpyDeviceToHost));
          if (back != gmodel[gi][l]) {
            fprintf(stderr, "multi-group: group %d layer %d differs\n", gi, l);
            return 1;
          }
        }
      for (int l = 0; l < OL; ++l) {
        back.resize(smodel[l].size());
        HIP_OK(hipMemcpy(back.data(), sdev[l], back.size(), hipMemcpyDeviceToHost));
        if (back != smodel[l]) {
          fprintf(stderr, "multi-group: sidecar layer %d differs\n", l);
          return 1;
        }
        uint64_t v = 0;
        if (read(fds[l], &v, 8) != 8 || v != 1) {
          fprintf(stderr, "multi-group: original layer %d was not announced once\n", l);
          return 1;
        }
      }
      ++cases;
    }
    fkv_layerwise_destroy(lw);
    for (int fd : fds)
      close(fd);
    for (int g = 0; g < 2; ++g)
      for (void *q : gdev[g])
        HIP_OK(hipFree(q));
    for (void *q : sdev)
      HIP_OK(hipFree(q));
    FKV_OK_OR_DIE(fkv_host_free(mhost));
    FKV_OK_OR_DIE(fkv_host_free(shost));
  }

  // ---- engine blocks <-> dense device buffer ----
  {
    const int n = 29;
    void *buf = nullptr;
    HIP_OK(hipMalloc(&buf, (size_t)n * CBS));
    std::vector<int64_t> g = pick(rng, N, n);
    fkv_layout_transform_desc t;
    memset(&t, 0, sizeof(t));
    t.backend = FKV_BACKEND_VLLM, t.num_layers_total = L;
    t.gpu_tensor_ptrs = ptrs.data(), t.num_gpu_tensor_ptrs = L, t.device = -1;
    t.gpu_kv_stride = GKS, t.gpu_block_stride = GBS, t.gpu_layer_stride = GLS;
    t.buffer_ptr = buf;
    t.buffer_layer_stride = CLS, t.buffer_kv_stride = CKS, t.buffer_block_stride = CBS;
    t.chunk_size = CHUNK, t.num_layers = L, t.kv_dim = KV, t.num_blocks = n;
    t.gpu_block_ids = g.data();
    t.sync = 1;
    FKV_OK_OR_DIE(fkv_layout_transform(&t, stream));
    std::vector<uint8_t> got((size_t)n * CBS), want((size_t)n * CBS);
    HIP_OK(hipMemcpy(got.data(), buf, got.size(), hipMemcpyDeviceToHost));
    for (int i = 0; i < n; ++i)
      for (int l = 0; l < L; ++l)
        for (int kv = 0; kv < KV; ++kv)
          memcpy(want.data() + i * CBS + l * CLS + kv * CKS, m.gpu[l].data() + kv * GKS + g[i] * GBS,
                 CHUNK);
    if (got != want) {
      fprintf(stderr, "layout transform differs\n");
      return 1;
    }
    HIP_OK(hipFree(buf));
    ++cases;
  }

// the next two sections are about the kernels themselves: not with stand-ins for them
#if !defined(FKV_EMULATED_RUNTIME) || defined(FKV_KERNELS_FROM_SOURCE)
  // ---- launch policy: every way a launch shares out its work, and the entry point that
  //      allocates nothing, on the same descriptor ----
  {
    fkv_launch_policy saved, p;
    FKV_OK_OR_DIE(fkv_launch_policy_get(-1, &saved));
    if (saved.xcd_count < 1 || (saved.d2h_busy_mask & ~saved.xcd_present_mask) ||
        (saved.h2d_busy_mask & ~saved.xcd_present_mask)) {
      fprintf(stderr, "launch policy: masks beyond the device's XCDs\n");
      return 1;
    }
    const int arbiters[] = {0, 2, 3};
    for (int pass = 0; pass < 4; ++pass) {
      p = saved;
      if (pass < 3)
        p.arbiter = arbiters[pass], p.safety_net_wait_us = 5;
      FKV_OK_OR_DIE(fkv_launch_policy_set(-1, &p));
      const int n = 33;
      std::vector<int64_t> g = pick(rng, N, n), c = pick(rng, NH, n);
      fkv_transfer_desc d;
      memset(&d, 0, sizeof(d));
      d.backend = FKV_BACKEND_VLLM;
      d.num_layers_total = L;
      d.gpu_tensor_ptrs = ptrs.data();
      d.num_gpu_tensor_ptrs = L;
      d.device = -1;
      d.gpu_kv_stride = GKS, d.gpu_block_stride = GBS, d.gpu_layer_stride = GLS;
      d.cpu_ptr = host;
      d.cpu_kv_stride = CKS, d.cpu_layer_stride = CLS, d.cpu_block_stride = CBS;
      d.chunk_size = CHUNK;
      d.start_layer_id = 0, d.num_layers = L, d.kv_dim = KV, d.num_blocks = n;
      d.gpu_block_ids = g.data(), d.cpu_block_ids = c.data();
      d.transfer_num_cta = 4;
      d.sync = 1;
      fkv_ce_config_default(&d.ce);
      for (int h2d = 0; h2d < 2; ++h2d) {
        d.is_host_to_device = h2d;
        // the last pass goes through the entry point that allocates nothing
        FKV_OK_OR_DIE(pass == 3 ? fkv_transfer_kv_blocks_noalloc(&d, stream)
                                : fkv_transfer_kv_blocks(&d, stream));
        m.put(g, c, h2d != 0);
        if (check(pass == 3 ? "no-alloc entry point" : "forced launch policy"))
          return 1;
      }
      if (pass == 3) {
        d.use_ce_transfer = 1;
        if (fkv_transfer_kv_blocks_noalloc(&d, stream) != FKV_ERR_UNSUPPORTED) {
          fprintf(stderr, "no-alloc entry point accepted the copy-engine path\n");
          return 1;
        }
      }
    }
    FKV_OK_OR_DIE(fkv_launch_policy_reset(-1));
    ++cases;
  }

  // ---- compressed staging: address table, payloads of different sizes out and back ----
  {
    const int n = 9, total = L * KV * n, first = 5, bsz = total - first;
    const int64_t stride = CHUNK + 64;
    std::vector<int64_t> g = pick(rng, N, n), c = pick(rng, NH, n);
    void **d_ptrs = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_ptrs), sizeof(void *) * bsz));
    fkv_chunk_ptrs_desc cp;
    memset(&cp, 0, sizeof(cp));
    cp.out_ptrs = d_ptrs;
    cp.backend = FKV_BACKEND_VLLM;
    cp.num_layers_total = L;
    cp.gpu_tensor_ptrs = ptrs.data();
    cp.num_gpu_tensor_ptrs = L;
    cp.device = -1;
    cp.gpu_kv_stride = GKS, cp.gpu_block_stride = GBS, cp.gpu_layer_stride = GLS;
    cp.gpu_block_ids = g.data();
    cp.start_layer_id = 0, cp.kv_dim = KV, cp.num_blocks = n, cp.batch_start = first, cp.bsz = bsz;
    cp.sync = 1;
    FKV_OK_OR_DIE(fkv_build_gpu_chunk_ptrs(&cp, stream));
    std::vector<void *> got_ptrs(bsz);
    HIP_OK(hipMemcpy(got_ptrs.data(), d_ptrs, sizeof(void *) * bsz, hipMemcpyDeviceToHost));
    for (int i = 0; i < bsz; ++i) {
      const int gi = first + i, l = gi / (KV * n), kv = (gi % (KV * n)) / n, b = gi % n;
      if (got_ptrs[i] != static_cast<uint8_t *>(dev[l]) + kv * GKS + g[b] * GBS) {
        fprintf(stderr, "chunk pointer %d differs\n", i);
        return 1;
      }
    }
    // payloads: the first `sz` bytes of every chunk the table names, written to the host
    // cache with their sizes, then read back into scrubbed staging
    uint8_t *d_stage = nullptr;
    uint64_t *d_sizes = nullptr;
    int32_t *d_over = nullptr;
    void *table_v = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_stage), (size_t)bsz * stride));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_sizes), sizeof(uint64_t) * bsz));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_over), sizeof(int32_t)));
    HIP_OK(hipMemset(d_over, 0, sizeof(int32_t)));
    FKV_OK_OR_DIE(fkv_host_alloc(sizeof(uint32_t) * NH * L * KV, &table_v));
    uint32_t *table = static_cast<uint32_t *>(table_v);
    memset(table, 0xff, sizeof(uint32_t) * NH * L * KV);
    std::vector<uint8_t> stage((size_t)bsz * stride);
    std::vector<uint64_t> sizes(bsz);
    for (int i = 0; i < bsz; ++i) {
      const int gi = first + i, l = gi / (KV * n), kv = (gi % (KV * n)) / n, b = gi % n;
      sizes[i] = i == 3 ? (uint64_t)CHUNK + 1 : (uint64_t)(rng() % (CHUNK + 1)); // one does not fit
      memcpy(stage.data() + (size_t)i * stride, m.gpu[l].data() + kv * GKS + g[b] * GBS,
             (size_t)std::min<uint64_t>(sizes[i], CHUNK));
    }
    HIP_OK(hipMemcpy(d_stage, stage.data(), stage.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_sizes, sizes.data(), sizeof(uint64_t) * bsz, hipMemcpyHostToDevice));
    fkv_staging_transfer_desc sd;
    memset(&sd, 0, sizeof(sd));
    sd.staging = d_stage, sd.staging_stride = stride, sd.comp_sizes = d_sizes;
    sd.cpu_ptr = host, sd.chunk_capacity = CHUNK, sd.overflow = d_over;
    sd.cpu_kv_stride = CKS, sd.cpu_layer_stride = CLS, sd.cpu_block_stride = CBS;
    sd.cpu_block_ids = c.data();
    sd.size_table = table, sd.size_table_block_stride = L * KV, sd.size_table_layer_stride = KV;
    sd.start_layer_id = 0, sd.kv_dim = KV, sd.num_blocks = n, sd.batch_start = first, sd.bsz = bsz;
    sd.is_write_cpu = 1, sd.device = -1, sd.sync = 1;
    FKV_OK_OR_DIE(fkv_staging_transfer(&sd, stream));
    int32_t over = 0;
    HIP_OK(hipMemcpy(&over, d_over, sizeof(over), hipMemcpyDeviceToHost));
    for (int i = 0; i < bsz; ++i) {
      const int gi = first + i, l = gi / (KV * n), kv = (gi % (KV * n)) / n, b = gi % n;
      const uint32_t want_sz = sizes[i] > (uint64_t)CHUNK ? 0 : (uint32_t)sizes[i];
      if (table[c[b] * L * KV + l * KV + kv] != want_sz) {
        fprintf(stderr, "size table entry of chunk %d differs\n", i);
        return 1;
      }
      if (sizes[i] <= (uint64_t)CHUNK)
        memcpy(m.host.data() + c[b] * CBS + l * CLS + kv * CKS, stage.data() + (size_t)i * stride,
               (size_t)sizes[i]);
    }
    if (over != 1 || check("staging transfer to the host"))
      return 1;
    HIP_OK(hipMemset(d_stage, 0xEE, stage.size()));
    HIP_OK(hipMemset(d_sizes, 0, sizeof(uint64_t) * bsz));
    sd.is_write_cpu = 0;
    FKV_OK_OR_DIE(fkv_staging_transfer(&sd, stream));
    std::vector<uint8_t> back(stage.size());
    std::vector<uint64_t> back_sizes(bsz);
    HIP_OK(hipMemcpy(back.data(), d_stage, back.size(), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(back_sizes.data(), d_sizes, sizeof(uint64_t) * bsz, hipMemcpyDeviceToHost));
    for (int i = 0; i < bsz; ++i) {
      const uint64_t want_sz = sizes[i] > (uint64_t)CHUNK ? 0 : sizes[i];
      if (back_sizes[i] != want_sz ||
          memcmp(back.data() + (size_t)i * stride, stage.data() + (size_t)i * stride, (size_t)want_sz) ||
          (want_sz < (uint64_t)stride && back[(size_t)i * stride + want_sz] != 0xEE)) {
        fprintf(stderr, "staging transfer from the host: payload %d differs\n", i);
        return 1;
      }
    }
    HIP_OK(hipFree(d_ptrs));
    HIP_OK(hipFree(d_stage));
    HIP_OK(hipFree(d_sizes));
    HIP_OK(hipFree(d_over));
    FKV_OK_OR_DIE(fkv_host_free(table_v));
    ++cases;
  }
#endif

  // ---- the board processes share: one's own postings never count as "elsewhere" ----
  {
    int32_t busy = 7;
    FKV_OK_OR_DIE(fkv_link_activity_post(-1, 1, 50000));
    FKV_OK_OR_DIE(fkv_link_activity_elsewhere(-1, 1, 20, &busy));
    if (busy != 0 || fkv_link_activity_post(-1, 1, -5) == FKV_OK ||
        fkv_link_activity_elsewhere(-1, 1, 20, nullptr) == FKV_OK) {
      fprintf(stderr, "link activity board: busy=%d\n", busy);
      return 1;
    }
    ++cases;
  }

  fkv_stats st;
  fkv_get_stats(&st);
  HIP_OK(hipStreamDestroy(stream));
  FKV_OK_OR_DIE(fkv_host_free(host));
  for (void *p : dev)
    HIP_OK(hipFree(p));
  printf("ok: %d cases through the C ABI (%d forced strategies refused), %llu calls, "
         "%llu kernel launches, %llu DMA copies\n",
         cases, refused, (unsigned long long)st.calls, (unsigned long long)st.kernel_launches,
         (unsigned long long)st.dma_copies);
  return 0;
}
