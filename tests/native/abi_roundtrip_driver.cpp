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
