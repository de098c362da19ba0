// Two threads of a plain C++ program, one putting and one getting through the C
// ABI at the same time, each on a stream of its own: the rates the link gives
// both directions at once without Python in the way, and a check that the calls
// are safe from concurrent threads (every block is compared afterwards).
//   two_way_driver [seconds per phase, default 1.0] [blocks per transfer, default 94]
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
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

namespace {
// the vLLM shape of a Llama-3-8B cache: 32 layers of [2, N, 16*8*128 bf16]
constexpr int L = 32, KV = 2, N = 768, NH = 768;
constexpr int64_t CHUNK = 16 * 8 * 128 * 2;
constexpr int64_t GKS = N * CHUNK, GBS = CHUNK, GLS = KV * N * CHUNK;
constexpr int64_t CKS = CHUNK, CLS = KV * CHUNK, CBS = (int64_t)L * KV * CHUNK;

double now() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

struct Loop {
  std::vector<int64_t> gpu_ids, cpu_ids;
  int h2d = 0;
  hipStream_t stream = nullptr;
  double seconds = 1.0, rate = 0;
  int rc = FKV_OK;
  long calls = 0;
};

void run_loop(Loop *lp, const uint64_t *ptrs, void *host) {
  (void)hipSetDevice(0);
  fkv_transfer_desc d;
  memset(&d, 0, sizeof(d));
  d.backend = FKV_BACKEND_VLLM, d.num_layers_total = L;
  d.gpu_tensor_ptrs = ptrs, d.num_gpu_tensor_ptrs = L, d.device = -1;
  d.gpu_kv_stride = GKS, d.gpu_block_stride = GBS, d.gpu_layer_stride = GLS;
  d.cpu_ptr = host, d.cpu_kv_stride = CKS, d.cpu_layer_stride = CLS, d.cpu_block_stride = CBS;
  d.chunk_size = CHUNK, d.start_layer_id = 0, d.num_layers = L, d.kv_dim = KV;
  d.num_blocks = (int32_t)lp->gpu_ids.size();
  d.gpu_block_ids = lp->gpu_ids.data(), d.cpu_block_ids = lp->cpu_ids.data();
  d.is_host_to_device = lp->h2d, d.transfer_num_cta = 4, d.sync = 1;
  const double t0 = now();
  do { // once at least
    lp->rc = fkv_transfer_kv_blocks(&d, lp->stream);
    if (lp->rc != FKV_OK)
      return;
    ++lp->calls;
  } while (now() - t0 < lp->seconds);
  lp->rate = (double)lp->calls * d.num_blocks * L * KV * CHUNK / (now() - t0) / 1e9;
}
} // namespace

int main(int argc, char **argv) {
  const double seconds = argc > 1 ? atof(argv[1]) : 1.0;
  const int per = argc > 2 ? atoi(argv[2]) : 94;
  if (per < 1 || 3 * per > N || seconds <= 0) { // three disjoint sets of engine blocks
    fprintf(stderr, "usage: two_way_driver [seconds] [blocks per transfer, at most %d]\n", N / 3);
    return 2;
  }
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev < 1) {
    fprintf(stderr, "no GPU\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  std::vector<void *> dev(L);
  std::vector<uint64_t> ptrs(L);
  std::vector<uint8_t> fill(GLS);
  uint64_t x = 88172645463325252ull;
  for (int l = 0; l < L; ++l) {
    for (size_t i = 0; i < fill.size(); i += 8) {
      x ^= x << 13, x ^= x >> 7, x ^= x << 17;
      memcpy(&fill[i], &x, 8);
    }
    HIP_OK(hipMalloc(&dev[l], GLS));
    HIP_OK(hipMemcpy(dev[l], fill.data(), GLS, hipMemcpyHostToDevice));
    ptrs[l] = (uint64_t)(uintptr_t)dev[l];
  }
  void *host = nullptr;
  if (fkv_host_alloc((size_t)NH * CBS, &host) != FKV_OK) {
    fprintf(stderr, "host pool: %s\n", fkv_last_error());
    return 1;
  }
  memset(host, 0, (size_t)NH * CBS);

  // puts move engine blocks [0, per) to host blocks [0, per); gets move host blocks
  // [per, 2 per) to engine blocks [N - per, N); a first put fills the host blocks of the gets
  Loop put, get, prime;
  for (int i = 0; i < per; ++i) {
    put.gpu_ids.push_back((i * 7) % per), put.cpu_ids.push_back(i);
    get.cpu_ids.push_back(per + i), get.gpu_ids.push_back(N - 1 - i);
    prime.gpu_ids.push_back(per + i), prime.cpu_ids.push_back(per + i);
  }
  put.h2d = 0, get.h2d = 1, prime.h2d = 0;
  HIP_OK(hipStreamCreateWithFlags(&put.stream, hipStreamNonBlocking));
  // the get stream must not share a hardware queue with the put stream
  std::vector<hipStream_t> spare;
  for (int attempt = 0; attempt < 8; ++attempt) {
    HIP_OK(hipStreamCreateWithFlags(&get.stream, hipStreamNonBlocking));
    int32_t concurrent = 0;
    if (fkv_streams_run_concurrently(0, put.stream, get.stream, &concurrent) == FKV_OK && concurrent)
      break;
    spare.push_back(get.stream);
  }
  prime.stream = put.stream, prime.seconds = 0;
  run_loop(&prime, ptrs.data(), host);
  if (prime.rc != FKV_OK) {
    fprintf(stderr, "priming put: %s\n", fkv_last_error());
    return 1;
  }

  put.seconds = get.seconds = seconds;
  run_loop(&put, ptrs.data(), host);
  const double put_alone = put.rate;
  run_loop(&get, ptrs.data(), host);
  const double get_alone = get.rate;
  put.calls = get.calls = 0;
  std::thread a(run_loop, &put, ptrs.data(), host), b(run_loop, &get, ptrs.data(), host);
  a.join();
  b.join();
  if (put.rc != FKV_OK || get.rc != FKV_OK) {
    fprintf(stderr, "transfer failed: %d %d\n", put.rc, get.rc);
    return 1;
  }
  HIP_OK(hipDeviceSynchronize());

  // every block where it belongs
  std::vector<uint8_t> layer(GLS);
  for (int l = 0; l < L; ++l) {
    HIP_OK(hipMemcpy(layer.data(), dev[l], GLS, hipMemcpyDeviceToHost));
    for (int kv = 0; kv < KV; ++kv)
      for (int i = 0; i < per; ++i) {
        const uint8_t *h_put = (const uint8_t *)host + put.cpu_ids[i] * CBS + l * CLS + kv * CKS;
        const uint8_t *g_put = layer.data() + kv * GKS + put.gpu_ids[i] * GBS;
        const uint8_t *h_get = (const uint8_t *)host + get.cpu_ids[i] * CBS + l * CLS + kv * CKS;
        const uint8_t *g_get = layer.data() + kv * GKS + get.gpu_ids[i] * GBS;
        const uint8_t *g_src = layer.data() + kv * GKS + prime.gpu_ids[i] * GBS;
        if (memcmp(h_put, g_put, CHUNK) || memcmp(h_get, g_get, CHUNK) || memcmp(h_get, g_src, CHUNK)) {
          fprintf(stderr, "layer %d kv %d block %d differs\n", l, kv, i);
          return 1;
        }
      }
  }
  fkv_stats st;
  fkv_get_stats(&st);
  printf("ok: puts alone %.1f GB/s, gets alone %.1f GB/s, together puts %.1f + gets %.1f = %.1f GB/s "
         "(%ld + %ld calls of %d blocks, %llu confined launches, %llu ranges left to the safety net)\n",
         put_alone, get_alone, put.rate, get.rate, put.rate + get.rate, put.calls, get.calls, per,
         (unsigned long long)st.confined_launches, (unsigned long long)st.safety_net_ranges);
  return 0;
}
