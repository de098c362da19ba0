// The gather/scatter kernel by itself on the CPU device model, for sanitizer builds: seeded
// launches over the whole space of shapes the host side can ask for (every vector width,
// chunks of whole slices, with a short last slice, shorter than a slice (packed), fit for
// the deep unroll; one to 1024 (layer, kv) pairs; more block positions than one id tile
// holds; id lists or none; plain and nontemporal stores; lanes that move adjacent vectors;
// fixed shares, claimed ranges, launches confined to some XCDs with a dirty claim counter;
// one to four jobs in one launch), every byte of every destination against a plain model.
//
// Every table, id list and chunk region is an allocation of exactly the size the kernel may
// touch, the last chunk of a region ending where the allocation ends: an address one vector
// too far is a report of AddressSanitizer, not a lucky read.
#include "fkv_internal.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#define REQUIRE(cond, ...)                                                                          \
  do {                                                                                              \
    if (!(cond)) {                                                                                  \
      fprintf(stderr, "copy_kernel_model_driver: " __VA_ARGS__);                                    \
      fprintf(stderr, " [%s:%d]\n", __FILE__, __LINE__);                                            \
      exit(1);                                                                                      \
    }                                                                                               \
  } while (0)

extern "C" unsigned long long fkv_emulated_workgroups_run();

namespace {

template <typename T> T *device_copy(const std::vector<T> &v) {
  T *p = nullptr;
  REQUIRE(hipMalloc(reinterpret_cast<void **>(&p), std::max<size_t>(1, v.size() * sizeof(T))) == hipSuccess,
          "hipMalloc");
  if (!v.empty())
    REQUIRE(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) == hipSuccess, "upload");
  return p;
}

// One side of a job: `lk` regions of `blocks` chunks, `stride` apart, each region an
// allocation that ends with its last chunk.
struct Side {
  std::vector<uint8_t *> region;
  size_t region_bytes = 0;
  void make(std::mt19937_64 &rng, int lk, int blocks, int64_t stride, int64_t chunk, bool pinned) {
    region_bytes = (size_t)((blocks - 1) * stride + chunk);
    region.resize(lk);
    for (auto &r : region) {
      if (pinned)
        REQUIRE(hipHostMalloc(reinterpret_cast<void **>(&r), region_bytes, 0) == hipSuccess, "pinned");
      else
        REQUIRE(hipMalloc(reinterpret_cast<void **>(&r), region_bytes) == hipSuccess, "device");
      for (size_t i = 0; i < region_bytes; ++i)
        r[i] = (uint8_t)rng();
    }
  }
  void release(bool pinned) {
    for (uint8_t *r : region)
      REQUIRE((pinned ? hipHostFree(r) : hipFree(r)) == hipSuccess, "free");
  }
};

struct Job {
  fkv::CopyKernelArgs a{};
  Side src, dst;
  std::vector<std::vector<uint8_t>> want; // the destination regions as they must end up
  std::vector<void *> tables;
  bool dst_pinned = false;
};

int pick(std::mt19937_64 &rng, int lo, int hi) { return lo + (int)(rng() % (uint64_t)(hi - lo + 1)); }

// A job of vector width `vec` and store kind `nt`; shape chosen by `rng`.
void make_job(std::mt19937_64 &rng, int vec, bool nt, bool small, Job &j) {
  const int64_t slice = 64 * 8 * vec;
  int64_t chunk;
  switch (pick(rng, 0, small ? 3 : 5)) {
  case 0: chunk = vec * pick(rng, 1, 40); break;                                    // packed, tiny
  case 1: chunk = vec * pick(rng, 41, 511); break;                                  // packed
  case 2: chunk = slice * pick(rng, 1, 3); break;                                   // whole slices
  case 3: chunk = slice * pick(rng, 0, 2) + vec * pick(rng, 1, 511); break;         // short last slice
  case 4: chunk = (int64_t)64 * 16 * vec * pick(rng, 1, 2); break;                  // deep-unroll shape
  default: chunk = slice * pick(rng, 3, 6) + vec * pick(rng, 0, 64); break;
  }
  const int shape = pick(rng, 0, 24); // 0: many (layer, kv) pairs, 1: more positions than an id tile
  int lk = shape == 0 ? pick(rng, 200, 1024) : pick(rng, 1, 24);
  int n = shape == 1 ? pick(rng, 1025, 2300) : pick(rng, 1, 48);
  if (shape == 0)
    n = pick(rng, 1, 3), chunk = std::min<int64_t>(chunk, vec * 64);
  if (shape == 1)
    lk = pick(rng, 1, 2), chunk = vec * pick(rng, 1, 24);
  const int pool_src = n + pick(rng, 0, 7), pool_dst = n + pick(rng, 0, 7);
  const int64_t stride_src = chunk + vec * pick(rng, 0, 9), stride_dst = chunk + vec * pick(rng, 0, 9);
  j.dst_pinned = !nt;
  j.src.make(rng, lk, pool_src, stride_src, chunk, nt);
  j.dst.make(rng, lk, pool_dst, stride_dst, chunk, j.dst_pinned);
  std::vector<int64_t> ids_src(n), ids_dst(pool_dst);
  for (auto &v : ids_src)
    v = pick(rng, 0, pool_src - 1); // a source block may be read twice
  std::iota(ids_dst.begin(), ids_dst.end(), 0);
  std::shuffle(ids_dst.begin(), ids_dst.end(), rng);
  ids_dst.resize(n);
  const bool no_src_ids = rng() % 4 == 0, no_dst_ids = rng() % 4 == 0;
  if (no_src_ids)
    std::iota(ids_src.begin(), ids_src.end(), 0);
  if (no_dst_ids)
    std::iota(ids_dst.begin(), ids_dst.end(), 0);
  j.want.resize(lk);
  std::vector<uint64_t> base_src(lk), base_dst(lk);
  for (int i = 0; i < lk; ++i) {
    base_src[i] = (uint64_t)(uintptr_t)j.src.region[i];
    base_dst[i] = (uint64_t)(uintptr_t)j.dst.region[i];
    j.want[i].assign(j.dst.region[i], j.dst.region[i] + j.dst.region_bytes);
    for (int p = 0; p < n; ++p)
      memcpy(j.want[i].data() + ids_dst[p] * stride_dst, j.src.region[i] + ids_src[p] * stride_src,
             (size_t)chunk);
  }
  fkv::CopyKernelArgs &a = j.a;
  a.base_src = device_copy(base_src);
  a.base_dst = device_copy(base_dst);
  a.ids_src = no_src_ids ? nullptr : device_copy(ids_src);
  a.ids_dst = no_dst_ids ? nullptr : device_copy(ids_dst);
  j.tables = {(void *)a.base_src, (void *)a.base_dst, (void *)a.ids_src, (void *)a.ids_dst};
  a.stride_src = stride_src, a.stride_dst = stride_dst, a.chunk_bytes = chunk;
  a.num_blocks = n, a.lk = lk, a.vec = vec, a.nt_store = nt;
  a.unroll = std::vector<int>{0, fkv::kCopyUnroll, fkv::kCopyUnrollDeep}[pick(rng, 0, 2)];
  a.lane_runs = (int)(rng() & 1);
  a.packed_grid_pct = std::vector<int>{0, 50, 100, 250}[pick(rng, 0, 3)];
}

void check_and_release(Job &j, unsigned long long seed, int index) {
  for (size_t i = 0; i < j.want.size(); ++i)
    REQUIRE(memcmp(j.dst.region[i], j.want[i].data(), j.want[i].size()) == 0,
            "seed %llu job %d: destination region %zu differs (vec %d chunk %lld blocks %d lk %d packed %d)",
            seed, index, i, j.a.vec, (long long)j.a.chunk_bytes, j.a.num_blocks, j.a.lk, j.a.packed);
  j.src.release(j.a.nt_store != 0);
  j.dst.release(j.dst_pinned);
  for (void *t : j.tables)
    if (t)
      REQUIRE(hipFree(t) == hipSuccess, "free table");
}

// How the workgroups come by their work: counters (dirty ones too), masks, ranges.
uint64_t *share_out(std::mt19937_64 &rng, fkv::CopyKernelArgs &a) {
  uint64_t *claim = nullptr;
  if (rng() % 3 != 0) {
    std::vector<uint64_t> dirty = {rng() % 2 ? 0 : rng()};
    claim = device_copy(dirty);
    a.claim = claim;
    a.xcd_mask = std::vector<uint32_t>{0, 0x0fu, 0xf0u, 0x55u, 0x01u, 0x80u, 0xffu}[pick(rng, 0, 6)];
    a.xcd_present = rng() % 4 ? 0 : 0xffu;
    a.claims_per_wg = pick(rng, 0, 8);
    a.safety_net_wait_us = pick(rng, 1, 20);
  }
  return claim;
}

void single(unsigned long long seed, hipStream_t stream) {
  std::mt19937_64 rng(seed);
  const int vec = 1 << pick(rng, 0, 4);
  Job j;
  make_job(rng, vec, rng() & 1, false, j);
  uint64_t *claim = share_out(rng, j.a);
  const int threads = std::vector<int>{1, 64, 128, 256, 1024, 4096}[pick(rng, 0, 5)];
  REQUIRE(fkv::launch_copy_kernel(j.a, pick(rng, 1, 40), threads, stream) == FKV_OK, "seed %llu: %s",
          seed, fkv_last_error());
  REQUIRE(hipStreamSynchronize(stream) == hipSuccess, "synchronize");
  check_and_release(j, seed, 0);
  if (claim)
    REQUIRE(hipFree(claim) == hipSuccess, "free counter");
}

void several(unsigned long long seed, hipStream_t stream) {
  std::mt19937_64 rng(seed);
  const int vec = 1 << pick(rng, 0, 4), njobs = pick(rng, 1, fkv::kCopyMaxJobs);
  const bool nt = rng() & 1;
  std::vector<Job> jobs(njobs);
  std::vector<fkv::CopyKernelArgs> args;
  for (Job &j : jobs) {
    make_job(rng, vec, nt, true, j);
    args.push_back(j.a);
  }
  uint64_t *claim = share_out(rng, args[0]);
  REQUIRE(fkv::launch_copy_jobs(args.data(), njobs, pick(rng, 1, 24),
                                std::vector<int>{64, 256, 1024}[pick(rng, 0, 2)], stream) == FKV_OK,
          "seed %llu: %s", seed, fkv_last_error());
  REQUIRE(hipStreamSynchronize(stream) == hipSuccess, "synchronize");
  for (int k = 0; k < njobs; ++k)
    check_and_release(jobs[k], seed, k);
  if (claim)
    REQUIRE(hipFree(claim) == hipSuccess, "free counter");
}

} // namespace

int main(int argc, char **argv) {
  const int launches = argc > 1 ? atoi(argv[1]) : 300;
  REQUIRE(fkv_emulated_workgroups_run() == 0, "fresh process");
  hipStream_t stream = nullptr;
  REQUIRE(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) == hipSuccess, "stream");
  for (int i = 0; i < launches; ++i) {
    if (i % 4 == 3)
      several(90000 + i, stream);
    else
      single(50000 + i, stream);
  }
  REQUIRE(hipStreamDestroy(stream) == hipSuccess, "stream");
  REQUIRE(fkv_emulated_workgroups_run() > 0, "the kernels ran from their sources");
  printf("ok: %d launches of the gather/scatter kernel on the CPU device model, %llu workgroups, "
         "%llu ranges by the safety net\n", launches, fkv_emulated_workgroups_run(),
         (unsigned long long)fkv::safety_net_ranges_of_current_device());
  return 0;
}
