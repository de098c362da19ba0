// What a stream pays between two host->GPU copy kernels while another stream
// writes to host memory: the measurement behind the library's choice of XCDs for
// the two directions and of its event flags.  Knows nothing of the library.
//
// A "writer" kernel streams device memory to pinned host memory from the XCDs of
// --writer-mask for the whole run; on a second stream twelve "reader" kernels of
// about 2 ms each copy pinned host memory to the device from the XCDs of
// --reader-mask, with something between each two of them:
//   --between none            nothing (back to back)
//   --between empty           an empty kernel
//   --between event-default   hipEventRecord of an event with default flags
//   --between event-nofence   hipEventRecord of an event with hipEventDisableSystemFence
// Prints the readers' rate inside and across their kernels, the mean gap between
// them, and the writer's rate.
//   link_gap_probe [--writer-mask 0x06] [--reader-mask 0xf0] [--writer-grid 192]
//                  [--reader-grid 48] [--between empty]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#define HIP_OK(x)                                                                   \
  do {                                                                              \
    hipError_t e_ = (x);                                                            \
    if (e_ != hipSuccess) {                                                         \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      return 1;                                                                     \
    }                                                                               \
  } while (0)

typedef unsigned int v4 __attribute__((ext_vector_type(4)));

// One wavefront per workgroup; workgroups outside `mask` leave.  Each of the others
// copies its own `vectors` 16-byte vectors `reps` times, 8 KiB in flight, and notes
// the earliest start and the latest end of the launch in `stamp` (100 MHz clock).
__global__ void stream_copy(const v4 *src, v4 *dst, size_t vectors, int reps,
                            unsigned long long *stamp, unsigned mask, unsigned *workers) {
  unsigned xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  if (!((mask >> (xcc & 7)) & 1))
    return;
  const unsigned long long t0 = wall_clock64();
  const v4 *s = src + blockIdx.x * vectors;
  v4 *d = dst + blockIdx.x * vectors;
  for (int r = 0; r < reps; ++r)
    for (size_t i = threadIdx.x; i < vectors; i += 64 * 8) {
      v4 x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        x[u] = __builtin_nontemporal_load(s + i + u * 64);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        d[i + u * 64] = x[u];
    }
  if (threadIdx.x == 0) {
    atomicMin(&stamp[0], t0);
    atomicMax(&stamp[1], wall_clock64());
    if (workers)
      atomicAdd(workers, 1u);
  }
}

__global__ void empty_kernel(int *p) {
  if (p == reinterpret_cast<int *>(1))
    *p = 0;
}

int main(int argc, char **argv) {
  unsigned writer_mask = 0x06, reader_mask = 0xf0;
  int writer_grid = 192, reader_grid = 48;
  std::string between = "empty";
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string k = argv[i];
    if (k == "--writer-mask")
      writer_mask = (unsigned)strtoul(argv[i + 1], nullptr, 0);
    else if (k == "--reader-mask")
      reader_mask = (unsigned)strtoul(argv[i + 1], nullptr, 0);
    else if (k == "--writer-grid")
      writer_grid = atoi(argv[i + 1]);
    else if (k == "--reader-grid")
      reader_grid = atoi(argv[i + 1]);
    else if (k == "--between")
      between = argv[i + 1];
    else {
      fprintf(stderr, "unknown option %s\n", argv[i]);
      return 2;
    }
  }
  if (writer_grid < 8 || reader_grid < 8 || writer_grid > 1024 || reader_grid > 1024 ||
      (between != "none" && between != "empty" && between != "event-default" &&
       between != "event-nofence")) {
    fprintf(stderr, "bad arguments\n");
    return 2;
  }
  const size_t per_wg = 4u << 20; // bytes per workgroup and repetition
  constexpr int kReaders = 12;
  void *host_w, *host_r, *dev_w, *dev_r;
  HIP_OK(hipHostMalloc(&host_w, per_wg * writer_grid, hipHostMallocMapped));
  HIP_OK(hipHostMalloc(&host_r, per_wg * reader_grid, hipHostMallocMapped));
  HIP_OK(hipMalloc(&dev_w, per_wg * writer_grid));
  HIP_OK(hipMalloc(&dev_r, per_wg * reader_grid));
  HIP_OK(hipMemset(dev_w, 1, per_wg * writer_grid));
  memset(host_r, 2, per_wg * reader_grid);
  unsigned long long *stamps; // [2 * k]: start, [2 * k + 1]: end; k == kReaders: the writer
  unsigned *workers;          // [0] writer, [1] last reader
  HIP_OK(hipHostMalloc(&stamps, sizeof(*stamps) * 2 * (kReaders + 1), hipHostMallocMapped));
  HIP_OK(hipHostMalloc(&workers, 2 * sizeof(unsigned), hipHostMallocMapped));
  for (int k = 0; k <= kReaders; ++k)
    stamps[2 * k] = ~0ull, stamps[2 * k + 1] = 0;
  workers[0] = workers[1] = 0;
  hipStream_t sw, sr;
  HIP_OK(hipStreamCreateWithFlags(&sw, hipStreamNonBlocking));
  HIP_OK(hipStreamCreateWithFlags(&sr, hipStreamNonBlocking));
  hipEvent_t ev[kReaders];
  for (hipEvent_t &e : ev)
    HIP_OK(hipEventCreateWithFlags(
        &e, hipEventDisableTiming |
                (between == "event-nofence" ? (unsigned)hipEventDisableSystemFence : 0u)));
  HIP_OK(hipDeviceSynchronize());

  hipLaunchKernelGGL(stream_copy, dim3(writer_grid), dim3(64), 0, sw, (const v4 *)dev_w,
                     (v4 *)host_w, per_wg / 16, 12, stamps + 2 * kReaders, writer_mask, workers);
  for (int k = 0; k < kReaders; ++k) {
    if (k > 0 && between == "empty")
      hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, sr, (int *)nullptr);
    hipLaunchKernelGGL(stream_copy, dim3(reader_grid), dim3(64), 0, sr, (const v4 *)host_r,
                       (v4 *)dev_r, per_wg / 16, 1, stamps + 2 * k, reader_mask,
                       k == kReaders - 1 ? workers + 1 : (unsigned *)nullptr);
    if (between == "event-default" || between == "event-nofence")
      HIP_OK(hipEventRecord(ev[k], sr));
  }
  HIP_OK(hipDeviceSynchronize());

  // readers 2..7 overlap the writer for certain
  double busy = 0, gaps = 0;
  for (int k = 2; k < 8; ++k) {
    busy += (stamps[2 * k + 1] - stamps[2 * k]) / 100.0;
    gaps += (stamps[2 * k] - stamps[2 * k - 1]) / 100.0;
  }
  const double reader_bytes = (double)workers[1] * per_wg * 6;
  const double writer_us = (stamps[2 * kReaders + 1] - stamps[2 * kReaders]) / 100.0;
  printf("writer mask 0x%02x (%u workgroups) %.1f GB/s | reader mask 0x%02x (%u workgroups), "
         "between its kernels: %s: %.1f GB/s inside the kernels, %.1f GB/s with the gaps, mean "
         "gap %.0f us\n",
         writer_mask, workers[0], workers[0] * 12.0 * per_wg / writer_us / 1e3, reader_mask,
         workers[1], between.c_str(), reader_bytes / busy / 1e3, reader_bytes / (busy + gaps) / 1e3,
         gaps / 6);
  return 0;
}
