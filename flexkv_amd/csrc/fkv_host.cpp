// Host-pool memory: mapped pinned allocation and chunked registration, plus the
// plain pinned-copy measurement that serves as the host-link reference rate.
//
// Counterpart of flexkv/transfer/host_buffer.py in the reference
// (cudaHostRegister :66-98, cudaHostUnregister :101-118,
// alloc_mapped_host_tensor :180-202).
#include "fkv_internal.h"

#include <algorithm>

namespace {
// Pieces of at most `chunk` bytes covering [0, bytes); one piece when chunk == 0
// or the buffer is not larger than a chunk (host_buffer.py:79-98).
int64_t piece_count(size_t bytes, size_t chunk) {
  if (chunk == 0 || bytes <= chunk)
    return 1;
  return (int64_t)((bytes + chunk - 1) / chunk);
}
} // namespace

extern "C" {

size_t fkv_host_chunk_bytes_from_gb(double chunk_gb) {
  if (chunk_gb <= 0)
    return 0;
  // 4 KiB of head-room under the requested size, then down to a page boundary
  long long c = (long long)(chunk_gb * (double)(1ull << 30)) - 4096;
  if (c <= 0)
    return 0;
  return (size_t)(c & ~0xFFFll);
}

int64_t fkv_host_register_plan(size_t bytes, size_t chunk_bytes, size_t *offsets,
                               size_t *sizes, int64_t capacity) {
  const int64_t n = piece_count(bytes, chunk_bytes);
  for (int64_t i = 0; i < n && i < capacity; ++i) {
    const size_t off = (n == 1) ? 0 : (size_t)i * chunk_bytes;
    if (offsets)
      offsets[i] = off;
    if (sizes)
      sizes[i] = (n == 1) ? bytes : std::min(chunk_bytes, bytes - off);
  }
  return n;
}

int fkv_host_alloc(size_t bytes, void **out) try {
  fkv::clear_error();
  if (!out || bytes == 0)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_host_alloc: bad arguments");
  void *p = nullptr;
  hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocPortable | hipHostMallocMapped);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fkv::fail(FKV_ERR_RUNTIME, "hipHostMalloc(%zu) failed: %s", bytes,
                     hipGetErrorString(e));
  }
  *out = p;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_host_free(void *ptr) try {
  fkv::clear_error();
  if (!ptr)
    return FKV_OK;
  FKV_HIP_TRY(hipHostFree(ptr));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_host_register(void *ptr, size_t bytes, size_t chunk_bytes) try {
  fkv::clear_error();
  if (!ptr || bytes == 0)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_host_register: bad arguments");
  const int64_t n = piece_count(bytes, chunk_bytes);
  std::vector<size_t> off((size_t)n), sz((size_t)n);
  fkv_host_register_plan(bytes, chunk_bytes, off.data(), sz.data(), n);
  for (int64_t i = 0; i < n; ++i) {
    hipError_t e = hipHostRegister(static_cast<uint8_t *>(ptr) + off[i], sz[i],
                                   hipHostRegisterPortable | hipHostRegisterMapped);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      for (int64_t k = i - 1; k >= 0; --k) // undo what was registered so far
        (void)hipHostUnregister(static_cast<uint8_t *>(ptr) + off[k]);
      (void)hipGetLastError();
      return fkv::fail(FKV_ERR_RUNTIME,
                       "hipHostRegister failed at offset=%zu bytes with error %d (%s)", off[i],
                       (int)e, hipGetErrorString(e));
    }
  }
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_host_unregister(void *ptr, size_t bytes, size_t chunk_bytes) try {
  fkv::clear_error();
  if (!ptr || bytes == 0)
    return fkv::fail(FKV_ERR_INVALID_ARG, "fkv_host_unregister: bad arguments");
  const int64_t n = piece_count(bytes, chunk_bytes);
  std::vector<size_t> off((size_t)n), sz((size_t)n);
  fkv_host_register_plan(bytes, chunk_bytes, off.data(), sz.data(), n);
  int bad = 0;
  for (int64_t i = n - 1; i >= 0; --i) {
    if (hipHostUnregister(static_cast<uint8_t *>(ptr) + off[i]) != hipSuccess) {
      (void)hipGetLastError();
      ++bad;
    }
  }
  if (bad)
    return fkv::fail(FKV_ERR_RUNTIME, "hipHostUnregister failed for %d of %lld pieces", bad,
                     (long long)n);
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_measure_link_peak(int32_t device, size_t bytes, int32_t reps, int32_t direction,
                          double *best_gbps, double *median_gbps) try {
  using namespace fkv;
  clear_error();
  if (bytes == 0 || reps < 1 || !best_gbps)
    return fail(FKV_ERR_INVALID_ARG, "fkv_measure_link_peak: bad arguments");
  DeviceGuard guard(device);
  if (!guard.ok())
    return fail(FKV_ERR_RUNTIME, "cannot select HIP device %d", device);
  void *h = nullptr, *d = nullptr;
  hipStream_t st = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = FKV_OK;
  std::vector<double> rates;
  auto cleanup = [&] {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (st) (void)hipStreamDestroy(st);
    if (d) (void)hipFree(d);
    if (h) (void)hipHostFree(h);
    (void)hipGetLastError();
  };
#define LP_TRY(x)                                                              \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      (void)hipGetLastError();                                                 \
      rc = fail(FKV_ERR_RUNTIME, "%s: %s", #x, hipGetErrorString(e_));         \
      cleanup();                                                               \
      return rc;                                                               \
    }                                                                          \
  } while (0)
  LP_TRY(hipHostMalloc(&h, bytes, hipHostMallocPortable | hipHostMallocMapped));
  LP_TRY(hipMalloc(&d, bytes));
  LP_TRY(hipStreamCreate(&st));
  LP_TRY(hipEventCreate(&e0));
  LP_TRY(hipEventCreate(&e1));
  std::fill_n(static_cast<uint8_t *>(h), bytes, (uint8_t)0x5a);
  LP_TRY(hipMemsetAsync(d, 0xa5, bytes, st));
  for (int r = -1; r < reps; ++r) { // r == -1 is an untimed warm-up
    LP_TRY(hipEventRecord(e0, st));
    if (direction == 0)
      LP_TRY(hipMemcpyAsync(h, d, bytes, hipMemcpyDeviceToHost, st));
    else
      LP_TRY(hipMemcpyAsync(d, h, bytes, hipMemcpyHostToDevice, st));
    LP_TRY(hipEventRecord(e1, st));
    LP_TRY(hipEventSynchronize(e1));
    float ms = 0;
    LP_TRY(hipEventElapsedTime(&ms, e0, e1));
    if (r >= 0 && ms > 0)
      rates.push_back((double)bytes / (ms * 1e-3) / 1e9);
  }
#undef LP_TRY
  cleanup();
  if (rates.empty())
    return fail(FKV_ERR_RUNTIME, "no timed repetition");
  std::sort(rates.begin(), rates.end());
  *best_gbps = rates.back();
  if (median_gbps)
    *median_gbps = rates[rates.size() / 2];
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
