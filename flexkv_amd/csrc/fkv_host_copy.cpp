#include "fkv_host_copy.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#if defined(__x86_64__)
#include <immintrin.h>
#define FKV_X86 1
#else
#define FKV_X86 0
#endif

namespace fkv {
namespace {

enum class Isa { Plain, Avx2, Avx512 };

Isa detect_isa() {
#if FKV_X86
  if (__builtin_cpu_supports("avx512f"))
    return Isa::Avx512;
  if (__builtin_cpu_supports("avx2"))
    return Isa::Avx2;
#endif
  return Isa::Plain;
}
Isa isa() {
  static const Isa v = detect_isa();
  return v;
}

#if FKV_X86
// Streaming stores need an aligned destination: copy the unaligned head and
// the sub-vector tail normally, stream the aligned middle.
template <int W, typename StoreFn>
inline void stream_copy(uint8_t *dst, const uint8_t *src, size_t n, StoreFn store) {
  size_t head = (W - (reinterpret_cast<uintptr_t>(dst) & (W - 1))) & (W - 1);
  head = std::min(head, n);
  if (head)
    std::memcpy(dst, src, head);
  size_t i = head;
  for (; i + W <= n; i += W)
    store(dst + i, src + i);
  if (i < n)
    std::memcpy(dst + i, src + i, n - i);
}

__attribute__((target("avx512f"))) void copy_avx512(uint8_t *dst, const uint8_t *src,
                                                    size_t n) {
  stream_copy<64>(dst, src, n, [](uint8_t *d, const uint8_t *s)
                                   __attribute__((target("avx512f"))) {
                                     _mm512_stream_si512(reinterpret_cast<__m512i *>(d),
                                                         _mm512_loadu_si512(s));
                                   });
}
__attribute__((target("avx2"))) void copy_avx2(uint8_t *dst, const uint8_t *src, size_t n) {
  stream_copy<32>(dst, src, n, [](uint8_t *d, const uint8_t *s)
                                   __attribute__((target("avx2"))) {
                                     _mm256_stream_si256(
                                         reinterpret_cast<__m256i *>(d),
                                         _mm256_loadu_si256(
                                             reinterpret_cast<const __m256i *>(s)));
                                   });
}
#endif

} // namespace

// A call to run() hands every helper a [begin, end) share, the caller works on its
// own share, then waits for the helpers.  Shares are published under the mutex with
// a generation counter, so a helper never sees a half-written job.
struct HostCrew::Impl {
  explicit Impl(int helpers) {
    ranges.resize(helpers);
    threads.reserve(helpers);
    for (int i = 0; i < helpers; ++i) {
      try {
        threads.emplace_back([this, i] { loop(i); });
      } catch (const std::exception &) { // the system has no more threads: work with those there are
        break;
      }
    }
    ranges.resize(threads.size());
  }
  ~Impl() {
    {
      std::lock_guard<std::mutex> lk(mu);
      quit = true;
    }
    wake.notify_all();
    for (auto &t : threads)
      if (t.joinable())
        t.join();
  }
  void loop(int idx) {
    uint64_t seen = 0;
    for (;;) {
      const std::function<void(int, int)> *fn = nullptr;
      std::pair<int, int> r;
      {
        std::unique_lock<std::mutex> lk(mu);
        wake.wait(lk, [&] { return quit || generation != seen; });
        if (quit)
          return;
        seen = generation;
        fn = body;
        r = ranges[idx];
      }
      if (r.first < r.second) {
        (*fn)(r.first, r.second);
        std::lock_guard<std::mutex> lk(mu);
        if (--pending == 0)
          done.notify_one();
      }
    }
  }

  std::vector<std::thread> threads;
  std::vector<std::pair<int, int>> ranges;
  std::mutex mu;
  std::condition_variable wake, done;
  const std::function<void(int, int)> *body = nullptr;
  uint64_t generation = 0;
  int pending = 0;
  bool quit = false;
};

HostCrew::HostCrew(int helpers) : impl_(new Impl(std::max(0, helpers))) {}
HostCrew::~HostCrew() { delete impl_; }
int HostCrew::helpers() const { return (int)impl_->threads.size(); }

void HostCrew::run(int total, const std::function<void(int, int)> &body) {
  Impl &m = *impl_;
  const int parts = helpers() + 1;
  const int share = (total + parts - 1) / parts;
  {
    std::lock_guard<std::mutex> lk(m.mu);
    m.body = &body;
    m.pending = 0;
    for (int h = 0; h < helpers(); ++h) {
      int b = std::min(total, (h + 1) * share);
      int e = std::min(total, b + share);
      m.ranges[h] = {b, e};
      if (b < e)
        ++m.pending;
    }
    ++m.generation;
  }
  m.wake.notify_all();
  body(0, std::min(share, total));
  std::unique_lock<std::mutex> lk(m.mu);
  m.done.wait(lk, [&m] { return m.pending == 0; });
  m.body = nullptr;
}

namespace {

HostCrew &crew_for_thread(int threads) {
  // Sized on first use by this thread, like the reference's thread_local pool
  // (csrc/ce_transfer.cu:412-418).
  thread_local HostCrew crew(std::max(0, threads - 1));
  return crew;
}

} // namespace

void host_copy_bytes(uint8_t *dst, const uint8_t *src, size_t n, bool streaming) {
#if FKV_X86
  if (streaming) {
    switch (isa()) {
    case Isa::Avx512:
      copy_avx512(dst, src, n);
      return;
    case Isa::Avx2:
      copy_avx2(dst, src, n);
      return;
    default:
      break;
    }
  }
#endif
  std::memcpy(dst, src, n);
}

void host_copy_fence(bool streaming) {
#if FKV_X86
  if (streaming && isa() != Isa::Plain)
    _mm_sfence();
#else
  (void)streaming;
#endif
}

namespace {
inline void prefetch_row(const uint8_t *p, bool for_write) {
  if (for_write)
    __builtin_prefetch(p, 1, 0);
  else
    __builtin_prefetch(p, 0, 0);
}
} // namespace

void host_rows_copy(uint8_t *staging, uint8_t *row_base, const int64_t *cpu_ids,
                    int num_blocks, int64_t block_stride, int64_t chunk, bool to_cpu,
                    bool rows_adjacent, int threads, bool streaming) {
  auto move = [&](uint8_t *row, uint8_t *stg, size_t n) {
    if (to_cpu)
      host_copy_bytes(row, stg, n, streaming);
    else
      host_copy_bytes(stg, row, n, streaming);
  };
  if (rows_adjacent) {
    int k = 0;
    while (k < num_blocks) {
      int first = k;
      while (k + 1 < num_blocks && cpu_ids[k + 1] == cpu_ids[k] + 1)
        ++k;
      ++k;
      move(row_base + cpu_ids[first] * block_stride, staging + (int64_t)first * chunk,
           (size_t)(k - first) * (size_t)chunk);
    }
    host_copy_fence(streaming);
    return;
  }
  constexpr int kPrefetchAhead = 16;
  std::function<void(int, int)> body = [&](int begin, int end) {
    for (int k = begin; k < end; ++k) {
      if (k + kPrefetchAhead < end)
        prefetch_row(row_base + cpu_ids[k + kPrefetchAhead] * block_stride, to_cpu);
      move(row_base + cpu_ids[k] * block_stride, staging + (int64_t)k * chunk, (size_t)chunk);
    }
    host_copy_fence(streaming);
  };
  if (threads <= 1 || num_blocks < 8) {
    body(0, num_blocks);
    return;
  }
  HostCrew &crew = crew_for_thread(threads);
  if (crew.helpers() == 0)
    body(0, num_blocks);
  else
    crew.run(num_blocks, body);
}

uint64_t host_gather_rows(HostCrew &crew, uint8_t *dense, const uint8_t *row0, const int64_t *ids,
                          int num_rows, int64_t row_stride, int outer, int64_t outer_stride,
                          int inner, int64_t inner_stride, int64_t piece_bytes) {
  std::atomic<uint64_t> busy_ns{0};
  const std::function<void(int, int)> body = [&](int begin, int end) {
    const auto t0 = std::chrono::steady_clock::now();
    for (int pos = begin; pos < end; ++pos) {
      const uint8_t *src = row0 + ids[pos] * row_stride;
      uint8_t *dst = dense + (int64_t)pos * outer * inner * piece_bytes;
      for (int o = 0; o < outer; ++o)
        for (int i = 0; i < inner; ++i, dst += piece_bytes)
          host_copy_bytes(dst, src + (int64_t)o * outer_stride + (int64_t)i * inner_stride,
                          (size_t)piece_bytes, true);
    }
    host_copy_fence(true);
    busy_ns.fetch_add((uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
                          std::chrono::steady_clock::now() - t0)
                          .count(),
                      std::memory_order_relaxed);
  };
  if (crew.helpers() == 0 || num_rows < 2 * (crew.helpers() + 1))
    body(0, num_rows);
  else
    crew.run(num_rows, body);
  return busy_ns.load(std::memory_order_relaxed);
}

} // namespace fkv
