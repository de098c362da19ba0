#include "fkv_host_copy.h"

#include <algorithm>
#include <condition_variable>
#include <cstring>
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

// Helper threads that belong to one calling thread.  A call to run() hands
// every helper a [begin, end) share, the caller works on its own share, then
// waits for the helpers.  Shares are published under the mutex with a
// generation counter, so a helper never sees a half-written job.
class RowCopyCrew {
public:
  explicit RowCopyCrew(int helpers) {
    for (int i = 0; i < helpers; ++i)
      threads_.emplace_back([this, i] { loop(i); });
    ranges_.resize(helpers);
  }
  ~RowCopyCrew() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      quit_ = true;
    }
    wake_.notify_all();
    for (auto &t : threads_)
      if (t.joinable())
        t.join();
  }
  int helpers() const { return (int)threads_.size(); }

  void run(int total, const std::function<void(int, int)> &body) {
    const int parts = helpers() + 1;
    const int share = (total + parts - 1) / parts;
    {
      std::lock_guard<std::mutex> lk(mu_);
      body_ = &body;
      pending_ = 0;
      for (int h = 0; h < helpers(); ++h) {
        int b = std::min(total, (h + 1) * share);
        int e = std::min(total, b + share);
        ranges_[h] = {b, e};
        if (b < e)
          ++pending_;
      }
      ++generation_;
    }
    wake_.notify_all();
    body(0, std::min(share, total));
    std::unique_lock<std::mutex> lk(mu_);
    done_.wait(lk, [this] { return pending_ == 0; });
    body_ = nullptr;
  }

private:
  void loop(int idx) {
    uint64_t seen = 0;
    for (;;) {
      const std::function<void(int, int)> *fn = nullptr;
      std::pair<int, int> r;
      {
        std::unique_lock<std::mutex> lk(mu_);
        wake_.wait(lk, [&] { return quit_ || generation_ != seen; });
        if (quit_)
          return;
        seen = generation_;
        fn = body_;
        r = ranges_[idx];
      }
      if (r.first < r.second) {
        (*fn)(r.first, r.second);
        std::lock_guard<std::mutex> lk(mu_);
        if (--pending_ == 0)
          done_.notify_one();
      }
    }
  }

  std::vector<std::thread> threads_;
  std::vector<std::pair<int, int>> ranges_;
  std::mutex mu_;
  std::condition_variable wake_, done_;
  const std::function<void(int, int)> *body_ = nullptr;
  uint64_t generation_ = 0;
  int pending_ = 0;
  bool quit_ = false;
};

RowCopyCrew &crew_for_thread(int threads) {
  // Sized on first use by this thread, like the reference's thread_local pool
  // (csrc/ce_transfer.cu:412-418).
  thread_local RowCopyCrew crew(std::max(0, threads - 1));
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
  RowCopyCrew &crew = crew_for_thread(threads);
  if (crew.helpers() == 0)
    body(0, num_blocks);
  else
    crew.run(num_blocks, body);
}

} // namespace fkv
