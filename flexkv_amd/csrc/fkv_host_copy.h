// Host-side strided row copies used by the staging strategies of the
// copy-engine path: staging[k] <-> cpu_base + cpu_ids[k] * block_stride.
//
// Same job as scatter_to_cpu / gather_from_cpu and their worker pool in the
// reference (csrc/ce_transfer.cu:316-641): optional streaming (non-temporal)
// stores so a multi-GiB transfer does not evict the host caches, and a small
// set of helper threads because one core cannot keep up with the host link.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>

namespace fkv {

// Helper threads that split an index range [0, total) with the thread that calls
// run(): every helper and the caller get one contiguous share, run() returns when
// all shares are done.  One caller at a time.
class HostCrew {
public:
  explicit HostCrew(int helpers);
  ~HostCrew();
  HostCrew(const HostCrew &) = delete;
  HostCrew &operator=(const HostCrew &) = delete;
  int helpers() const;
  void run(int total, const std::function<void(int, int)> &body);

private:
  struct Impl;
  Impl *impl_;
};

// Copies `n` bytes; with `streaming` the stores bypass the cache when the CPU
// has AVX2/AVX-512.  Callers fence once per batch with host_copy_fence().
void host_copy_bytes(uint8_t *dst, const uint8_t *src, size_t n, bool streaming);
void host_copy_fence(bool streaming);

// Row scatter (to_cpu) or gather (!to_cpu) between a packed staging buffer and
// strided host rows.  `row_base` already includes layer, kv and in-chunk
// offsets.  When `rows_adjacent` (block_stride == chunk) runs of consecutive ids
// are merged into one copy.  `threads` <= 1 keeps all work on the caller.
void host_rows_copy(uint8_t *staging, uint8_t *row_base, const int64_t *cpu_ids,
                    int num_blocks, int64_t block_stride, int64_t chunk, bool to_cpu,
                    bool rows_adjacent, int threads, bool streaming);

// Gathers pieces of strided host rows into a dense buffer with a crew:
//   for pos in [0, num_rows), o in [0, outer), i in [0, inner):
//     dense[((pos * outer + o) * inner + i) * piece_bytes ...] =
//         row0 + ids[pos] * row_stride + o * outer_stride + i * inner_stride
// Streaming stores throughout (the buffer is read next by a copy engine, not by a
// core).  Returns the time the threads spent copying, summed, in nanoseconds.
// The host half of the H2D direction of SEGMENT_SCATTER (gather_from_cpu,
// csrc/ce_transfer.cu:585-641) for a whole batch of layers at once.
uint64_t host_gather_rows(HostCrew &crew, uint8_t *dense, const uint8_t *row0, const int64_t *ids,
                          int num_rows, int64_t row_stride, int outer, int64_t outer_stride,
                          int inner, int64_t inner_stride, int64_t piece_bytes);

} // namespace fkv
