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

namespace fkv {

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

} // namespace fkv
