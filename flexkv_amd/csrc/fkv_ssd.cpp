// Host pool <-> SSD files: the step before a host->GPU restore when the blocks
// of a request sit one tier further down, and the step after a GPU->host put
// that spills them there.
//
// Takes the place of transfer_kv_blocks_ssd / SSDIOCTX / IOUring of the
// reference (csrc/transfer_ssd.{h,cpp}).  Same contract: an SSD block id names
// (device, file, block-in-file) by round-robin striping; inside a file a chunk
// lives at  block_in_file*block_stride + layer*ssd_layer_stride + kv*ssd_kv_stride,
// in the host pool at  cpu_block*block_stride + layer*cpu_layer_stride +
// kv*cpu_kv_stride  (one block stride for both sides, csrc/transfer_ssd.cpp:68-72).
//
// Built differently.  A call is first turned into a list of *extents* (file
// offset, host address, length) generated in ascending file order per file;
// extents adjacent in the file are merged into one vectored request whose iovecs
// are the maximal host-contiguous runs, whatever the layouts are.  A block-first
// pool then moves a whole block per request, runs of neighbouring blocks one
// request per run; a layer-first pool one request per (layer, kv, run of
// blocks).  The request list is then executed by one of two engines: an
// io_uring driven directly through its system calls (the image has no
// liburing), or a pool of threads doing preadv/pwritev.  Short transfers are
// completed with follow-up calls in both.
//
// With ssd_io_opt off the requests are one chunk each, as in the reference's
// baseline mode; the bytes moved are the same.
#include "fkv_internal.h"

#include <fcntl.h>
#include <linux/io_uring.h>
#include <sys/mman.h>
#include <sys/syscall.h>
#include <sys/uio.h>
#include <unistd.h>

#include <exception>
#include <algorithm>
#include <atomic>
#include <cerrno>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <limits.h>
#include <mutex>
#include <thread>

namespace {

using fkv::fail;

constexpr int kMaxIov = 1024;                 // IOV_MAX on Linux
constexpr int64_t kMaxRequestBytes = 16 << 20; // keeps requests many enough to run in parallel

struct Request {
  int fd = -1;
  int fallback_fd = -1; // buffered descriptor of the same file when `fd` is O_DIRECT
  int64_t file_off = 0;
  int64_t bytes = 0;
  uint32_t iov_first = 0; // into Plan::iovs
  uint32_t iov_count = 0;
};

struct Plan {
  std::vector<Request> requests;
  std::vector<iovec> iovs;
};

// Where an SSD block id lives: csrc/transfer_ssd.cpp:33-38, 65-67.
struct BlockPlace {
  int device, file;
  int64_t in_file;
};
BlockPlace locate(int64_t ssd_block_id, int round_robin, int num_devices, int files_per_device) {
  const int64_t stripe = ssd_block_id / round_robin;
  const int64_t in_device = (stripe / num_devices) * round_robin + ssd_block_id % round_robin;
  return {(int)(stripe % num_devices), (int)(in_device % files_per_device),
          in_device / files_per_device};
}

// Appends extent (file_off, ptr, len) of `fd`; merges it into the open request
// when it continues that request in the file.
struct PlanBuilder {
  Plan &plan;
  bool merge;
  explicit PlanBuilder(Plan &p, bool m) : plan(p), merge(m) {}
  void add(int fd, int fallback_fd, int64_t file_off, void *ptr, int64_t len) {
    if (merge && !plan.requests.empty()) {
      Request &r = plan.requests.back();
      if (r.fd == fd && r.file_off + r.bytes == file_off && r.bytes + len <= kMaxRequestBytes) {
        iovec &last = plan.iovs.back();
        if (static_cast<char *>(last.iov_base) + last.iov_len == ptr) {
          last.iov_len += (size_t)len;
          r.bytes += len;
          return;
        }
        if ((int)r.iov_count < kMaxIov) {
          plan.iovs.push_back({ptr, (size_t)len});
          ++r.iov_count;
          r.bytes += len;
          return;
        }
      }
    }
    Request r;
    r.fd = fd;
    r.fallback_fd = fallback_fd;
    r.file_off = file_off;
    r.bytes = len;
    r.iov_first = (uint32_t)plan.iovs.size();
    r.iov_count = 1;
    plan.iovs.push_back({ptr, (size_t)len});
    plan.requests.push_back(r);
  }
};

bool aligned4k(int64_t v) { return (v & 4095) == 0; }

// A plan of a few large requests keeps only a few workers busy (and a buffered
// request is one thread's memcpy): cut requests so that every worker gets about
// two, in pieces of at least 1 MiB on 4 KiB boundaries.
void split_for_parallelism(Plan *plan, int workers) {
  if (workers <= 1 || plan->requests.empty() || (int)plan->requests.size() >= 2 * workers)
    return;
  int64_t total = 0;
  for (const Request &r : plan->requests)
    total += r.bytes;
  const int64_t piece = std::max<int64_t>(1 << 20, (total / (2 * workers)) & ~int64_t(4095));
  Plan cut;
  for (const Request &r : plan->requests) {
    const int64_t pieces = std::max<int64_t>(1, (r.bytes + piece / 2) / piece);
    uint32_t iov = r.iov_first;
    size_t used = 0; // bytes of iovec `iov` already placed
    int64_t placed = 0;
    for (int64_t j = 0; j < pieces; ++j) {
      Request q = r;
      q.file_off = r.file_off + placed;
      q.bytes = j == pieces - 1 ? r.bytes - placed : piece;
      q.iov_first = (uint32_t)cut.iovs.size();
      q.iov_count = 0;
      for (int64_t need = q.bytes; need > 0;) {
        const iovec &v = plan->iovs[iov];
        const size_t take = (size_t)std::min<int64_t>((int64_t)(v.iov_len - used), need);
        cut.iovs.push_back({static_cast<char *>(v.iov_base) + used, take});
        ++q.iov_count;
        need -= (int64_t)take;
        used += take;
        if (used == v.iov_len) {
          ++iov;
          used = 0;
        }
      }
      cut.requests.push_back(q);
      placed += q.bytes;
    }
  }
  *plan = std::move(cut);
}

// preadv / pwritev until `total` bytes have moved (csrc/transfer_ssd.cpp:262-325).
bool transfer_iov_full(int fd, const iovec *iov, int iovcnt, int64_t offset, int64_t total,
                       bool is_read, int64_t already = 0) {
  std::vector<iovec> rest(iov, iov + iovcnt);
  size_t head = 0;
  int64_t done = 0;
  auto advance = [&](int64_t n) {
    done += n;
    while (n > 0 && head < rest.size()) {
      if ((int64_t)rest[head].iov_len > n) {
        rest[head].iov_base = static_cast<char *>(rest[head].iov_base) + n;
        rest[head].iov_len -= (size_t)n;
        n = 0;
      } else {
        n -= (int64_t)rest[head].iov_len;
        ++head;
      }
    }
  };
  advance(already);
  errno = 0; // so that a transfer cut short by the end of the file reports no stale code
  while (done < total) {
    const int cnt = (int)std::min<size_t>(rest.size() - head, kMaxIov);
    const ssize_t n = is_read ? preadv(fd, rest.data() + head, cnt, offset + done)
                              : pwritev(fd, rest.data() + head, cnt, offset + done);
    if (n < 0) {
      if (errno == EINTR)
        continue;
      return false;
    }
    if (n == 0)
      break; // end of file
    advance(n);
  }
  return done == total;
}

// What an engine reports back.  `direct_refused` counts requests the kernel would
// not do with O_DIRECT on this host memory (EFAULT: the pages cannot be pinned
// for DMA, as with host memory mapped by the GPU driver; EINVAL: alignment the
// device does not take) and that were then done through the page cache.
struct Outcome {
  std::atomic<int> failed{0}, err{0}, direct_refused{0};
  void note_failure(int e) {
    int zero = 0;
    err.compare_exchange_strong(zero, e);
    failed.fetch_add(1, std::memory_order_relaxed);
  }
};

// A failed O_DIRECT request is repeated on the buffered descriptor.
bool retry_buffered(const Plan &plan, const Request &r, bool is_read, int e, Outcome *out) {
  if (r.fallback_fd < 0 || (e != EFAULT && e != EINVAL))
    return false;
  if (!transfer_iov_full(r.fallback_fd, plan.iovs.data() + r.iov_first, (int)r.iov_count,
                         r.file_off, r.bytes, is_read))
    return false;
  out->direct_refused.fetch_add(1, std::memory_order_relaxed);
  return true;
}

// ---- io_uring through its system calls -----------------------------------
class Ring {
public:
  Ring(int entries, unsigned flags) {
    if (entries <= 0)
      return;
    io_uring_params p;
    std::memset(&p, 0, sizeof(p));
    p.flags = flags;
    fd_ = (int)syscall(__NR_io_uring_setup, (unsigned)entries, &p);
    if (fd_ < 0)
      return;
    sq_bytes_ = p.sq_off.array + p.sq_entries * sizeof(unsigned);
    cq_bytes_ = p.cq_off.cqes + p.cq_entries * sizeof(io_uring_cqe);
    const bool single = p.features & IORING_FEAT_SINGLE_MMAP;
    if (single)
      sq_bytes_ = cq_bytes_ = std::max(sq_bytes_, cq_bytes_);
    sq_ptr_ = mmap(nullptr, sq_bytes_, PROT_READ | PROT_WRITE, MAP_SHARED | MAP_POPULATE, fd_,
                   IORING_OFF_SQ_RING);
    cq_ptr_ = single ? sq_ptr_
                     : mmap(nullptr, cq_bytes_, PROT_READ | PROT_WRITE,
                            MAP_SHARED | MAP_POPULATE, fd_, IORING_OFF_CQ_RING);
    sqes_bytes_ = p.sq_entries * sizeof(io_uring_sqe);
    sqes_ = static_cast<io_uring_sqe *>(mmap(nullptr, sqes_bytes_, PROT_READ | PROT_WRITE,
                                             MAP_SHARED | MAP_POPULATE, fd_, IORING_OFF_SQES));
    if (sq_ptr_ == MAP_FAILED || cq_ptr_ == MAP_FAILED || sqes_ == MAP_FAILED) {
      close_all();
      return;
    }
    char *sq = static_cast<char *>(sq_ptr_), *cq = static_cast<char *>(cq_ptr_);
    sq_tail_ = reinterpret_cast<std::atomic<unsigned> *>(sq + p.sq_off.tail);
    sq_mask_ = *reinterpret_cast<unsigned *>(sq + p.sq_off.ring_mask);
    sq_flags_ = reinterpret_cast<std::atomic<unsigned> *>(sq + p.sq_off.flags);
    sq_array_ = reinterpret_cast<unsigned *>(sq + p.sq_off.array);
    cq_head_ = reinterpret_cast<std::atomic<unsigned> *>(cq + p.cq_off.head);
    cq_tail_ = reinterpret_cast<std::atomic<unsigned> *>(cq + p.cq_off.tail);
    cq_mask_ = *reinterpret_cast<unsigned *>(cq + p.cq_off.ring_mask);
    cqes_ = reinterpret_cast<io_uring_cqe *>(cq + p.cq_off.cqes);
    entries_ = (int)p.sq_entries;
    sqpoll_ = flags & IORING_SETUP_SQPOLL;
  }
  ~Ring() { close_all(); }
  bool enabled() const { return entries_ > 0; }

  // Runs all requests; at most `entries_` are in flight.
  // `through_page_cache`: the descriptors are buffered ones.  Such a request is a
  // memcpy when its pages are cached, and the kernel would do it inline in the
  // submitting thread, one after the other; IOSQE_ASYNC hands every request to
  // the ring's worker pool instead, so the copies run side by side.
  void run(const Plan &plan, bool is_read, unsigned short ioprio, bool through_page_cache,
           Outcome *out) {
    const size_t n = plan.requests.size();
    size_t next = 0, finished = 0;
    int inflight = 0;
    unsigned unsubmitted = 0; // queued in the ring, not yet taken by the kernel
    unsigned local_tail = sq_tail_->load(std::memory_order_relaxed);
    while (finished < n) {
      while (next < n && inflight < entries_) {
        const Request &r = plan.requests[next];
        io_uring_sqe *sqe = &sqes_[local_tail & sq_mask_];
        std::memset(sqe, 0, sizeof(*sqe));
        sqe->opcode = is_read ? IORING_OP_READV : IORING_OP_WRITEV;
        sqe->fd = r.fd;
        sqe->off = (uint64_t)r.file_off;
        sqe->addr = (uint64_t)(uintptr_t)(plan.iovs.data() + r.iov_first);
        sqe->len = r.iov_count;
        sqe->ioprio = ioprio;
        sqe->flags = through_page_cache ? IOSQE_ASYNC : 0;
        sqe->user_data = next;
        sq_array_[local_tail & sq_mask_] = local_tail & sq_mask_;
        ++local_tail;
        ++next;
        ++inflight;
        ++unsubmitted;
      }
      sq_tail_->store(local_tail, std::memory_order_release);
      unsigned enter_flags = IORING_ENTER_GETEVENTS;
      if (sqpoll_ && (sq_flags_->load(std::memory_order_acquire) & IORING_SQ_NEED_WAKEUP))
        enter_flags |= IORING_ENTER_SQ_WAKEUP;
      const long rc = syscall(__NR_io_uring_enter, fd_, sqpoll_ ? 0u : unsubmitted, 1u,
                              enter_flags, nullptr, 0);
      if (rc < 0 && errno != EINTR && errno != EAGAIN && errno != EBUSY) {
        const int e = errno; // the ring is unusable
        for (size_t k = finished; k < n; ++k)
          out->note_failure(e);
        return;
      }
      if (sqpoll_)
        unsubmitted = 0;
      else if (rc > 0)
        unsubmitted -= std::min<unsigned>(unsubmitted, (unsigned)rc);
      unsigned head = cq_head_->load(std::memory_order_relaxed);
      const unsigned tail = cq_tail_->load(std::memory_order_acquire);
      for (; head != tail; ++head) {
        const io_uring_cqe &c = cqes_[head & cq_mask_];
        const Request &r = plan.requests[(size_t)c.user_data];
        bool ok = c.res == r.bytes;
        int e = c.res < 0 ? -c.res : 0;
        if (!ok && c.res >= 0) { // short transfer: finish it here
          ok = transfer_iov_full(r.fd, plan.iovs.data() + r.iov_first, (int)r.iov_count,
                                 r.file_off, r.bytes, is_read, c.res);
          e = ok ? 0 : (errno ? errno : EIO);
        }
        if (!ok && !retry_buffered(plan, r, is_read, e, out))
          out->note_failure(e);
        ++finished;
        --inflight;
      }
      cq_head_->store(head, std::memory_order_release);
    }
  }

private:
  void close_all() {
    if (sqes_ && sqes_ != MAP_FAILED)
      munmap(sqes_, sqes_bytes_);
    if (cq_ptr_ && cq_ptr_ != MAP_FAILED && cq_ptr_ != sq_ptr_)
      munmap(cq_ptr_, cq_bytes_);
    if (sq_ptr_ && sq_ptr_ != MAP_FAILED)
      munmap(sq_ptr_, sq_bytes_);
    if (fd_ >= 0)
      close(fd_);
    fd_ = -1;
    entries_ = 0;
    sqes_ = nullptr;
    sq_ptr_ = cq_ptr_ = nullptr;
  }
  int fd_ = -1, entries_ = 0;
  bool sqpoll_ = false;
  void *sq_ptr_ = nullptr, *cq_ptr_ = nullptr;
  size_t sq_bytes_ = 0, cq_bytes_ = 0, sqes_bytes_ = 0;
  io_uring_sqe *sqes_ = nullptr;
  io_uring_cqe *cqes_ = nullptr;
  std::atomic<unsigned> *sq_tail_ = nullptr, *sq_flags_ = nullptr, *cq_head_ = nullptr,
                        *cq_tail_ = nullptr;
  unsigned sq_mask_ = 0, cq_mask_ = 0;
  unsigned *sq_array_ = nullptr;
};

// ---- thread engine --------------------------------------------------------
// Requests are taken from a shared counter, so a slow file does not hold up the
// threads that finished their share.
void run_threads(const Plan &plan, bool is_read, int num_threads, Outcome *out) {
  const size_t n = plan.requests.size();
  num_threads = (int)std::max<size_t>(1, std::min<size_t>(num_threads, n));
  std::atomic<size_t> next{0};
  auto work = [&] {
    for (;;) {
      const size_t i = next.fetch_add(1, std::memory_order_relaxed);
      if (i >= n)
        return;
      const Request &r = plan.requests[i];
      if (transfer_iov_full(r.fd, plan.iovs.data() + r.iov_first, (int)r.iov_count, r.file_off,
                            r.bytes, is_read))
        continue;
      const int e = errno ? errno : EIO; // 0: the file ended before the request did
      if (!retry_buffered(plan, r, is_read, e, out))
        out->note_failure(e);
    }
  };
  std::vector<std::thread> pool;
  for (int t = 1; t < num_threads; ++t) {
    try {
      pool.emplace_back(work);
    } catch (const std::exception &) { // no more threads to be had: those there are do the work
      break;
    }
  }
  work();
  for (auto &t : pool)
    t.join();
}

#ifndef IOPRIO_CLASS_SHIFT
#define IOPRIO_CLASS_SHIFT 13
#endif
constexpr int kIoprioRT = 1, kIoprioBE = 2;
unsigned short ioprio_value(int cls, int data) {
  return (unsigned short)((cls << IOPRIO_CLASS_SHIFT) | data);
}

} // namespace

struct fkv_ssd_ctx {
  int num_devices = 0, files_per_device = 0;
  std::vector<int> fd_buffered, fd_direct; // [device][file]
  std::unique_ptr<Ring> ring;
  std::mutex ring_mu; // one call at a time drives the ring
  // Host pool for which O_DIRECT was refused: later calls on it go buffered at once.
  std::atomic<uintptr_t> no_direct_pool{0};
  std::atomic<bool> last_direct{false}; // the last call went through O_DIRECT
  unsigned short read_ioprio = 0, write_ioprio = 0;
  ~fkv_ssd_ctx() {
    for (int fd : fd_buffered)
      if (fd >= 0)
        close(fd);
    for (int fd : fd_direct)
      if (fd >= 0)
        close(fd);
  }
};

namespace {

struct SsdCall {
  int32_t start_layer, num_layers, num_blocks, kv_dim, round_robin;
  void *cpu_ptr;
  const int64_t *ssd_ids, *cpu_ids;
  int64_t cpu_layer_stride, cpu_kv_stride, ssd_layer_stride, ssd_kv_stride, chunk, block_stride;
  bool opt;
};

int check_call(const SsdCall &c) {
  if (c.num_blocks < 0 || c.num_layers < 0 || c.start_layer < 0 || c.kv_dim < 1 ||
      c.round_robin < 1 || c.chunk <= 0 || c.block_stride <= 0)
    return fail(FKV_ERR_INVALID_ARG,
                "ssd transfer: num_blocks=%d layers=[%d,+%d) kv_dim=%d round_robin=%d chunk=%lld "
                "block_stride=%lld",
                c.num_blocks, c.start_layer, c.num_layers, c.kv_dim, c.round_robin,
                (long long)c.chunk, (long long)c.block_stride);
  if (c.num_blocks > 0 && c.num_layers > 0 && (!c.cpu_ptr || !c.ssd_ids || !c.cpu_ids))
    return fail(FKV_ERR_INVALID_ARG, "ssd transfer: null pointer");
  for (int i = 0; i < c.num_blocks; ++i)
    if (c.ssd_ids[i] < 0 || c.cpu_ids[i] < 0)
      return fail(FKV_ERR_INVALID_ARG, "negative block id at position %d", i);
  return FKV_OK;
}

// The request list of one call.  `fds[device*files + file]`, -1 entries allowed
// when only the shape of the plan is of interest.
void build_plan(const SsdCall &c, int num_devices, int files_per_device, const int *fds,
                const int *fallback_fds, Plan *plan) {
  struct Blk {
    int device, file;
    int64_t in_file, cpu;
  };
  std::vector<Blk> blks(c.num_blocks);
  for (int i = 0; i < c.num_blocks; ++i) {
    const BlockPlace p = locate(c.ssd_ids[i], c.round_robin, num_devices, files_per_device);
    blks[i] = {p.device, p.file, p.in_file, c.cpu_ids[i]};
  }
  std::stable_sort(blks.begin(), blks.end(), [](const Blk &a, const Blk &b) {
    if (a.device != b.device)
      return a.device < b.device;
    if (a.file != b.file)
      return a.file < b.file;
    return a.in_file < b.in_file;
  });
  PlanBuilder out(*plan, c.opt);
  char *host = static_cast<char *>(c.cpu_ptr);
  // Ascending file order is block-major when a block's layers lie inside its block
  // stride, (layer, kv)-major otherwise.
  const bool file_block_major = c.ssd_layer_stride < c.block_stride || c.num_layers <= 1;
  size_t i = 0;
  while (i < blks.size()) {
    size_t j = i;
    while (j < blks.size() && blks[j].device == blks[i].device && blks[j].file == blks[i].file)
      ++j;
    const int slot = blks[i].device * files_per_device + blks[i].file;
    const int fd = fds[slot], fallback = fallback_fds ? fallback_fds[slot] : -1;
    auto chunk_of = [&](const Blk &b, int l, int kv) {
      out.add(fd, fallback, b.in_file * c.block_stride + l * c.ssd_layer_stride + kv * c.ssd_kv_stride,
              host + b.cpu * c.block_stride + l * c.cpu_layer_stride + kv * c.cpu_kv_stride,
              c.chunk);
    };
    if (file_block_major) {
      for (size_t k = i; k < j; ++k)
        for (int l = c.start_layer; l < c.start_layer + c.num_layers; ++l)
          for (int kv = 0; kv < c.kv_dim; ++kv)
            chunk_of(blks[k], l, kv);
    } else {
      for (int l = c.start_layer; l < c.start_layer + c.num_layers; ++l)
        for (int kv = 0; kv < c.kv_dim; ++kv)
          for (size_t k = i; k < j; ++k)
            chunk_of(blks[k], l, kv);
    }
    i = j;
  }
}

// O_DIRECT needs every offset, address and length on a 4 KiB boundary
// (csrc/transfer_ssd.cpp:347-365).
bool direct_io_possible(const SsdCall &c) {
  const bool layer_strides_used = c.num_layers > 1 || c.start_layer > 0;
  return aligned4k((int64_t)(uintptr_t)c.cpu_ptr) && aligned4k(c.block_stride) &&
         aligned4k(c.chunk) &&
         (!layer_strides_used ||
          (aligned4k(c.cpu_layer_stride) && aligned4k(c.ssd_layer_stride))) &&
         (c.kv_dim == 1 || (aligned4k(c.cpu_kv_stride) && aligned4k(c.ssd_kv_stride)));
}

} // namespace

extern "C" {

int fkv_ssd_locate(int64_t ssd_block_id, int32_t round_robin, int32_t num_devices,
                   int32_t files_per_device, int32_t *device, int32_t *file, int64_t *block_in_file) try {
  fkv::clear_error();
  if (ssd_block_id < 0 || round_robin < 1 || num_devices < 1 || files_per_device < 1 || !device ||
      !file || !block_in_file)
    return fail(FKV_ERR_INVALID_ARG, "fkv_ssd_locate: bad arguments");
  const BlockPlace p = locate(ssd_block_id, round_robin, num_devices, files_per_device);
  *device = p.device;
  *file = p.file;
  *block_in_file = p.in_file;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_ssd_open(const char *const *paths, int32_t num_devices, int32_t files_per_device,
                 int32_t iouring_entries, int32_t iouring_flags, fkv_ssd_ctx **out) try {
  fkv::clear_error();
  if (!paths || !out || num_devices < 1 || files_per_device < 1)
    return fail(FKV_ERR_INVALID_ARG, "fkv_ssd_open: bad arguments");
  auto ctx = std::make_unique<fkv_ssd_ctx>();
  ctx->num_devices = num_devices;
  ctx->files_per_device = files_per_device;
  const int n = num_devices * files_per_device;
  ctx->fd_buffered.assign(n, -1);
  ctx->fd_direct.assign(n, -1);
  for (int i = 0; i < n; ++i) {
    ctx->fd_buffered[i] = open(paths[i], O_RDWR);
    if (ctx->fd_buffered[i] < 0) // csrc/transfer_ssd.h:263-270
      return fail(FKV_ERR_RUNTIME, "Failed to open file %s: %s", paths[i], std::strerror(errno));
    // Some file systems (tmpfs) have no O_DIRECT; those files are always buffered.
    ctx->fd_direct[i] = open(paths[i], O_RDWR | O_DIRECT);
    (void)posix_fadvise(ctx->fd_buffered[i], 0, 0, POSIX_FADV_SEQUENTIAL);
  }
  if (iouring_entries > 0) {
    ctx->ring = std::make_unique<Ring>(iouring_entries, (unsigned)iouring_flags);
    if (!ctx->ring->enabled()) {
      fprintf(stderr, "[fkv] io_uring unavailable (%s); SSD transfers use the thread engine\n",
              std::strerror(errno));
      ctx->ring.reset();
    }
  }
  // reads ahead of writes where the scheduler lets us (csrc/transfer_ssd.h:49-58)
  // (probe whether this thread may use the real-time class, then put back what it had)
  const long had = syscall(SYS_ioprio_get, 1, 0);
  const bool rt = syscall(SYS_ioprio_set, 1, 0, ioprio_value(kIoprioRT, 0)) == 0;
  if (rt)
    (void)syscall(SYS_ioprio_set, 1, 0, had >= 0 ? (int)had : 0);
  ctx->read_ioprio = rt ? ioprio_value(kIoprioRT, 0) : ioprio_value(kIoprioBE, 0);
  ctx->write_ioprio = ioprio_value(kIoprioBE, 4);
  *out = ctx.release();
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_ssd_uses_iouring(const fkv_ssd_ctx *ctx) { return ctx && ctx->ring ? 1 : 0; }

int fkv_ssd_last_direct(const fkv_ssd_ctx *ctx) { return ctx && ctx->last_direct.load() ? 1 : 0; }

void fkv_ssd_close(fkv_ssd_ctx *ctx) { delete ctx; }

int fkv_ssd_transfer(fkv_ssd_ctx *ctx, int32_t start_layer, int32_t num_layers, void *cpu_ptr,
                     const int64_t *ssd_block_ids, const int64_t *cpu_block_ids,
                     int32_t num_blocks, int64_t cpu_layer_stride, int64_t cpu_kv_stride,
                     int64_t ssd_layer_stride, int64_t ssd_kv_stride, int64_t chunk_size,
                     int64_t block_stride, int32_t is_read, int32_t round_robin,
                     int32_t num_threads_per_device, int32_t kv_dim, int32_t ssd_io_opt) try {
  fkv::clear_error();
  if (!ctx)
    return fail(FKV_ERR_INVALID_ARG, "fkv_ssd_transfer: null context");
  const SsdCall c{start_layer, num_layers, num_blocks, kv_dim, round_robin, cpu_ptr,
                  ssd_block_ids, cpu_block_ids, cpu_layer_stride, cpu_kv_stride,
                  ssd_layer_stride, ssd_kv_stride, chunk_size, block_stride, ssd_io_opt != 0};
  FKV_TRY(check_call(c));
  if (num_blocks == 0 || num_layers == 0)
    return FKV_OK;
  // the label of the reference's range, csrc/layerwise.cpp:1068-1073
  fkv::Range range("%s Blocks (%d blocks, %.2fMB each)", is_read ? "SSD->CPU" : "CPU->SSD",
                   num_blocks, (double)num_layers * kv_dim * chunk_size / (1024.0 * 1024.0));
  bool direct = direct_io_possible(c) &&
                ctx->no_direct_pool.load(std::memory_order_relaxed) != (uintptr_t)cpu_ptr;
  for (int fd : ctx->fd_direct)
    direct = direct && fd >= 0;
  Plan plan;
  build_plan(c, ctx->num_devices, ctx->files_per_device,
             (direct ? ctx->fd_direct : ctx->fd_buffered).data(),
             direct ? ctx->fd_buffered.data() : nullptr, &plan);
  split_for_parallelism(&plan, ctx->ring ? 16 : std::max(1, num_threads_per_device) *
                                                   ctx->num_devices);
  Outcome out;
  if (ctx->ring) {
    std::lock_guard<std::mutex> lk(ctx->ring_mu);
    ctx->ring->run(plan, is_read != 0, is_read ? ctx->read_ioprio : ctx->write_ioprio, !direct,
                   &out);
  } else {
    run_threads(plan, is_read != 0, std::max(1, num_threads_per_device) * ctx->num_devices,
                &out);
  }
  if (out.direct_refused.load())
    ctx->no_direct_pool.store((uintptr_t)cpu_ptr, std::memory_order_relaxed);
  ctx->last_direct = direct && !out.direct_refused.load();
  if (out.failed.load()) // csrc/transfer_ssd.cpp:497-499
    return fail(FKV_ERR_RUNTIME, "Failed to transfer data (%d of %zu %s requests: %s)",
                out.failed.load(), plan.requests.size(), is_read ? "read" : "write",
                std::strerror(out.err.load()));
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int64_t fkv_ssd_plan(int32_t num_devices, int32_t files_per_device, int32_t start_layer,
                     int32_t num_layers, const int64_t *ssd_block_ids,
                     const int64_t *cpu_block_ids, int32_t num_blocks, int64_t cpu_layer_stride,
                     int64_t cpu_kv_stride, int64_t ssd_layer_stride, int64_t ssd_kv_stride,
                     int64_t chunk_size, int64_t block_stride, int32_t round_robin,
                     int32_t kv_dim, int32_t ssd_io_opt, int64_t *out, int64_t capacity) {
  fkv::clear_error();
  if (num_devices < 1 || files_per_device < 1)
    return -1;
  // host addresses are reported as offsets from a base that is never touched
  char *const base = reinterpret_cast<char *>((uintptr_t)1 << 40);
  const SsdCall c{start_layer, num_layers, num_blocks, kv_dim, round_robin, base,
                  ssd_block_ids, cpu_block_ids, cpu_layer_stride, cpu_kv_stride,
                  ssd_layer_stride, ssd_kv_stride, chunk_size, block_stride, ssd_io_opt != 0};
  if (check_call(c) != FKV_OK)
    return -1;
  std::vector<int> fds(num_devices * files_per_device);
  for (size_t i = 0; i < fds.size(); ++i)
    fds[i] = (int)i; // the "descriptor" is device * files_per_device + file
  Plan plan;
  if (num_blocks > 0 && num_layers > 0)
    build_plan(c, num_devices, files_per_device, fds.data(), nullptr, &plan);
  int64_t rows = 0;
  for (const Request &r : plan.requests)
    for (uint32_t k = 0; k < r.iov_count; ++k, ++rows) {
      if (!out || rows >= capacity)
        continue;
      const iovec &v = plan.iovs[r.iov_first + k];
      int64_t *row = out + rows * 5;
      row[0] = &r - plan.requests.data();
      row[1] = r.fd;
      row[2] = r.file_off;
      row[3] = static_cast<char *>(v.iov_base) - base;
      row[4] = (int64_t)v.iov_len;
    }
  return rows;
}

} // extern "C"
