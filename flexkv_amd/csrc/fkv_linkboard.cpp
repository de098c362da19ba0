// Link activity shared between the processes that use one GPU.
//
// The arbiter of fkv_core.cpp keeps a put and a get that run at the same time on
// different XCDs, but it only sees the launches of its own process.  Serving
// stacks put the two directions into different processes (a worker for puts, a
// layerwise worker for restores), so every process also posts, per direction,
// until when it expects the link to be busy with its launches, on a small board
// in /dev/shm named after the user and the GPU's PCI address.  A launch asks the
// board whether another process has posted activity of the other direction.
// Times are CLOCK_MONOTONIC, which all processes of a host share.  A board that
// cannot be opened (no /dev/shm, FKV_LINK_BOARD=0) means: nobody else is there.
#include "fkv_internal.h"

#include <cctype>
#include <cerrno>
#include <csignal>
#include <cstdlib>
#include <cstring>
#include <fcntl.h>
#include <map>
#include <mutex>
#include <sys/mman.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

namespace fkv {
namespace {

constexpr uint32_t kBoardMagic = 0x464b4c42; // "FKLB"
constexpr int kBoardSlots = 32;

struct BoardSlot {
  std::atomic<int32_t> pid;
  int32_t pad;
  std::atomic<int64_t> busy_until_ns[2]; // [0] GPU->host, [1] host->GPU
};
struct Board {
  std::atomic<uint32_t> magic;
  uint32_t pad;
  BoardSlot slot[kBoardSlots];
};
static_assert(std::atomic<int64_t>::is_always_lock_free, "board needs lock-free 64-bit atomics");

int64_t monotonic_ns() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000000ll + ts.tv_nsec;
}

struct BoardHandle {
  Board *board = nullptr;
  int slot = -1;       // this process's slot, -1 when none was free
  int32_t owner = 0;   // pid that claimed the slot (a forked child claims its own)
};

bool pid_is_gone(int32_t pid) { return pid > 0 && kill(pid, 0) == -1 && errno == ESRCH; }

void claim_slot(BoardHandle &h) {
  const int32_t me = (int32_t)getpid();
  h.owner = me;
  h.slot = -1;
  for (int i = 0; i < kBoardSlots; ++i)
    if (h.board->slot[i].pid.load(std::memory_order_relaxed) == me) {
      h.slot = i;
      return;
    }
  for (int i = 0; i < kBoardSlots; ++i) {
    BoardSlot &s = h.board->slot[i];
    int32_t cur = s.pid.load(std::memory_order_relaxed);
    if (cur != 0 && !pid_is_gone(cur))
      continue;
    if (s.pid.compare_exchange_strong(cur, me, std::memory_order_acq_rel)) {
      s.busy_until_ns[0].store(0, std::memory_order_relaxed);
      s.busy_until_ns[1].store(0, std::memory_order_relaxed);
      h.slot = i;
      return;
    }
  }
}

BoardHandle open_board(const std::string &key) {
  BoardHandle h;
  std::string name = "/dev/shm/fkv_link_" + std::to_string((unsigned)getuid()) + "_";
  for (char c : key)
    name += (std::isalnum((unsigned char)c) ? c : '_');
  // The path is predictable: never follow a link planted there, and use the file
  // only if it is a regular file of this user that is empty (new) or a board already.
  int fd = open(name.c_str(), O_RDWR | O_CREAT | O_CLOEXEC | O_NOFOLLOW, 0600);
  if (fd < 0)
    return h;
  struct stat st;
  if (fstat(fd, &st) != 0 || !S_ISREG(st.st_mode) || st.st_uid != getuid() ||
      (st.st_size != 0 && st.st_size != (off_t)sizeof(Board))) {
    close(fd);
    return h;
  }
  const bool fresh = st.st_size == 0;
  if (fresh && ftruncate(fd, sizeof(Board)) != 0) {
    close(fd);
    return h;
  }
  void *p = mmap(nullptr, sizeof(Board), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (p == MAP_FAILED)
    return h;
  Board *b = static_cast<Board *>(p); // a fresh file is all zeroes: no slot taken
  // Whoever finds the magic absent writes it (a process that created the file at the
  // same moment does the same); any other content is not a board and is left alone.
  uint32_t expect = 0;
  if (!b->magic.compare_exchange_strong(expect, kBoardMagic, std::memory_order_acq_rel) &&
      expect != kBoardMagic) {
    munmap(p, sizeof(Board));
    return h;
  }
  h.board = b;
  claim_slot(h);
  return h;
}

// Key of the board of `device`: FKV_LINK_BOARD_KEY when set (tests, or engines that
// address one GPU through different device numbers), else the PCI address.
bool board_key(int device, std::string *key) {
  if (const char *k = std::getenv("FKV_LINK_BOARD_KEY")) {
    if (*k) {
      *key = std::string(k) + "_" + std::to_string(device);
      return true;
    }
  }
  char bus[64] = {0};
  if (hipDeviceGetPCIBusId(bus, (int)sizeof(bus), device) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  *key = bus;
  return true;
}

BoardHandle *board_of(int device) {
  static const bool enabled = [] {
    const char *v = std::getenv("FKV_LINK_BOARD");
    return !(v && !std::strcmp(v, "0"));
  }();
  if (!enabled)
    return nullptr;
  static std::mutex mu;
  static std::map<int, BoardHandle *> all; // live until the process ends
  std::lock_guard<std::mutex> lk(mu);
  auto it = all.find(device);
  if (it == all.end()) {
    std::string key;
    BoardHandle *h = new BoardHandle();
    if (board_key(device, &key))
      *h = open_board(key);
    it = all.emplace(device, h).first;
  }
  BoardHandle *h = it->second;
  if (!h->board)
    return nullptr;
  if (h->owner != (int32_t)getpid())
    claim_slot(*h);
  return h;
}

} // namespace

void link_board_post(int device, bool h2d, int64_t expected_ns) {
  BoardHandle *h = board_of(device);
  if (!h || h->slot < 0)
    return;
  std::atomic<int64_t> &until = h->board->slot[h->slot].busy_until_ns[h2d ? 1 : 0];
  const int64_t now = monotonic_ns();
  // launches queue up behind each other: the new one ends after the posted ones
  const int64_t prev = until.load(std::memory_order_relaxed);
  until.store((prev > now ? prev : now) + (expected_ns > 0 ? expected_ns : 0),
              std::memory_order_relaxed);
}

bool link_board_busy_elsewhere(int device, bool h2d, int64_t window_ns) {
  BoardHandle *h = board_of(device);
  if (!h)
    return false;
  const int32_t me = (int32_t)getpid();
  const int64_t now = monotonic_ns();
  for (int i = 0; i < kBoardSlots; ++i) {
    const BoardSlot &s = h->board->slot[i];
    const int32_t pid = s.pid.load(std::memory_order_relaxed);
    if (pid == 0 || pid == me)
      continue;
    const int64_t until = s.busy_until_ns[h2d ? 1 : 0].load(std::memory_order_relaxed);
    // an entry far in the future is a leftover of a crashed run or a foreign clock
    if (until && now < until + window_ns && until - now < 60ll * 1000000000ll)
      return true;
  }
  return false;
}

namespace {
int resolve_device(int32_t device) {
  if (device >= 0)
    return device;
  int cur = 0;
  if (hipGetDevice(&cur) != hipSuccess) {
    (void)hipGetLastError();
    cur = 0;
  }
  return cur;
}
} // namespace

} // namespace fkv

extern "C" int fkv_link_activity_post(int32_t device, int32_t is_host_to_device,
                                      int64_t expected_us) try {
  using namespace fkv;
  clear_error();
  if (expected_us < 0)
    return fail(FKV_ERR_INVALID_ARG, "fkv_link_activity_post: negative duration");
  link_board_post(resolve_device(device), is_host_to_device != 0, expected_us * 1000);
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

extern "C" int fkv_link_activity_elsewhere(int32_t device, int32_t is_host_to_device,
                                           int32_t window_ms, int32_t *busy) try {
  using namespace fkv;
  clear_error();
  if (!busy)
    return fail(FKV_ERR_INVALID_ARG, "fkv_link_activity_elsewhere: null result pointer");
  *busy = link_board_busy_elsewhere(resolve_device(device), is_host_to_device != 0,
                                    (int64_t)(window_ms < 0 ? 0 : window_ms) * 1000000)
              ? 1
              : 0;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}
