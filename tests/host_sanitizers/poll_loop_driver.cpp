// The polling loop of the layerwise restore on scripted event statuses: batches are
// announced in order and only when every GPU has finished them; a status that is neither
// "done" nor "not yet" ends the loop without announcing what is left; a stop request ends
// it too.  No device, no runtime.
#include "fkv_poll.h"

#include <cstdio>
#include <random>
#include <vector>

namespace {
constexpr int kDone = 0, kNotReady = 600, kFault = 719;
int fail(const char *what) {
  fprintf(stderr, "poll loop: %s\n", what);
  return 1;
}
} // namespace

int main() {
  std::mt19937 rng(5);
  int runs = 0;
  for (int rep = 0; rep < 300; ++rep) {
    const int batches = 1 + (int)(rng() % 9), gpus = 1 + (int)(rng() % 3);
    // ready_after[b][g]: queries of (b, g) that say "not yet" before it says "done"
    std::vector<std::vector<int>> ready_after(batches, std::vector<int>(gpus));
    for (auto &b : ready_after)
      for (int &x : b)
        x = (int)(rng() % 4);
    const int fault_batch = rep % 3 == 0 ? (int)(rng() % batches) : -1;
    const int fault_gpu = (int)(rng() % gpus);
    std::vector<int> announced_order;
    std::atomic<bool> stop{false};
    size_t announced = 0;
    const int status = fkv::poll_batches_in_order(
        (size_t)batches, gpus, kDone, kNotReady,
        [&](size_t b, int g) {
          if ((int)b == fault_batch && g == fault_gpu && ready_after[b][g]-- <= 0)
            return kFault;
          if ((int)b == fault_batch && g == fault_gpu)
            return kNotReady;
          if (ready_after[b][g] > 0) {
            --ready_after[b][g];
            return kNotReady;
          }
          // a batch is only ever asked about once everything before it was announced
          if (announced_order.size() != b)
            return -1;
          return kDone;
        },
        [&](size_t b) { announced_order.push_back((int)b); }, stop, &announced);
    const int want = fault_batch < 0 ? batches : fault_batch;
    if (status != (fault_batch < 0 ? kDone : kFault))
      return fail("wrong final status");
    if ((int)announced != want || (int)announced_order.size() != want)
      return fail("wrong number of batches announced");
    for (int i = 0; i < want; ++i)
      if (announced_order[i] != i)
        return fail("batches announced out of order");
    ++runs;
  }
  // a stop request ends a loop whose batch never becomes ready
  {
    std::atomic<bool> stop{false};
    int queries = 0;
    size_t announced = 7;
    const int status = fkv::poll_batches_in_order(
        3, 1, kDone, kNotReady,
        [&](size_t, int) {
          if (++queries == 50)
            stop.store(true);
          return kNotReady;
        },
        [&](size_t) {}, stop, &announced);
    if (status != kDone || announced != 0 || queries != 50)
      return fail("stop request");
    ++runs;
  }
  printf("ok: %d scripted polls\n", runs);
  return 0;
}
