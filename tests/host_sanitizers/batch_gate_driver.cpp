// The gate between the thread that launches a gathered layerwise restore batch by batch
// and everything that looks at batch events (fkv_gate.h), together with the polling loop
// (fkv_poll.h): a scripted launcher publishes batches at its own pace and sometimes gives
// up part-way; waiters block on batches of their choice; a poller announces batches in
// order.  Nobody may see a batch as recorded before it was published, nobody may wait for
// good, and what is announced is exactly what was published.  No device, no runtime.
#include "fkv_gate.h"
#include "fkv_poll.h"

#include <chrono>
#include <cstdio>
#include <random>
#include <thread>
#include <vector>

namespace {
constexpr int kDone = 0, kNotReady = 600, kFault = 719;
int fail(const char *what, int rep) {
  fprintf(stderr, "batch gate, run %d: %s\n", rep, what);
  return 1;
}
} // namespace

int main() {
  std::mt19937 seed_rng(11);
  fkv::BatchGate gate; // one gate for all runs, reset in between, like a group's
  int runs = 0;
  for (int rep = 0; rep < 200; ++rep) {
    const int batches = 1 + (int)(seed_rng() % 12);
    const int gives_up_at = rep % 3 == 0 ? (int)(seed_rng() % batches) : -1; // before this batch
    const int published_in_the_end = gives_up_at < 0 ? batches : gives_up_at;
    const unsigned s0 = (unsigned)seed_rng();
    gate.reset();
    std::vector<std::atomic<int>> published(batches); // set by the launcher just before publish
    for (auto &p : published)
      p.store(0);
    std::atomic<int> errors{0};

    std::thread launcher([&] {
      std::mt19937 rng(s0);
      for (int b = 0; b < batches; ++b) {
        if (b == gives_up_at) {
          gate.fail();
          return;
        }
        if (rng() % 3 == 0)
          std::this_thread::sleep_for(std::chrono::microseconds(rng() % 200));
        published[b].store(1, std::memory_order_release); // "the event was recorded"
        gate.publish(b + 1);
      }
    });
    std::vector<std::thread> waiters;
    for (int w = 0; w < 4; ++w)
      waiters.emplace_back([&, w] {
        std::mt19937 rng(s0 + 17 * (w + 1));
        for (int k = 0; k < 6; ++k) {
          const int b = (int)(rng() % batches);
          const bool landed = gate.wait(b);
          if (landed != (b < published_in_the_end))
            errors.fetch_add(1);
          if (landed && !published[b].load(std::memory_order_acquire))
            errors.fetch_add(1); // seen as recorded before it was
        }
      });
    std::vector<int> announced;
    std::atomic<bool> stop{false};
    int status = kDone;
    std::thread poller([&] {
      status = fkv::poll_batches_in_order(
          (size_t)batches, 1, kDone, kNotReady,
          [&](size_t b, int) {
            const int state = gate.peek((int)b);
            if (state <= 0)
              return state < 0 ? kFault : kNotReady;
            if (!published[b].load(std::memory_order_acquire))
              errors.fetch_add(1);
            return kDone;
          },
          [&](size_t b) { announced.push_back((int)b); }, stop);
    });
    launcher.join();
    for (auto &t : waiters)
      t.join();
    poller.join();
    if (errors.load())
      return fail("a waiter or the poller saw a wrong state", rep);
    if ((int)announced.size() != published_in_the_end)
      return fail("announced batches differ from published ones", rep);
    for (int i = 0; i < (int)announced.size(); ++i)
      if (announced[i] != i)
        return fail("announced out of order", rep);
    if (status != (gives_up_at < 0 ? kDone : kFault))
      return fail("wrong final status of the poller", rep);
    if (gate.failed() != (gives_up_at >= 0) || gate.recorded() != published_in_the_end)
      return fail("wrong final state of the gate", rep);
    ++runs;
  }
  printf("ok: %d scripted restores through the gate\n", runs);
  return 0;
}
