// Which batches of a layerwise restore have had their events recorded.
//
// A restore whose rows host threads gather first is launched batch by batch from a
// thread of the library, so the event of a batch may not have been recorded yet when a
// consumer asks for it, and an event that was never recorded reads as complete.
// Everything that looks at a batch event goes through this gate first: the launching
// thread publishes how many batches it has recorded, or that it gave up; consumers
// block (or ask without blocking) until their batch is recorded or never will be.
// Free of any runtime call, so that it can be exercised without a device.
#pragma once

#include <atomic>
#include <condition_variable>
#include <mutex>

namespace fkv {

class BatchGate {
public:
  // A new restore: nothing recorded, not failed.  No consumer may be waiting.
  void reset() {
    std::lock_guard<std::mutex> lk(mu_);
    recorded_.store(0, std::memory_order_release);
    failed_ = false;
  }
  // The events of batches [0, n) have been recorded.
  void publish(int n) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      recorded_.store(n, std::memory_order_release);
    }
    cv_.notify_all();
  }
  // The launching thread gave up: batches from recorded() on never land.
  void fail() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      failed_ = true;
    }
    cv_.notify_all();
  }
  int recorded() const { return recorded_.load(std::memory_order_acquire); }
  // Blocks until the event of batch `b` has been recorded; false when it never will be.
  bool wait(int b) {
    if (b < recorded())
      return true;
    std::unique_lock<std::mutex> lk(mu_);
    cv_.wait(lk, [&] { return failed_ || b < recorded_.load(std::memory_order_relaxed); });
    return b < recorded_.load(std::memory_order_relaxed);
  }
  // Without blocking: 1 recorded, 0 not yet, -1 never.
  int peek(int b) {
    if (b < recorded())
      return 1;
    std::lock_guard<std::mutex> lk(mu_);
    if (b < recorded_.load(std::memory_order_relaxed))
      return 1;
    return failed_ ? -1 : 0;
  }
  // Only meaningful once the launching thread has ended.
  bool failed() {
    std::lock_guard<std::mutex> lk(mu_);
    return failed_;
  }
  void clear_failure() {
    std::lock_guard<std::mutex> lk(mu_);
    failed_ = false;
  }

private:
  std::mutex mu_;
  std::condition_variable cv_;
  std::atomic<int> recorded_{0};
  bool failed_ = false;
};

} // namespace fkv
