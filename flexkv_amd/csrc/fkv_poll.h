// The loop of the layerwise restore's polling thread, free of any runtime call so
// that it can be exercised without a device: announce batches in order as all GPUs
// finish them; stop, without announcing what is left, at the first status that is
// neither "done" nor "not yet".  (csrc/layerwise.cpp:36-68 polls cudaEventQuery the
// same way but treats every error as "not yet" and spins.)
#pragma once

#include <atomic>
#include <cstddef>
#include <thread>

namespace fkv {

// `query(batch, gpu)` returns `done`, `not_ready`, or any other value = a device error.
// Returns `done` when every batch was announced or the loop was told to stop, else the
// error that ended it.  `announced` (optional) receives the number of batches announced.
template <class Query, class Notify>
int poll_batches_in_order(size_t num_batches, int num_gpus, int done, int not_ready, Query query,
                          Notify notify, const std::atomic<bool> &stop,
                          size_t *announced = nullptr) {
  size_t next = 0;
  int result = done;
  while (result == done && next < num_batches && !stop.load(std::memory_order_acquire)) {
    bool all = true;
    for (int g = 0; g < num_gpus && all; ++g) {
      const int status = query(next, g);
      if (status == done)
        continue;
      all = false;
      if (status != not_ready)
        result = status; // the batches behind a failed one will never land
    }
    if (result != done)
      break;
    if (all) {
      notify(next);
      ++next;
    } else {
      std::this_thread::yield();
    }
  }
  if (announced)
    *announced = next;
  return result;
}

} // namespace fkv
