// A CPU model of the device side of HIP, for sanitizer builds of the library's kernel
// sources: with this header included first, a .hip file compiles as ordinary C++, and a
// kernel launch runs the kernel's own code on the emulated stream's thread, one workgroup
// after the other, every work-item of a workgroup on a host thread of its own and
// __syncthreads() a barrier among them.  AddressSanitizer then checks every address the
// kernel computes (tables, id lists, both ends of every copy), ThreadSanitizer the order
// between work-items that the barriers and atomics establish, and the launch shaping on
// the host runs as it does in the product.  Test infrastructure (emulated_hip_runtime.cpp
// holds the implementation); nothing here is fast.
//
// What the model does not have: wavefronts (no cross-lane operations; the kernels here use
// none), more than one workgroup in flight (a workgroup never waits for another one in
// these kernels: the safety net of a confined launch only looks at a counter for a bounded
// time), memory that is not coherent.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <functional>

namespace cpu_device_model {
struct Index {
  unsigned x = 0, y = 0, z = 0;
};
struct Extent {
  unsigned x = 1, y = 1, z = 1;
};
extern thread_local Index thread_index, block_index;
extern thread_local Extent block_extent, grid_extent;

void sync_threads();
// The launch's dynamically sized LDS, one array per workgroup, zeroed never (as on the device).
void *dynamic_lds();
// XCDs take the workgroups of a launch in turn; which one takes workgroup 0 changes
// from launch to launch.
unsigned xcc_id();
void nap();
inline long long wall_clock_ticks() { // the device's constant 100 MHz clock
  return std::chrono::duration_cast<std::chrono::nanoseconds>(
             std::chrono::steady_clock::now().time_since_epoch())
             .count() /
         10;
}
void launch(hipStream_t stream, dim3 grid, dim3 block, size_t lds_bytes, std::function<void()> work_item);
} // namespace cpu_device_model

#undef __shared__
#define __shared__ static // one workgroup at a time
#ifndef __launch_bounds__
#define __launch_bounds__(...)
#endif
#ifndef __align__
#define __align__(n) __attribute__((aligned(n)))
#endif
#ifndef HIP_SYMBOL
#define HIP_SYMBOL(variable) variable // a __device__ variable is a variable of this process
#endif
#define threadIdx cpu_device_model::thread_index
#define blockIdx cpu_device_model::block_index
#define blockDim cpu_device_model::block_extent
#define gridDim cpu_device_model::grid_extent
#define __syncthreads() cpu_device_model::sync_threads()
#define wall_clock64() cpu_device_model::wall_clock_ticks()
#define __builtin_amdgcn_s_sleep(n) cpu_device_model::nap()
#ifndef __HIP_MEMORY_SCOPE_AGENT
#define __HIP_MEMORY_SCOPE_AGENT 4
#endif
#define __hip_atomic_load(pointer, order, scope) __atomic_load_n(pointer, order)
#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, ...)                             \
  cpu_device_model::launch(stream, grid, block, lds_bytes, [=] { (kernel)(__VA_ARGS__); })

template <typename T, typename U> inline T atomicAdd(T *p, U v) {
  return __atomic_fetch_add(p, (T)v, __ATOMIC_RELAXED);
}
template <typename T, typename U> inline T atomicOr(T *p, U v) {
  return __atomic_fetch_or(p, (T)v, __ATOMIC_RELAXED);
}
template <typename T> inline T atomicCAS(T *p, T expected, T desired) {
  __atomic_compare_exchange_n(p, &expected, desired, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED);
  return expected; // what was there
}
using std::max;
using std::min;
