// Sharing an engine's KV tensors with a transfer worker in another process.
//
// Counterpart of the direct-IPC branch of TensorSharedHandle in the reference
// (flexkv/common/memory_handle.py:1144-1250): the owner exports the handle of
// the allocation a tensor lives in plus the tensor's offset inside it, the
// worker opens the handle once per process and addresses base + offset.
// A handle is opened at most once per process (a second open of the same
// allocation is an error in the runtime), so opens are cached and counted.
#include "fkv_internal.h"

#include <cstring>
#include <map>
#include <mutex>
#include <string>

namespace {

struct Mapping {
  void *base = nullptr;
  int device = 0;
  int refs = 0;
};

std::mutex g_mu;
std::map<std::string, Mapping> g_open; // by the 64 handle bytes + device

std::string key_of(const uint8_t *handle, int device) {
  std::string k(reinterpret_cast<const char *>(handle), FKV_IPC_HANDLE_BYTES);
  k.push_back((char)device);
  return k;
}

} // namespace

extern "C" {

int fkv_ipc_export(const void *device_ptr, uint8_t *handle_out, int64_t *offset_out,
                   int64_t *allocation_bytes_out) try {
  using namespace fkv;
  clear_error();
  if (!device_ptr || !handle_out || !offset_out)
    return fail(FKV_ERR_INVALID_ARG, "fkv_ipc_export: null argument");
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  FKV_HIP_TRY(hipMemGetAddressRange(&base, &size, const_cast<void *>(device_ptr)));
  hipIpcMemHandle_t h;
  static_assert(sizeof(h) == FKV_IPC_HANDLE_BYTES, "hipIpcMemHandle_t is 64 bytes");
  FKV_HIP_TRY(hipIpcGetMemHandle(&h, base));
  std::memcpy(handle_out, &h, sizeof(h));
  *offset_out = (int64_t)((const uint8_t *)device_ptr - (const uint8_t *)base);
  if (allocation_bytes_out)
    *allocation_bytes_out = (int64_t)size;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_ipc_open(const uint8_t *handle, int32_t device, void **base_out) try {
  using namespace fkv;
  clear_error();
  if (!handle || !base_out)
    return fail(FKV_ERR_INVALID_ARG, "fkv_ipc_open: null argument");
  DeviceGuard guard(device);
  int dev = 0;
  FKV_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mu);
  Mapping &m = g_open[key_of(handle, dev)];
  if (m.refs == 0) {
    hipIpcMemHandle_t h;
    std::memcpy(&h, handle, sizeof(h));
    void *base = nullptr;
    hipError_t e = hipIpcOpenMemHandle(&base, h, hipIpcMemLazyEnablePeerAccess);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      g_open.erase(key_of(handle, dev));
      return fail(FKV_ERR_RUNTIME, "hipIpcOpenMemHandle failed on device %d: %s", dev,
                  hipGetErrorString(e));
    }
    m.base = base;
    m.device = dev;
  }
  ++m.refs;
  *base_out = m.base;
  return FKV_OK;
} catch (...) {
  return fkv::caught(__func__);
}

int fkv_ipc_close(void *base) try {
  using namespace fkv;
  clear_error();
  if (!base)
    return FKV_OK;
  std::lock_guard<std::mutex> lock(g_mu);
  for (auto it = g_open.begin(); it != g_open.end(); ++it) {
    if (it->second.base != base)
      continue;
    if (--it->second.refs > 0)
      return FKV_OK;
    DeviceGuard guard(it->second.device);
    hipError_t e = hipIpcCloseMemHandle(base);
    g_open.erase(it);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(FKV_ERR_RUNTIME, "hipIpcCloseMemHandle failed: %s", hipGetErrorString(e));
    }
    return FKV_OK;
  }
  return fail(FKV_ERR_INVALID_ARG, "fkv_ipc_close: %p was not opened by fkv_ipc_open", base);
} catch (...) {
  return fkv::caught(__func__);
}

} // extern "C"
