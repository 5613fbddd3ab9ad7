// Thin C-ABI over the HIP runtime calls the host API needs
// (include/iris_amd.h); takes the place of the ctypes bindings of
// iris/_hip.py.  Every function returns the hipError_t of the call it wraps.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

#include "common.hpp"

namespace iris_amd {

int current_cu_count() {
  static int cached[64] = {};
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] > 0) return cached[dev];
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
  cached[dev] = cus;
  return cus;
}

}  // namespace iris_amd

extern "C" {

const char* iris_hip_error_string(int err) { return hipGetErrorString(static_cast<hipError_t>(err)); }

int iris_hip_device_count(int* count) { return hipGetDeviceCount(count); }

int iris_hip_set_device(int device) { return hipSetDevice(device); }

int iris_hip_get_device(int* device) { return hipGetDevice(device); }

int iris_hip_cu_count(int device, int* cu_count) {
  return hipDeviceGetAttribute(cu_count, hipDeviceAttributeMultiprocessorCount, device);
}

int iris_hip_wall_clock_rate(int device, int* khz) {
  return hipDeviceGetAttribute(khz, hipDeviceAttributeWallClockRate, device);
}

int iris_hip_malloc_finegrained(void** ptr, size_t size) {
  return hipExtMallocWithFlags(ptr, size, hipDeviceMallocFinegrained);
}

int iris_hip_malloc(void** ptr, size_t size) { return hipMalloc(ptr, size); }

int iris_hip_free(void* ptr) { return hipFree(ptr); }

int iris_hip_ipc_get_handle(void* handle64, void* ptr) {
  static_assert(sizeof(hipIpcMemHandle_t) == 64, "IPC handle size");
  hipIpcMemHandle_t h;
  const hipError_t err = hipIpcGetMemHandle(&h, ptr);
  if (err == hipSuccess) std::memcpy(handle64, &h, sizeof(h));
  return err;
}

int iris_hip_ipc_open_handle(void** ptr, const void* handle64) {
  hipIpcMemHandle_t h;
  std::memcpy(&h, handle64, sizeof(h));
  return hipIpcOpenMemHandle(ptr, h, hipIpcMemLazyEnablePeerAccess);
}

int iris_hip_device_synchronize(void) { return hipDeviceSynchronize(); }

int iris_hip_arch_name(int device, char* buf, size_t len) {
  if (!buf || len == 0) return hipErrorInvalidValue;
  hipDeviceProp_t prop;
  const hipError_t err = hipGetDeviceProperties(&prop, device);
  if (err != hipSuccess) return err;
  std::snprintf(buf, len, "%s", prop.gcnArchName);
  return hipSuccess;
}

int iris_amd_abi_version(void) { return 5; }

}  // extern "C"
