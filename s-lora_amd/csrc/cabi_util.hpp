// Host-side helpers of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace slora {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Raises a kernel's dynamic shared memory limit once per device: a function attribute belongs
// to the device that was current when it was set.  `done` is the call site's own table (one
// flag per device id; ids beyond it set the attribute on every call).  Benign if two threads
// race: the call is idempotent.
struct PerDeviceOnce {
  bool done[64] = {};
};
inline bool raise_dynamic_lds(const void* kernel, int bytes, PerDeviceOnce& once) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const bool remember = dev >= 0 && dev < 64;
  if (remember && once.done[dev]) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (remember) once.done[dev] = true;
  return true;
}

}  // namespace slora
