// Version and error strings of the C ABI.
#include <hip/hip_runtime.h>

#include "slora_hip.h"

extern "C" {

int slora_version(void) { return SLORA_VERSION; }

const char* slora_strerror(int code) {
  switch (code) {
    case SLORA_OK: return "ok";
    case SLORA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case SLORA_ERR_BAD_DTYPE: return "dtype must be fp16 or bf16 (scales: fp16, bf16 or fp32)";
    case SLORA_ERR_BAD_SHAPE: return "negative size, qkvo outside 0..3 or a stride smaller than the row";
    case SLORA_ERR_UNSUPPORTED: return "No suitable kernel.";
    case SLORA_ERR_ALIGNMENT: return "buffer is not 16-byte aligned";
    case SLORA_ERR_LAUNCH: return "HIP kernel launch failed";
    case SLORA_ERR_TOO_LARGE: return "size exceeds the fixed capacity of this entry point (see its maximum in slora_hip.h)";
    default: return "unknown error";
  }
}

int slora_plan_status(const void* plan, int* status, void* stream) {
  if (plan == nullptr || status == nullptr) return SLORA_ERR_NULL_POINTER;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // word 7 of both plan headers
  if (hipMemcpyAsync(status, static_cast<const int*>(plan) + 7, sizeof(int), hipMemcpyDeviceToHost, s) != hipSuccess ||
      hipStreamSynchronize(s) != hipSuccess) {
    (void)hipGetLastError();
    return SLORA_ERR_LAUNCH;
  }
  return SLORA_OK;
}

}  // extern "C"
