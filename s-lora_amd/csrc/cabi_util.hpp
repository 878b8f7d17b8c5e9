// Host-side helpers of the C ABI.
#pragma once

#include <stdint.h>

namespace slora {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace slora
