// Device helpers shared by the decode (BGMV) and prefill (segmented GEMM)
// kernels.  gfx950 only: 64-lane wavefronts, DPP row operations, 16-byte
// global loads.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "slora_hip.h"

namespace slora {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---- storage types ---------------------------------------------------------
// A storage type turns one 32-bit word holding two 16-bit elements into two
// floats, and rounds a float back to 16 bits (round-to-nearest-even).
struct F16 {
  static __device__ __forceinline__ float lo(uint32_t v) { return (float)__builtin_bit_cast(f16x2, v).x; }
  static __device__ __forceinline__ float hi(uint32_t v) { return (float)__builtin_bit_cast(f16x2, v).y; }
  static __device__ __forceinline__ float to_float(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
  // c + a.lo*b.lo + a.hi*b.hi in float, straight from the packed words (v_dot2_f32_f16)
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  }
  // y + d with both operands of the storage type, one rounding
  static __device__ __forceinline__ uint16_t add(uint16_t y, uint16_t d) {
    _Float16 s = __builtin_bit_cast(_Float16, y) + __builtin_bit_cast(_Float16, d);
    return __builtin_bit_cast(uint16_t, s);
  }
  // the same on both halves of a packed word (v_pk_add_f16)
  static __device__ __forceinline__ uint32_t add2(uint32_t y, uint32_t d) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, y) + __builtin_bit_cast(f16x2, d));
  }
};

struct BF16 {
  static __device__ __forceinline__ float lo(uint32_t v) { return __uint_as_float(v << 16); }
  static __device__ __forceinline__ float hi(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
  static __device__ __forceinline__ float to_float(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
  // v_dot2_f32_bf16
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
  static __device__ __forceinline__ uint16_t add(uint16_t y, uint16_t d) {
    // the sum of two bf16 values is exact in float unless their exponents are
    // more than 16 apart, where the smaller one cannot move the rounding
    return from_float(to_float(y) + to_float(d));
  }
  static __device__ __forceinline__ uint32_t add2(uint32_t y, uint32_t d) {
    return (uint32_t)add((uint16_t)(y & 0xffffu), (uint16_t)(d & 0xffffu)) |
           ((uint32_t)add((uint16_t)(y >> 16), (uint16_t)(d >> 16)) << 16);
  }
};

// scale table element -> float, in the table's own type
__device__ __forceinline__ float load_scale(const void* scales, int scales_dtype, int64_t a) {
  if (scales_dtype == SLORA_DTYPE_F32) return ((const float*)scales)[a];
  uint16_t v = ((const uint16_t*)scales)[a];
  return scales_dtype == SLORA_DTYPE_F16 ? F16::to_float(v) : BF16::to_float(v);
}

// ---- 16-byte accesses ------------------------------------------------------
__device__ __forceinline__ u32x4 ldg16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
// 16 bytes that this launch reads once (weight pages) or reads and writes once (outputs):
// nontemporal, so they do not push reused lines (activations, tables) out of the caches.
__device__ __forceinline__ u32x4 ldg16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void stg16_stream(void* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x4 zero16() { return u32x4{0u, 0u, 0u, 0u}; }

// Values one workgroup writes and another workgroup of the SAME launch reads (the shrink
// results that the expand half of a one-launch LoRA consumes): relaxed atomics at device
// scope, which go through to the level every XCD sees instead of a line that one XCD's L2
// or a compute unit's vector cache may still hold.  Between launches plain accesses do.
__device__ __forceinline__ u32x4 ldg16_coherent(const void* p) {
  const uint64_t* q = reinterpret_cast<const uint64_t*>(p);
  const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return u32x4{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
}
__device__ __forceinline__ uint16_t ld16_coherent(const uint16_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st16_coherent(uint16_t* p, uint16_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// acc += sum_i f32(w_i) * f32(x_i) over the 8 elements of two 16-byte vectors
template <typename T>
__device__ __forceinline__ float dot8(u32x4 w, u32x4 x, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = T::dot2(w[i], x[i], acc);
  return acc;
}

// ---- cross-lane sums -------------------------------------------------------
// DPP controls: quad_perm(a,b,c,d) = a | b<<2 | c<<4 | d<<6; 0x141 = row_half_mirror,
// 0x140 = row_mirror.  After xor-1 and xor-2 every quad is uniform, so the two
// mirrors act as xor-4 and xor-8.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
  return v + __int_as_float(o);
}

// Sum over aligned groups of G lanes (G a power of two <= 64); every lane of
// a group ends up holding the group's sum.
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  if (G >= 2) v = dpp_add<0xB1>(v);   // quad_perm(1,0,3,2)
  if (G >= 4) v = dpp_add<0x4E>(v);   // quad_perm(2,3,0,1)
  if (G >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
  if (G >= 16) v = dpp_add<0x140>(v); // row_mirror
  if (G >= 32) v += __shfl_xor(v, 16, 64);
  if (G >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// Sum over the whole wavefront, result valid in every lane.
__device__ __forceinline__ float wave_sum(float v) {
  v = group_sum<16>(v);
  int iv = __float_as_int(v);
  float a = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
  return (a + b) + (c + d);
}

}  // namespace slora
