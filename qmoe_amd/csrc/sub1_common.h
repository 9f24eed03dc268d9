// Shared by the library's translation units: error reporting and bf16 helpers.
#ifndef SUB1_COMMON_H_
#define SUB1_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>

#include "sub1_hip.h"

namespace sub1 {

// Records the message for sub1_last_error() on this thread and returns `code`.
int fail(int code, const char *fmt, ...);

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// round-to-nearest-even (what __float2bfloat16 in the reference kernel does)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// res = min * s1 + max * s2 with one rounding of the product max * s2 and one of
// the fused sum; minmax holds (min, max) as two bf16.
__device__ __forceinline__ float row_result(uint32_t minmax, float s1, float s2) {
  float mn = __uint_as_float(minmax << 16);
  float mx = __uint_as_float(minmax & 0xffff0000u);
  return __fmaf_rn(mn, s1, __fmul_rn(mx, s2));
}

// Wait until this wavefront's own global stores have been acknowledged by L2.
// A workgroup barrier alone does not do that (the lanes of a workgroup share an
// L1, so workgroup scope needs no such wait), but a release at agent scope that
// ONE lane performs after the barrier writes back only what has reached L2.
__device__ __forceinline__ void drain_stores() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

inline bool misaligned(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0;
}

}  // namespace sub1

#define HIP_TRY(expr)                                                               \
  do {                                                                              \
    hipError_t e_ = (expr);                                                         \
    if (e_ != hipSuccess)                                                           \
      return sub1::fail(SUB1_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_));      \
  } while (0)

#endif  // SUB1_COMMON_H_
