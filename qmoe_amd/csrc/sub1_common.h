// Shared by the library's translation units: error reporting and bf16 helpers.
#ifndef SUB1_COMMON_H_
#define SUB1_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>

#include "sub1_hip.h"

namespace sub1 {

// Records the message for sub1_last_error() on this thread and returns `code`.
int fail(int code, const char *fmt, ...);

// Records which kernel the calling thread's entry point launched last
// (sub1_last_kernel()); `name` is a string literal.
void note_kernel(const char *name);

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

// Sticky fault flags.  A kernel whose bounded wait gives up, or that finds the
// caller's dec changed under a table derived from it, cannot return an error;
// it sets a word in pinned host memory instead, which no launch ever clears
// and which the host reads without synchronising (sub1_fault_flags).
constexpr int kFaultWait = 0;   // a wait between workgroups reached its time limit: wrong output
constexpr int kFaultDec = 1;    // dec no longer holds what the cached table was derived from
constexpr int kFaultWords = 4;

// Device-visible address of the flag words; allocates them (pinned host
// memory, once per process) unless may_allocate is false, in which case a
// missing allocation is an error.
int fault_words(int32_t **device_ptr, bool may_allocate);
// The flag as the host sees it now (false while the words do not exist).
bool fault_flag_host(int word);

// Longest wait between workgroups, in ticks of the device's constant-rate
// clock (wall_clock64), and how much the tests overstate the count a wait
// expects (0 outside tests).
int64_t wait_limit_ticks();
int expect_extra();

__device__ __forceinline__ void raise_fault(int32_t *sticky, int word) {
  __hip_atomic_store(&sticky[word], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Thread 0's bounded wait until *counter reaches `expect`: relaxed looks at
// agent scope, the clock read every 16th look, one acquire at the end.  On
// time-out the wait-fault flag is set, *gave_up (the launch's own count) goes
// up by one and the caller carries on (its output
// is then wrong, but every access stays inside the caller's buffers and the
// kernel exits).
__device__ __forceinline__ void bounded_wait(const int32_t *counter, int expect,
                                             int64_t limit_ticks, int32_t *sticky,
                                             int32_t *gave_up) {
  int looks = 0;
  int64_t t0 = 0;
  while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < expect) {
    if ((++looks & 15) == 1) {
      const int64_t now = static_cast<int64_t>(wall_clock64());
      if (looks == 1) t0 = now;
      if (now - t0 > limit_ticks) {
        raise_fault(sticky, kFaultWait);
        __hip_atomic_fetch_add(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
    __builtin_amdgcn_s_sleep(2);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

}  // namespace sub1

#define HIP_TRY(expr)                                                               \
  do {                                                                              \
    hipError_t e_ = (expr);                                                         \
    if (e_ != hipSuccess)                                                           \
      return sub1::fail(SUB1_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_));      \
  } while (0)

#endif  // SUB1_COMMON_H_
