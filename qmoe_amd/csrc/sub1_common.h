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

// Control words at the head of an expert launch's workspace.  The caller zeroes
// the workspace once; every launch leaves the words it counts with at zero
// again (the last workgroup out clears the ticket, the last workgroup that
// waited on a token's word clears that word), so a launch is one kernel and
// needs no clearing kernel before it.  Words 1 and 2 only ever grow.
constexpr int kCtrlTicket = 0;     // tiles handed out
constexpr int kCtrlGaveUp = 1;     // waits that reached their time limit, all launches so far
constexpr int kCtrlBadIds = 2;     // tokens whose expert id was >= experts, all launches so far
constexpr int kCtrlTiles = 3;      // tiles of a launch with tokens grouped by expert
constexpr int kCtrlExits = 4;      // workgroups of a persistent launch that have left
constexpr int kCtrlLaunch = 6;     // and 7, one 64-bit count: launches that handed h over by tag
// Words 64 on: the tagged copy of h, for launches of a token or two whose
// workgroups hand h over without counting.  An entry is 64 bits, a bf16 value
// under a 48-bit tag, written and read as one word: the tag is the number of
// such launches on this workspace so far plus one, so an entry that carries it
// was written by this launch (zeroed memory carries none), and nothing has to
// be cleared, counted or fenced.  Only those launches touch the region, and it
// lies at the same place whatever the batch.
constexpr int kTaggedTokens = 2;
constexpr int kCtrlTagged = 64;
constexpr int kTaggedWidth = 12288;   // entries per token: the widest h of a prepared stack
constexpr int kCtrlHeader = kCtrlTagged + kTaggedTokens * kTaggedWidth * 2;   // then one word per token:
// low half: workgroups that have written their part of the token's h;
// high half: workgroups that have waited for it (the last of them clears the word).
// The words lie 64 bytes apart: every workgroup of a token adds to its word and
// polls it, and words that share a 64-byte sector queue behind each other in
// the L2 (16 tokens' words in one sector cost a 16-token launch 1.5-2.5 us).
constexpr int kTokenWaited = 1 << 16;
constexpr int kCtrlTokenStride = 16;   // int32 words from one token's word to the next

__host__ __device__ constexpr int token_word(int token) { return kCtrlHeader + token * kCtrlTokenStride; }

inline int64_t control_bytes(int tokens) {
  return (static_cast<int64_t>(kCtrlHeader) * 4 + static_cast<int64_t>(tokens) * kCtrlTokenStride * 4 + 255) / 256 * 256;
}

// Where a launch of `tokens` tokens keeps h: the last tokens * d_ff * 2 bytes
// of the workspace (down to a multiple of 256).  A workspace serves launches of
// any size that fits it, in any order: h of a small launch must not land on the
// words that a larger launch counts with afterwards, and from the end it
// cannot, because the words of the largest launch that fits end before its h
// begins, and every smaller launch's h lies inside that one's.
inline char *h_base(void *workspace, int64_t workspace_bytes, int tokens, int d_ff) {
  const int64_t at = (workspace_bytes - static_cast<int64_t>(tokens) * d_ff * 2) & ~static_cast<int64_t>(255);
  return static_cast<char *>(workspace) + at;
}

// Thread 0's bounded wait until the low half of *counter reaches `expect`: relaxed looks at
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
  while ((__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffff) < expect) {
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

// Thread 0 of a workgroup that has waited on a token's word says so; the last
// of the token's `waiters` puts the word back to zero for the next launch.
__device__ __forceinline__ void waited_on(int32_t *counter, int waiters) {
  const int32_t before = __hip_atomic_fetch_add(counter, kTokenWaited, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
  if ((before >> 16) + 1 == waiters)
    __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Thread 0 of a workgroup that leaves a persistent launch; the last one out
// puts the ticket back to zero.
__device__ __forceinline__ void leave_launch(int32_t *ctrl, int workgroups) {
  const int32_t before = __hip_atomic_fetch_add(&ctrl[kCtrlExits], 1, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
  if (before + 1 == workgroups) {
    __hip_atomic_store(&ctrl[kCtrlTicket], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&ctrl[kCtrlExits], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace sub1

#define HIP_TRY(expr)                                                               \
  do {                                                                              \
    hipError_t e_ = (expr);                                                         \
    if (e_ != hipSuccess)                                                           \
      return sub1::fail(SUB1_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_));      \
  } while (0)

#endif  // SUB1_COMMON_H_
