// gfx950 kernels and C ABI of libsub1_hip on the reference's packed layout:
// the decode-fused matrix-vector product over dictionary-coded ternary
// weights, the encoder, a plain decoder and the grouped expert-FFN launch that
// needs no preparation.  Written for 64-wide wavefronts.  The single product
// (matvec_wave_kernel) gives a wavefront to a row: lane j takes codeword j of
// each run of 64, a prefix sum across the lanes places it, a butterfly adds the
// lanes' sums.  The expert launch (moe_kernel) gives a lane to a row, so a
// wavefront advances 64 independent code streams without cross-lane traffic.
// Either way the work per codeword is proportional to the non-zero weights in
// it (at most three for the fixed dictionary).
//
// Reference behaviour being reproduced (not its implementation):
//   sub1_cuda_kernel.cu:129-202  Sub1MatVec       -> matvec_wave_kernel / moe_kernel
//   sub1_cuda_kernel.cu:211-239  Sub1PreparePack  -> pack_count_kernel
//   sub1_cuda_kernel.cu:241-250  Sub1Pack         -> pack_emit_kernel
//   test.py:103-115              decompress       -> decode_kernel
//   sub1.py:306-321              expert loop      -> moe_kernel
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#include "sub1_common.h"

namespace sub1 {

thread_local std::string g_err;
thread_local const char *g_kernel = "";

void note_kernel(const char *name) { g_kernel = name; }

int fail(int code, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

namespace {
std::mutex g_fault_mutex;
int32_t *g_fault_host = nullptr;     // pinned, mapped: kFaultWords words
int32_t *g_fault_device = nullptr;   // the same words as the GPUs address them
std::atomic<int64_t> g_wait_limit_us{250000};
std::atomic<int> g_expect_extra{0};
std::atomic<int> g_clock_khz{0};     // rate of wall_clock64 on the device first asked
}  // namespace

int fault_words(int32_t **device_ptr, bool may_allocate) {
  std::lock_guard<std::mutex> lock(g_fault_mutex);
  if (!g_fault_host) {
    if (!may_allocate)
      return fail(SUB1_ERR_INTERNAL, "call sub1_init() once before an entry point that does not allocate");
    void *host = nullptr, *dev = nullptr;
    HIP_TRY(hipHostMalloc(&host, kFaultWords * sizeof(int32_t),
                          hipHostMallocPortable | hipHostMallocMapped));
    for (int i = 0; i < kFaultWords; i++) static_cast<int32_t *>(host)[i] = 0;
    HIP_TRY(hipHostGetDevicePointer(&dev, host, 0));
    g_fault_host = static_cast<int32_t *>(host);
    g_fault_device = static_cast<int32_t *>(dev);
  }
  *device_ptr = g_fault_device;
  return SUB1_OK;
}

bool fault_flag_host(int word) {
  std::lock_guard<std::mutex> lock(g_fault_mutex);
  return g_fault_host && *const_cast<volatile int32_t *>(&g_fault_host[word]) != 0;
}

int64_t wait_limit_ticks() {
  int khz = g_clock_khz.load();
  if (khz <= 0) {
    int device = 0, rate = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&rate, hipDeviceAttributeWallClockRate, device) == hipSuccess &&
        rate > 0)
      khz = rate;
    else
      khz = 100000;   // 100 MHz
    g_clock_khz.store(khz);
  }
  return g_wait_limit_us.load() * khz / 1000;
}

int expect_extra() { return g_expect_extra.load(); }

}  // namespace sub1

namespace {

using sub1::bf16_to_f32;
using sub1::f32_to_bf16;
using sub1::fail;
using sub1::misaligned;
using sub1::row_result;

// ------------------------------------------------------------ slot table ---
//
// The reference table spends two 32-bit words per entry on 28 two-bit digits
// of which at most three are non-zero.  The kernels use a derived one-word
// form that lists the non-zeros:
//   bits 0-3          pair count L (the entry spans 2L weights)
//   bits 4+7j..10+7j  slot j = 3*pos + sym  (pos 0..27, sym 1 = row min,
//                     2 = row max), 0 = no further non-zero
// 3*pos+sym is directly an offset into the tripled activation array below.
constexpr int kSlots = 3;
constexpr int kSlotBits = 7;
constexpr uint32_t kSlotMask = (1u << kSlotBits) - 1;

__global__ void derive_slot_table_kernel(const int32_t *__restrict__ dec,
                                         uint32_t *__restrict__ tab,
                                         int32_t *__restrict__ unsupported) {
  int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= SUB1_DICT_ENTRIES) return;
  uint32_t w0 = static_cast<uint32_t>(dec[2 * e]);
  uint32_t w1 = static_cast<uint32_t>(dec[2 * e + 1]);
  uint32_t out = w0 & 0xfu;
  int n = 0;
  bool bad = false;
  for (int d = 0; d < 28; d++) {
    uint32_t w = d < 14 ? w0 : w1;
    uint32_t t = (w >> (4 + 2 * (d % 14))) & 3u;
    if (t == 0) continue;
    if (t == 3 || n == kSlots) {
      bad = true;
      break;
    }
    out |= static_cast<uint32_t>(3 * d + t) << (4 + kSlotBits * n);
    n++;
  }
  tab[e] = out;
  if (bad) atomicOr(unsupported, 1);
}

// The cached table is found by the address of the caller's dec.  To notice an
// address that now holds something else, 64 words of dec at fixed scattered
// places are kept beside the table and compared by one wavefront of every
// launch; a difference sets the sticky kFaultDec flag (the host then drops its
// cached tables).
constexpr int kPrintWords = 64;
__host__ __device__ constexpr int print_index(int i) {
  return (i * 4099 + 7) & (SUB1_DEC_WORDS - 1);
}

__global__ void capture_print_kernel(const int32_t *__restrict__ dec, int32_t *__restrict__ print) {
  if (threadIdx.x < kPrintWords) print[threadIdx.x] = dec[print_index(threadIdx.x)];
}

__device__ __forceinline__ void compare_print(const int32_t *__restrict__ dec,
                                              const int32_t *__restrict__ print,
                                              int32_t *sticky) {
  if (threadIdx.x < kPrintWords && dec[print_index(threadIdx.x)] != print[threadIdx.x])
    sub1::raise_fault(sticky, sub1::kFaultDec);
}

// ----------------------------------------------- activations in LDS --------
//
// x is kept in LDS as fp32, tripled:  M[3k] = 0, M[3k+1] = x[k], M[3k+2] = 0.
// Reading the pair (M[i], M[i-1]) at i = 3k+sym gives (x,0) for sym 1, (0,x)
// for sym 2 and (0,0) for an empty slot (i = 3k), so a slot costs two adds and
// no select; the pair is one ds_read2_b32.  One spare dword in front makes
// M[-1] readable, and 28 zero columns behind the row cover the digits of a
// last codeword that hang over the row end (the reference pads the same way,
// sub1_cuda_kernel.cu:147-151).
__host__ __device__ constexpr int lds_dwords_for_width(int width) {
  return 1 + 3 * (width + 28) + 3;
}

template <int kThreads>
__device__ __forceinline__ void stage_activations(float *lds, const uint16_t *x,
                                                  int width) {
  const int n = width + 29;
  if (threadIdx.x == 0) lds[0] = 0.f;
  for (int k = threadIdx.x; k < n; k += kThreads) {
    float v = k < width ? bf16_to_f32(x[k]) : 0.f;
    float *m = lds + 1 + 3 * k;
    m[0] = 0.f;
    m[1] = v;
    m[2] = 0.f;
  }
}

// One codeword: three slots, then advance the column (in dwords of M).
__device__ __forceinline__ void add_codeword(uint32_t e, const float *M, int &colw,
                                             float &s1, float &s2) {
#pragma unroll
  for (int j = 0; j < kSlots; j++) {
    int idx = colw + static_cast<int>((e >> (4 + kSlotBits * j)) & kSlotMask);
    s1 += M[idx];
    s2 += M[idx - 1];
  }
  colw += static_cast<int>(e & 0xfu) * 6;
}

__device__ __forceinline__ void load_codes8(const uint16_t *p, uint32_t (&w)[4]) {
  // the stream is only 2-byte aligned; gfx950 global loads take any alignment
  __builtin_memcpy(w, p, 16);
}

// Sum of activations under the symbol-1 and symbol-2 weights of one row, in
// fp32, in the library's canonical order: the row's codes in groups of 32, a
// partial sum per group taken left to right from zero, the partial sums added
// first group first.  (The grouping lets the prepared kernels split a row
// between wavefronts without changing a bit of the result.)
// The table word of a code: from the copy of the table's first `held` words in
// LDS where the code lies in it, from the table in global memory otherwise.  A
// gather from the 256 KB table costs a compute unit about 54 ns per wavefront
// instruction (every lane fetches a cache line of its own through the L1), one
// from LDS 3 ns, and the low codes are the frequent ones: the first 21 500
// entries take 64% of the codes of weights with 90% zeros.
struct TableView {
  const uint32_t *tab;
  const uint32_t *held_words;
  uint32_t held;
  __device__ __forceinline__ uint32_t operator[](uint32_t code) const {
    return code < held ? held_words[code] : tab[code];
  }
};

__device__ __forceinline__ void row_sums(const TableView tab,
                                         const uint16_t *__restrict__ codes, int len,
                                         const float *M, float &s1, float &s2) {
  s1 = 0.f;
  s2 = 0.f;
  float p1 = 0.f, p2 = 0.f;
  int colw = 0;
  int i = 0;
  uint32_t w[4];
  if (len >= 8) load_codes8(codes, w);
  for (; i + 8 <= len; i += 8) {
    uint32_t cur[4] = {w[0], w[1], w[2], w[3]};
    if (i + 16 <= len) load_codes8(codes + i + 8, w);
    uint32_t e[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      e[2 * j] = tab[cur[j] & 0xffffu];
      e[2 * j + 1] = tab[cur[j] >> 16];
    }
#pragma unroll
    for (int j = 0; j < 8; j++) add_codeword(e[j], M, colw, p1, p2);
    if (((i + 8) & 31) == 0) {   // a group of 32 codes is complete
      s1 += p1;
      s2 += p2;
      p1 = 0.f;
      p2 = 0.f;
    }
  }
  int rem = len - i;
  if (rem > 0) {
    if (len >= 8) {
      // the row's last eight codes; the first 8-rem of them are already done
      load_codes8(codes + len - 8, w);
      int skip = 8 - rem;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        uint32_t code = (j & 1) ? (w[j / 2] >> 16) : (w[j / 2] & 0xffffu);
        uint32_t e = tab[code];
        if (j < skip) e = 0u;  // entry 0 of the slot form: nothing, no advance
        add_codeword(e, M, colw, p1, p2);
      }
    } else {
      for (int j = 0; j < rem; j++) add_codeword(tab[codes[j]], M, colw, p1, p2);
    }
  }
  s1 += p1;   // the last, possibly partial, group (adds +0 if it was just folded)
  s2 += p2;
}

// ------------------------------------------------------------- matvec ------
//
// One product y += W x on the packed layout, built for the latency of a single
// call (reference sub1_cuda_kernel.cu:163-201 re-thought for 64-wide
// wavefronts): a WAVEFRONT per row.  Lane j takes codeword j of each run of 64
// consecutive codes of the row: one coalesced 128-byte load per run; its
// dictionary entry straight from the caller's dec (8 bytes per lane, from L2: no
// derived table and nothing remembered between calls); the column at which the
// codeword starts from a DPP prefix sum of the entries' lengths across the
// lanes; the activation under each of the entry's non-zero digits (at most
// three for the fixed dictionary) from x through the vector cache; products
// x * (row min | row max) added in fp32 per lane; and at the row's end a
// butterfly sum over the 64 lanes.  Every load a wavefront needs is requested
// as early as its address is known: row offsets, (min, max) and y at once, all
// code loads of the row before the first table read.
//
// Order of additions (the oracle's sub1o_matvec_wave): lane j adds its
// codewords j, j + 64, ... in turn, the digits of a codeword left to right, one
// fused multiply-add each; then six butterfly steps, lane l adding lane l ^ m
// for m = 1, 2, 4, 8, 16, 32; bf16; y += in bf16.

// dpp_ctrl values of the row shifts and row broadcasts (CDNA ISA, DPP)
constexpr int kDppRowShr1 = 0x111, kDppRowShr2 = 0x112, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;
constexpr int kDppBcast15 = 0x142, kDppBcast31 = 0x143;
constexpr int kDppQuadXor1 = 0xb1, kDppQuadXor2 = 0x4e;      // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int kDppHalfMirror = 0x141, kDppRowMirror = 0x140;

template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_or_zero(int v) {
  // lanes outside the row mask and lanes whose source lies outside the row get 0
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, kRowMask, 0xf, false);
}

// Inclusive prefix sum over the 64 lanes.
__device__ __forceinline__ int wave_prefix_sum(int v) {
  v += dpp_or_zero<kDppRowShr1, 0xf>(v);
  v += dpp_or_zero<kDppRowShr2, 0xf>(v);
  v += dpp_or_zero<kDppRowShr4, 0xf>(v);
  v += dpp_or_zero<kDppRowShr8, 0xf>(v);
  v += dpp_or_zero<kDppBcast15, 0xa>(v);   // row 0 -> row 1, row 2 -> row 3
  v += dpp_or_zero<kDppBcast31, 0xc>(v);   // rows 0-1 -> rows 2-3
  return v;
}

template <int kCtrl>
__device__ __forceinline__ float dpp_float(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, false));
}

// Lane l receives the sum of the butterfly over all 64 lanes: l + (l ^ 1), then
// ^ 2, ^ 4, ^ 8, ^ 16, ^ 32.  After the steps 1 and 2 the four lanes of a quad
// hold the same value, so the mirror within eight lanes pairs a lane with the
// other quad exactly as ^ 4 does, and the mirror within a row of sixteen as ^ 8.
__device__ __forceinline__ float wave_butterfly_sum(float v) {
  v += dpp_float<kDppQuadXor1>(v);
  v += dpp_float<kDppQuadXor2>(v);
  v += dpp_float<kDppHalfMirror>(v);
  v += dpp_float<kDppRowMirror>(v);
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  return v;
}

constexpr int kWaveRuns = 4;   // runs of 64 codes whose loads are requested together

template <int kWaves>
__global__ __launch_bounds__(64 * kWaves) void matvec_wave_kernel(
    const int32_t *__restrict__ dec, const uint16_t *__restrict__ w_comp,
    const int32_t *__restrict__ row_off, const uint32_t *__restrict__ minmax,
    const uint16_t *__restrict__ x, uint16_t *__restrict__ y, int height, int width,
    int64_t ldx, int64_t ldy) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (row >= height) return;
  x += static_cast<int64_t>(blockIdx.y) * ldx;
  y += static_cast<int64_t>(blockIdx.y) * ldy;
  const int off = __builtin_amdgcn_readfirstlane(row_off[row]);
  const int len = __builtin_amdgcn_readfirstlane(row_off[row + 1]) - off;
  const uint32_t mm = minmax[row];
  const uint16_t y_old = y[row];
  const float w_min = __uint_as_float(mm << 16), w_max = __uint_as_float(mm & 0xffff0000u);
  const uint16_t *codes = w_comp + off;
  const uint2 *table = reinterpret_cast<const uint2 *>(dec);
  float acc = 0.f;
  int col = 0;   // the column at which the current run of codes starts
  for (int c0 = 0; c0 < len; c0 += 64 * kWaveRuns) {
    // the codes of up to kWaveRuns runs, then their dictionary entries
    int code[kWaveRuns];
    uint2 entry[kWaveRuns];
#pragma unroll
    for (int u = 0; u < kWaveRuns; u++) {
      const int i = c0 + 64 * u + lane;
      code[u] = i < len ? codes[i] : -1;
    }
#pragma unroll
    for (int u = 0; u < kWaveRuns; u++)
      entry[u] = code[u] >= 0 ? table[code[u]] : make_uint2(0u, 0u);   // no code: no digits, length 0

#pragma unroll
    for (int u = 0; u < kWaveRuns; u++) {
      if (c0 + 64 * u >= len) break;
      const int span = 2 * static_cast<int>(entry[u].x & 15u);     // weights the codeword covers
      const int upto = wave_prefix_sum(span);
      int at = col + upto - span;                                  // where this lane's codeword starts
      col += __builtin_amdgcn_readlane(upto, 63);
      unsigned long long digits = static_cast<unsigned long long>(entry[u].x >> 4) |
                                  (static_cast<unsigned long long>(entry[u].y >> 4) << 28);
      while (digits) {
        const int d = (__ffsll(digits) - 1) >> 1;
        const int sym = static_cast<int>(digits >> (2 * d)) & 3;
        digits &= ~(3ull << (2 * d));
        if (at + d < width) {   // digits past the width are dropped
          const float xv = bf16_to_f32(x[at + d]);
          acc = __fmaf_rn(xv, sym == 1 ? w_min : (sym == 2 ? w_max : 0.f), acc);
        }
      }
    }
  }
  const float res = wave_butterfly_sum(acc);
  if (lane == 0) {
    // reference sub1_cuda_kernel.cu:200: y[row] += bf16(res), the sum in bf16
    y[row] = f32_to_bf16(bf16_to_f32(y_old) + bf16_to_f32(f32_to_bf16(res)));
  }
}

// ------------------------------------------------------------- decode ------

__global__ void decode_kernel(const int32_t *__restrict__ dec,
                              const uint16_t *__restrict__ w_comp,
                              const int32_t *__restrict__ row_off,
                              const uint32_t *__restrict__ minmax,
                              uint8_t *__restrict__ out_tern,
                              uint16_t *__restrict__ out_w,
                              int32_t *__restrict__ bad_rows, int height, int width) {
  int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= height) return;
  uint16_t deq[3] = {0, 0, 0};
  if (minmax) {
    uint32_t mm = minmax[row];
    deq[1] = static_cast<uint16_t>(mm & 0xffffu);
    deq[2] = static_cast<uint16_t>(mm >> 16);
  }
  int64_t base = static_cast<int64_t>(row) * width;
  int idx = 0;
  for (int c = row_off[row]; c < row_off[row + 1]; c++) {
    int e = w_comp[c];
    uint32_t w0 = static_cast<uint32_t>(dec[2 * e]);
    uint32_t w1 = static_cast<uint32_t>(dec[2 * e + 1]);
    int n = 2 * static_cast<int>(w0 & 0xfu);
    for (int d = 0; d < n; d++) {
      if (idx + d >= width) break;
      uint32_t w = d < 14 ? w0 : w1;
      uint32_t t = (w >> (4 + 2 * (d % 14))) & 3u;
      if (out_tern) out_tern[base + idx + d] = static_cast<uint8_t>(t);
      if (out_w) out_w[base + idx + d] = t < 3 ? deq[t] : 0;
    }
    idx += n;
  }
  if (idx != ((width + 1) & ~1) && bad_rows) atomicAdd(bad_rows, 1);
}

// --------------------------------------------------------------- pack ------

constexpr int kTrieRoot = SUB1_DICT_ENTRIES;

__global__ void pack_count_kernel(const int32_t *__restrict__ trie,
                                  int32_t *__restrict__ w_tern,
                                  int32_t *__restrict__ row_cnt, int height,
                                  int width) {
  int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= height) return;
  int32_t *w = w_tern + static_cast<int64_t>(row) * width;
  int node = kTrieRoot;
  int n = 0;
  for (int i = 0; i < width; i += 2) {
    int lo = w[i];
    int hi = i + 1 < width ? w[i + 1] : 0;
    int sym = 3 * hi + lo;
    int child = trie[9 * node + sym];
    if (child < 0) {
      // n <= i/2 < i: the slot written was already consumed
      w[n++] = node;
      child = trie[9 * kTrieRoot + sym];
    }
    node = child;
  }
  w[n++] = node;
  row_cnt[row + 1] = n;
}

// Inclusive prefix sum over cnt[1..height] in place, cnt[0] = 0.  One
// workgroup; each thread owns a contiguous segment.
constexpr int kScanThreads = 1024;

__global__ __launch_bounds__(kScanThreads) void row_offset_scan_kernel(
    int32_t *__restrict__ cnt, int height) {
  __shared__ int32_t part[kScanThreads];
  const int tid = threadIdx.x;
  const int seg = (height + kScanThreads - 1) / kScanThreads;
  const int lo = 1 + tid * seg;
  const int hi = min(height + 1, lo + seg);
  int32_t s = 0;
  for (int i = lo; i < hi; i++) s += cnt[i];
  part[tid] = s;
  __syncthreads();
  for (int d = 1; d < kScanThreads; d *= 2) {
    int32_t v = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int32_t run = tid ? part[tid - 1] : 0;
  if (tid == 0) cnt[0] = 0;
  for (int i = lo; i < hi; i++) {
    run += cnt[i];
    cnt[i] = run;
  }
}

__global__ void pack_emit_kernel(const int32_t *__restrict__ w_codes,
                                 const int32_t *__restrict__ row_off,
                                 uint16_t *__restrict__ w_comp, int height,
                                 int width) {
  // one wavefront per row, lanes stride over the row's codes
  int row = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  if (row >= height) return;
  int lane = threadIdx.x % 64;
  int off = row_off[row];
  int n = row_off[row + 1] - off;
  const int32_t *src = w_codes + static_cast<int64_t>(row) * width;
  for (int i = lane; i < n; i += 64)
    w_comp[off + i] = static_cast<uint16_t>(src[i]);
}

// ------------------------------------------------------ grouped experts ----
//
// Persistent grid.  Work is cut into tiles (token, projection, block of
// kThreads rows), numbered with all wi tiles before all wo tiles, and handed
// out by an atomic ticket.  A wo tile of token t needs all of h[t], so it
// waits until the wi tiles of t have signalled; those have smaller tickets,
// were therefore taken by workgroups that are already running, and never wait
// themselves, so the wait always ends.
struct MoeArgs {
  const uint32_t *tab;
  const uint16_t *w_comp;
  const int64_t *wi_code_base;
  const int64_t *wo_code_base;
  const int32_t *wi_row_off;
  const int32_t *wo_row_off;
  const uint32_t *wi_minmax;
  const uint32_t *wo_minmax;
  const int32_t *token_expert;
  const uint16_t *x;
  uint16_t *y;
  uint16_t *h;
  int32_t *ctrl;  // the control words (sub1_common.h): ticket, fault counts, a word per token
  int tokens, d_model, d_ff, experts;
  int wi_tiles, wo_tiles;  // per token
  int tile_rows;           // rows of a tile: the workgroup's threads (a row each) or more (rows in turn)
  int act_dwords;          // LDS dwords of the activations; the table's first words follow
  int held;                // words of the table kept in LDS (0: none)
  int wi_expect;           // wi tiles a wo tile waits for (wi_tiles outside tests)
  int64_t wait_ticks;      // longest wait, in ticks of wall_clock64
  int32_t *sticky;         // fault flags in pinned host memory
  const int32_t *dec;      // the caller's table and the words kept of it
  const int32_t *print;
};

using sub1::kCtrlHeader;

template <int kThreads>
__global__ __launch_bounds__(kThreads) void moe_kernel(MoeArgs a) {
  extern __shared__ float lds[];
  __shared__ int s_ticket;
  const int n_wi = a.tokens * a.wi_tiles;
  const int n_all = n_wi + a.tokens * a.wo_tiles;
  if (blockIdx.x == 0) compare_print(a.dec, a.print, a.sticky);
  // the table's first words into LDS, once per workgroup (a persistent grid)
  uint32_t *held_words = reinterpret_cast<uint32_t *>(lds + a.act_dwords);
  for (int i = threadIdx.x; i < a.held; i += kThreads) held_words[i] = a.tab[i];
  const TableView table{a.tab, held_words, static_cast<uint32_t>(a.held)};
  for (;;) {
    __syncthreads();  // previous tile's readers of lds and s_ticket are done
    if (threadIdx.x == 0)
      s_ticket = __hip_atomic_fetch_add(&a.ctrl[0], 1, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int ticket = s_ticket;
    if (ticket >= n_all) break;

    if (ticket < n_wi) {
      const int t = ticket / a.wi_tiles;
      const int blk = ticket - t * a.wi_tiles;
      int e = a.token_expert[t];
      if (e >= a.experts) e = -1;
      if (e >= 0) {
        stage_activations<kThreads>(lds, a.x + static_cast<int64_t>(t) * a.d_model,
                                    a.d_model);
        __syncthreads();
        const int row_end = min(a.d_ff, (blk + 1) * a.tile_rows);
        for (int row = blk * a.tile_rows + threadIdx.x; row < row_end; row += kThreads) {
          const int32_t *ro = a.wi_row_off + static_cast<int64_t>(e) * (a.d_ff + 1);
          const int off = ro[row];
          const int len = ro[row + 1] - off;
          float s1, s2;
          row_sums(table, a.w_comp + a.wi_code_base[e] + off, len, lds + 1, s1, s2);
          float res = row_result(
              a.wi_minmax[static_cast<int64_t>(e) * a.d_ff + row], s1, s2);
          uint16_t hb = f32_to_bf16(res);
          if (hb & 0x8000u) hb = 0;  // relu
          // stored at agent scope: written through this die's L2, where the
          // workgroups on other dies will read it
          __hip_atomic_store(&a.h[static_cast<int64_t>(t) * a.d_ff + row], hb, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      // every wavefront waits for its h stores to be acknowledged, then the
      // barrier, then thread 0 counts the tile (a release fence here would write
      // back the whole L2)
      sub1::drain_stores();
      __syncthreads();
      if (threadIdx.x == 0 && e >= 0)   // a dropped token's word stays untouched
        __hip_atomic_fetch_add(&a.ctrl[sub1::token_word(t)], 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    } else {
      const int j = ticket - n_wi;
      const int t = j / a.wo_tiles;
      const int blk = j - t * a.wo_tiles;
      int e = a.token_expert[t];
      if (e >= a.experts) {
        if (blk == 0 && threadIdx.x == 0)
          __hip_atomic_fetch_add(&a.ctrl[sub1::kCtrlBadIds], 1, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
        e = -1;
      }
      const int row_end = min(a.d_model, (blk + 1) * a.tile_rows);
      if (e < 0) {
        for (int row = blk * a.tile_rows + threadIdx.x; row < row_end; row += kThreads) {
          int64_t i = static_cast<int64_t>(t) * a.d_model + row;
          a.y[i] = a.x[i];
        }
        continue;
      }
      if (threadIdx.x == 0)
        sub1::bounded_wait(&a.ctrl[sub1::token_word(t)], a.wi_expect, a.wait_ticks, a.sticky,
                           &a.ctrl[sub1::kCtrlGaveUp]);
      __syncthreads();  // thread 0's acquire now covers the whole workgroup
      stage_activations<kThreads>(lds, a.h + static_cast<int64_t>(t) * a.d_ff, a.d_ff);
      __syncthreads();
      for (int row = blk * a.tile_rows + threadIdx.x; row < row_end; row += kThreads) {
        const int32_t *ro = a.wo_row_off + static_cast<int64_t>(e) * (a.d_model + 1);
        const int off = ro[row];
        const int len = ro[row + 1] - off;
        float s1, s2;
        row_sums(table, a.w_comp + a.wo_code_base[e] + off, len, lds + 1, s1, s2);
        float res = row_result(
            a.wo_minmax[static_cast<int64_t>(e) * a.d_model + row], s1, s2);
        a.y[static_cast<int64_t>(t) * a.d_model + row] = f32_to_bf16(res);
      }
      // said once the tile's work is done: it takes a round trip to memory
      if (threadIdx.x == 0) sub1::waited_on(&a.ctrl[sub1::token_word(t)], a.wo_tiles);
    }
  }
  if (threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
}

__global__ void zero_i32_kernel(int32_t *p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ------------------------------------------------- derived-table cache -----

struct TableSlot {
  int device;
  const int32_t *dec;
  uint32_t *tab;          // kDictEntries table words, a flag word, kPrintWords of dec
  const int32_t *print;
};

std::mutex g_tab_mutex;
std::vector<TableSlot> g_tabs;
bool g_purged = false;   // the tables were dropped for the kFaultDec flag now standing

void drop_tables_locked(const int32_t *dec, bool all) {
  for (size_t i = 0; i < g_tabs.size();) {
    if (all || g_tabs[i].dec == dec) {
      (void)hipFree(g_tabs[i].tab);   // synchronises: no launch is still reading it
      g_tabs.erase(g_tabs.begin() + i);
    } else {
      i++;
    }
  }
}

// The compact table for `dec` on the current device, and the fault flags.  The
// first call with an address derives the table (one allocation, two small
// kernels, one synchronisation: not for a stream that is being captured).
int slot_table_for(const int32_t *dec, hipStream_t stream, TableSlot *out, int32_t **sticky) {
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  int rc = sub1::fault_words(sticky, true);
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(g_tab_mutex);
  // a launch found other contents at a cached address: every cached table is
  // suspect, derive them afresh (once per raised flag)
  const bool flagged = sub1::fault_flag_host(sub1::kFaultDec);
  if (flagged && !g_purged) {
    drop_tables_locked(nullptr, true);
    g_purged = true;
  }
  if (!flagged) g_purged = false;
  for (const TableSlot &s : g_tabs)
    if (s.device == device && s.dec == dec) {
      *out = s;
      return SUB1_OK;
    }
  uint32_t *tab = nullptr;
  HIP_TRY(hipMalloc(&tab, (SUB1_DICT_ENTRIES + 64 + kPrintWords) * sizeof(uint32_t)));
  int32_t *flag = reinterpret_cast<int32_t *>(tab + SUB1_DICT_ENTRIES);
  int32_t *print = flag + 64;
  zero_i32_kernel<<<1, 64, 0, stream>>>(flag, 1);
  derive_slot_table_kernel<<<SUB1_DICT_ENTRIES / 256, 256, 0, stream>>>(dec, tab, flag);
  capture_print_kernel<<<1, 64, 0, stream>>>(dec, print);
  int32_t bad = 0;
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpyAsync(&bad, flag, sizeof bad, hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess || bad) {
    (void)hipFree(tab);
    if (e != hipSuccess) return fail(SUB1_ERR_HIP, "deriving the table: %s", hipGetErrorString(e));
    return fail(SUB1_ERR_SHAPE,
                "dec holds an entry with a digit 3 or more than %d non-zero weights",
                kSlots);
  }
  g_tabs.push_back({device, dec, tab, print});
  *out = g_tabs.back();
  return SUB1_OK;
}

constexpr int kMatvecThreads = 256;
constexpr int kMoeThreads = 256;
constexpr int kMoeSweepThreads = 1024;   // one workgroup per compute unit, the table's head in its LDS

template <typename K>
int allow_lds(K kernel, size_t bytes) {
  if (bytes > 48 * 1024)
    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(bytes)));
  return SUB1_OK;
}

hipEvent_t g_ev_begin = nullptr, g_ev_end = nullptr;

}  // namespace

// ================================================================ C ABI =====

extern "C" const char *sub1_last_error(void) { return sub1::g_err.c_str(); }

extern "C" const char *sub1_last_kernel(void) { return sub1::g_kernel; }

extern "C" int sub1_abi_version(void) { return 4; }

extern "C" int sub1_matvec_tokens(const int32_t *dec, const int16_t *w_comp,
                                  const int32_t *row_off, const void *ter_minmax,
                                  const void *x, void *y, int height, int width,
                                  int tokens, int64_t ldx, int64_t ldy, void *stream) {
  if (tokens == 0) return SUB1_OK;
  if (!dec || !row_off || !ter_minmax || !x || !y)
    return fail(SUB1_ERR_NULL, "sub1_matvec: NULL argument");
  if (height < 1 || width < 1)
    return fail(SUB1_ERR_SHAPE, "sub1_matvec: height %d width %d", height, width);
  if (tokens < 0 || tokens > 65535)
    return fail(SUB1_ERR_SHAPE, "sub1_matvec: tokens %d outside 0..65535", tokens);
  if (tokens > 1 && (ldx < width || ldy < height))
    return fail(SUB1_ERR_SHAPE, "sub1_matvec: row strides smaller than the rows");
  if (!w_comp) return fail(SUB1_ERR_NULL, "sub1_matvec: NULL w_comp");
  if (misaligned(dec, 4) || misaligned(row_off, 4) || misaligned(ter_minmax, 4) ||
      misaligned(w_comp, 2) || misaligned(x, 2) || misaligned(y, 2))
    return fail(SUB1_ERR_ALIGN, "sub1_matvec: misaligned pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  constexpr int kWaves = 4;   // rows per workgroup
  dim3 grid((height + kWaves - 1) / kWaves, tokens);
  sub1::note_kernel("matvec_wave_kernel<4>");
  matvec_wave_kernel<kWaves><<<grid, 64 * kWaves, 0, s>>>(
      dec, reinterpret_cast<const uint16_t *>(w_comp), row_off,
      static_cast<const uint32_t *>(ter_minmax), static_cast<const uint16_t *>(x),
      static_cast<uint16_t *>(y), height, width, ldx, ldy);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_matvec(const int32_t *dec, const int16_t *w_comp,
                           const int32_t *row_off, const void *ter_minmax,
                           const void *x, void *y, int height, int width,
                           void *stream) {
  return sub1_matvec_tokens(dec, w_comp, row_off, ter_minmax, x, y, height, width, 1,
                            width, height, stream);
}

extern "C" int sub1_pack_count(const int32_t *trie, int32_t *w_tern, int32_t *row_off,
                               int height, int width, void *stream) {
  if (!trie || !w_tern || !row_off) return fail(SUB1_ERR_NULL, "sub1_pack_count: NULL argument");
  if (height < 1 || width < 1)
    return fail(SUB1_ERR_SHAPE, "sub1_pack_count: height %d width %d", height, width);
  if (misaligned(trie, 4) || misaligned(w_tern, 4) || misaligned(row_off, 4))
    return fail(SUB1_ERR_ALIGN, "sub1_pack_count: misaligned pointer");
  // the cumulative count is kept in int32 like the reference's row_off
  if (static_cast<int64_t>(height) * ((width + 1) / 2) > INT32_MAX)
    return fail(SUB1_ERR_SHAPE, "sub1_pack_count: more than 2^31 pairs in one call");
  hipStream_t s = static_cast<hipStream_t>(stream);
  pack_count_kernel<<<(height + 63) / 64, 64, 0, s>>>(trie, w_tern, row_off, height, width);
  row_offset_scan_kernel<<<1, kScanThreads, 0, s>>>(row_off, height);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_pack_emit(const int32_t *w_tern, const int32_t *row_off,
                              int16_t *w_comp, int height, int width, void *stream) {
  if (!w_tern || !row_off || !w_comp) return fail(SUB1_ERR_NULL, "sub1_pack_emit: NULL argument");
  if (height < 1 || width < 1)
    return fail(SUB1_ERR_SHAPE, "sub1_pack_emit: height %d width %d", height, width);
  if (misaligned(w_tern, 4) || misaligned(row_off, 4) || misaligned(w_comp, 2))
    return fail(SUB1_ERR_ALIGN, "sub1_pack_emit: misaligned pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  pack_emit_kernel<<<(height + 3) / 4, 256, 0, s>>>(
      w_tern, row_off, reinterpret_cast<uint16_t *>(w_comp), height, width);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_decode(const int32_t *dec, const int16_t *w_comp,
                           const int32_t *row_off, const void *ter_minmax,
                           uint8_t *out_tern, void *out_w, int32_t *bad_rows, int height,
                           int width, void *stream) {
  if (!dec || !w_comp || !row_off) return fail(SUB1_ERR_NULL, "sub1_decode: NULL argument");
  if (out_w && !ter_minmax) return fail(SUB1_ERR_NULL, "sub1_decode: out_w needs ter_minmax");
  if (height < 1 || width < 1)
    return fail(SUB1_ERR_SHAPE, "sub1_decode: height %d width %d", height, width);
  if (misaligned(dec, 4) || misaligned(row_off, 4) || misaligned(w_comp, 2) ||
      misaligned(ter_minmax, 4) || misaligned(out_w, 2) || misaligned(bad_rows, 4))
    return fail(SUB1_ERR_ALIGN, "sub1_decode: misaligned pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  decode_kernel<<<(height + 63) / 64, 64, 0, s>>>(
      dec, reinterpret_cast<const uint16_t *>(w_comp), row_off,
      static_cast<const uint32_t *>(ter_minmax), out_tern,
      static_cast<uint16_t *>(out_w), bad_rows, height, width);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int64_t sub1_moe_workspace_bytes(int tokens, int d_ff) {
  if (tokens < 0 || d_ff < 0) return 0;
  return sub1::control_bytes(tokens) + static_cast<int64_t>(tokens) * d_ff * 2;
}

extern "C" int sub1_moe_grouped(const sub1_moe_stack *st, const int32_t *token_expert,
                                const void *x, void *y, int tokens, void *workspace,
                                int64_t workspace_bytes, void *stream) {
  if (!st) return fail(SUB1_ERR_NULL, "sub1_moe_grouped: NULL stack");
  if (tokens == 0) return SUB1_OK;
  if (!token_expert || !x || !y)
    return fail(SUB1_ERR_NULL, "sub1_moe_grouped: NULL argument");
  if (!st->dec || !st->w_comp || !st->wi_code_base || !st->wo_code_base ||
      !st->wi_row_off || !st->wo_row_off || !st->wi_minmax || !st->wo_minmax)
    return fail(SUB1_ERR_NULL, "sub1_moe_grouped: NULL pointer in the stack");
  if (st->experts < 1 || st->d_model < 1 || st->d_ff < 1 ||
      st->d_model > SUB1_MAX_WIDTH || st->d_ff > SUB1_MAX_WIDTH)
    return fail(SUB1_ERR_SHAPE, "sub1_moe_grouped: experts %d d_model %d d_ff %d (sizes 1..%d)",
                st->experts, st->d_model, st->d_ff, SUB1_MAX_WIDTH);
  if (tokens < 0 || tokens > (1 << 20))
    return fail(SUB1_ERR_SHAPE, "sub1_moe_grouped: tokens %d outside 0..2^20", tokens);
  if (!workspace || workspace_bytes < sub1_moe_workspace_bytes(tokens, st->d_ff))
    return fail(SUB1_ERR_SHAPE, "sub1_moe_grouped: workspace of %lld bytes needed",
                static_cast<long long>(sub1_moe_workspace_bytes(tokens, st->d_ff)));
  if (misaligned(workspace, 256) || misaligned(st->dec, 4) || misaligned(st->w_comp, 2) ||
      misaligned(st->wi_code_base, 8) || misaligned(st->wo_code_base, 8) ||
      misaligned(st->wi_row_off, 4) || misaligned(st->wo_row_off, 4) ||
      misaligned(st->wi_minmax, 4) || misaligned(st->wo_minmax, 4) ||
      misaligned(token_expert, 4) || misaligned(x, 2) || misaligned(y, 2))
    return fail(SUB1_ERR_ALIGN, "sub1_moe_grouped: misaligned pointer");

  hipStream_t s = static_cast<hipStream_t>(stream);
  TableSlot slot;
  int32_t *sticky = nullptr;
  int rc = slot_table_for(st->dec, s, &slot, &sticky);
  if (rc) return rc;

  MoeArgs a;
  a.tab = slot.tab;
  a.dec = st->dec;
  a.print = slot.print;
  a.sticky = sticky;
  a.w_comp = reinterpret_cast<const uint16_t *>(st->w_comp);
  a.wi_code_base = st->wi_code_base;
  a.wo_code_base = st->wo_code_base;
  a.wi_row_off = st->wi_row_off;
  a.wo_row_off = st->wo_row_off;
  a.wi_minmax = static_cast<const uint32_t *>(st->wi_minmax);
  a.wo_minmax = static_cast<const uint32_t *>(st->wo_minmax);
  a.token_expert = token_expert;
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.ctrl = static_cast<int32_t *>(workspace);
  a.h = reinterpret_cast<uint16_t *>(sub1::h_base(workspace, workspace_bytes, tokens, st->d_ff));
  a.tokens = tokens;
  a.d_model = st->d_model;
  a.d_ff = st->d_ff;
  a.experts = st->experts;
  a.wait_ticks = sub1::wait_limit_ticks();
  int device = 0, cus = 0, per_cu = 0;
  HIP_TRY(hipGetDevice(&device));
  HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const int wmax = st->d_model > st->d_ff ? st->d_model : st->d_ff;
  a.act_dwords = lds_dwords_for_width(wmax);
  // With at least a token per compute unit the launch is a sweep, and what
  // bounds it is the table: one workgroup of 16 wavefronts per compute unit,
  // whole projections as tiles (a thread takes rows in turn), and all the LDS
  // that the activations leave for the table's first words.  Fewer tokens: tiles
  // of 256 rows, several workgroups per compute unit, the table from memory
  // (staging it would cost every workgroup more than it saves on one tile).
  const size_t lds_limit = 160 * 1024 - 64;
  const bool sweep = tokens >= cus &&
                     a.act_dwords * sizeof(float) + 16384 * sizeof(uint32_t) <= lds_limit;
  const int threads = sweep ? kMoeSweepThreads : kMoeThreads;
  a.tile_rows = sweep ? wmax : kMoeThreads;
  a.held = 0;
  if (sweep) {
    const size_t room = (lds_limit - a.act_dwords * sizeof(float)) / sizeof(uint32_t);
    a.held = static_cast<int>(room < SUB1_DICT_ENTRIES ? room : SUB1_DICT_ENTRIES);
  }
  a.wi_tiles = (st->d_ff + a.tile_rows - 1) / a.tile_rows;
  a.wo_tiles = (st->d_model + a.tile_rows - 1) / a.tile_rows;
  a.wi_expect = a.wi_tiles + sub1::expect_extra();
  int64_t tiles = static_cast<int64_t>(tokens) * (a.wi_tiles + a.wo_tiles);
  if (tiles > INT32_MAX - (1 << 20))
    return fail(SUB1_ERR_SHAPE, "sub1_moe_grouped: too many tiles");
  const size_t lds = (static_cast<size_t>(a.act_dwords) + a.held) * sizeof(float);
  if (sweep) {
    rc = allow_lds(moe_kernel<kMoeSweepThreads>, lds);
    per_cu = 1;
  } else {
    rc = allow_lds(moe_kernel<kMoeThreads>, lds);
    if (!rc)
      HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, moe_kernel<kMoeThreads>,
                                                           kMoeThreads, lds));
  }
  if (rc) return rc;
  if (per_cu < 1) return fail(SUB1_ERR_INTERNAL, "sub1_moe_grouped: kernel does not fit a CU");
  int64_t grid = static_cast<int64_t>(cus) * per_cu;
  if (grid > tiles) grid = tiles;

  if (sweep) {
    sub1::note_kernel("moe_kernel<1024>");
    moe_kernel<kMoeSweepThreads><<<static_cast<unsigned>(grid), threads, lds, s>>>(a);
  } else {
    sub1::note_kernel("moe_kernel<256>");
    moe_kernel<kMoeThreads><<<static_cast<unsigned>(grid), threads, lds, s>>>(a);
  }
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

// ---------------------------------------------------------- routing ------
//
// A wavefront per token: the first largest element of the token's row of the
// router's mask (what torch.argmax returns, reference sub1.py:311) and whether
// the row has a non-zero element at all (a token that the router's capacity
// limit dropped has none and keeps its input, reference sub1.py:312-318).
template <typename T>
__global__ __launch_bounds__(256) void route_from_mask_kernel(const T *__restrict__ mask,
                                                              int tokens, int experts,
                                                              int32_t *__restrict__ route,
                                                              int64_t *__restrict__ index) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= tokens) return;
  const int lane = threadIdx.x & 63;
  const T *row = mask + static_cast<int64_t>(t) * experts;
  long long best = 0;
  int at = experts;   // no element yet
  bool any = false;
  for (int e = lane; e < experts; e += 64) {
    const long long v = static_cast<long long>(row[e]);
    any = any || v != 0;
    if (at == experts || v > best) {
      best = v;
      at = e;
    }
  }
  // the lanes' candidates, largest value first, lowest index among equals
  for (int m = 1; m < 64; m <<= 1) {
    const long long v = __shfl_xor(best, m, 64);
    const int a = __shfl_xor(at, m, 64);
    if (a < experts && (at == experts || v > best || (v == best && a < at))) {
      best = v;
      at = a;
    }
  }
  const bool some = __ballot(any) != 0ull;
  if (lane == 0) {
    route[t] = some ? at : -1;
    if (index) index[t] = at;
  }
}

extern "C" int sub1_route_from_mask(const void *mask, int element_bytes, int tokens, int experts,
                                    int32_t *route, int64_t *expert_index, void *stream) {
  if (!mask || !route) return fail(SUB1_ERR_NULL, "sub1_route_from_mask: NULL argument");
  if (tokens < 0 || experts < 1)
    return fail(SUB1_ERR_SHAPE, "sub1_route_from_mask: tokens %d experts %d", tokens, experts);
  if (element_bytes != 1 && element_bytes != 4 && element_bytes != 8)
    return fail(SUB1_ERR_SHAPE, "sub1_route_from_mask: elements of %d bytes (1, 4 or 8)",
                element_bytes);
  if (misaligned(mask, element_bytes) || misaligned(route, 4) || misaligned(expert_index, 8))
    return fail(SUB1_ERR_ALIGN, "sub1_route_from_mask: misaligned pointer");
  if (tokens == 0) return SUB1_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned grid = static_cast<unsigned>((tokens + 3) / 4);
  if (element_bytes == 8)
    route_from_mask_kernel<<<grid, 256, 0, s>>>(static_cast<const int64_t *>(mask), tokens,
                                                experts, route, expert_index);
  else if (element_bytes == 4)
    route_from_mask_kernel<<<grid, 256, 0, s>>>(static_cast<const int32_t *>(mask), tokens,
                                                experts, route, expert_index);
  else
    route_from_mask_kernel<<<grid, 256, 0, s>>>(static_cast<const uint8_t *>(mask), tokens,
                                                experts, route, expert_index);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_fault_flags(int32_t *flags) {
  if (!flags) return fail(SUB1_ERR_NULL, "sub1_fault_flags: NULL argument");
  flags[0] = sub1::fault_flag_host(sub1::kFaultWait) ? 1 : 0;
  flags[1] = sub1::fault_flag_host(sub1::kFaultDec) ? 1 : 0;
  return SUB1_OK;
}

extern "C" const int32_t *sub1_fault_words_host(void) {
  std::lock_guard<std::mutex> lock(sub1::g_fault_mutex);
  return sub1::g_fault_host;
}

// Wait faults cleared so far.  A wait that gave up may have left the control
// words of its workspace at other values than zero (a writer that reports after
// the waiters have given up and cleared the word), and nothing in a later
// launch would notice: whoever owns a workspace compares this count with the
// one it saw when it last zeroed the buffer, and zeroes it again when they
// differ (ExpertStack.workspace and PreparedStack.workspace do).
std::atomic<int64_t> g_fault_epoch{0};

extern "C" int64_t sub1_fault_epoch(void) { return g_fault_epoch.load(); }

extern "C" int sub1_clear_faults(void) {
  // a standing kFaultDec flag means a cached table is stale: drop them all, so
  // that the calls after the reset derive theirs afresh
  if (sub1::fault_flag_host(sub1::kFaultDec)) {
    std::lock_guard<std::mutex> lock(g_tab_mutex);
    drop_tables_locked(nullptr, true);
  }
  if (sub1::fault_flag_host(sub1::kFaultWait)) g_fault_epoch.fetch_add(1);
  std::lock_guard<std::mutex> lock(sub1::g_fault_mutex);
  if (sub1::g_fault_host)
    for (int i = 0; i < sub1::kFaultWords; i++)
      *const_cast<volatile int32_t *>(&sub1::g_fault_host[i]) = 0;
  return SUB1_OK;
}

extern "C" int sub1_set_wait_limit_us(int64_t microseconds) {
  if (microseconds < 1 || microseconds > 60000000)
    return fail(SUB1_ERR_SHAPE, "sub1_set_wait_limit_us: %lld outside 1..60000000",
                static_cast<long long>(microseconds));
  sub1::g_wait_limit_us.store(microseconds);
  return SUB1_OK;
}

extern "C" int sub1_test_overstate_wait(int extra) {
  if (extra < 0) return fail(SUB1_ERR_SHAPE, "sub1_test_overstate_wait: negative count");
  sub1::g_expect_extra.store(extra);
  return SUB1_OK;
}

extern "C" int sub1_unregister_dec(const int32_t *dec) {
  std::lock_guard<std::mutex> lock(g_tab_mutex);
  drop_tables_locked(dec, dec == nullptr);
  return SUB1_OK;
}

extern "C" int sub1_timing_begin(void *stream) {
  if (!g_ev_begin) {
    HIP_TRY(hipEventCreate(&g_ev_begin));
    HIP_TRY(hipEventCreate(&g_ev_end));
  }
  HIP_TRY(hipEventRecord(g_ev_begin, static_cast<hipStream_t>(stream)));
  return SUB1_OK;
}

extern "C" int sub1_timing_end(void *stream, double *elapsed_us) {
  if (!g_ev_begin) return fail(SUB1_ERR_INTERNAL, "sub1_timing_end without sub1_timing_begin");
  if (!elapsed_us) return fail(SUB1_ERR_NULL, "sub1_timing_end: NULL argument");
  HIP_TRY(hipEventRecord(g_ev_end, static_cast<hipStream_t>(stream)));
  HIP_TRY(hipEventSynchronize(g_ev_end));
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, g_ev_begin, g_ev_end));
  *elapsed_us = 1e3 * static_cast<double>(ms);
  return SUB1_OK;
}
