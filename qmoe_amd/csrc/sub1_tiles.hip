// Many tokens through one compressed matrix on the matrix cores.
//
// Sub1Linear.forward on a sequence (reference sub1.py:132-143 launches one
// product per token and calls that "naive") is a skinny GEMM Y += X W^T, and
// the matrix cores do it (v_mfma_f32_32x32x16_bf16) once the ternary weights
// are bf16 values again.  Nothing is walked per token and nothing is scattered:
// the work no longer grows with tokens x non-zeros.
//
// The tile form of a matrix (sub1_tiles_*) is made for that, once, from the
// packed codes: 2 bits per weight, whatever the density, cut into units of
// 32 rows x 128 columns of 64 x 16 bytes.  In unit (u, w) lane l = 32 h + r
// holds the weights of row 32 u + r that it feeds the matrix core as its share
// of the B operand: in step s (0..7) of the window the eight columns
// 128 w + 16 s + 8 h + q.  Word s / 2 of its 16 bytes holds steps s and s + 1;
// the weight of step s = 2 m + e and q = 2 k + o sits in bits
// 16 o + 8 e + 2 k (+1) of word m, as 0 (the row's min), 1 (its max) or 2
// (zero).  A wavefront fetches a unit with one coalesced 16-byte load per
// lane.  Rows are padded to a multiple of 64 and columns to a multiple of 128
// with zeros; (min, max) per row are copied.
//
// From the codes to bf16 pairs without a table: (word >> 2 k) & 0x00030003
// times 0x0202 plus 0x01000100 is a byte selector that picks, out of the row's
// (min, max) word and a zero word, the two weights of pair k (v_perm_b32):
// four plain instructions per pair of weights.
//
// Kernel: a workgroup owns 64 rows x 64 tokens; its wavefronts split the
// windows of 128 columns among themselves (wavefront v takes v, v + n, ...).  Per
// window a wavefront copies the tokens' activations, 64 x 128, through
// registers into its own 16 KB of LDS (coalesced 16-byte loads, four tokens an
// instruction; the 16-byte pieces of a token are XOR-swizzled with the token's
// number so that neither the stores nor the operand reads meet in a bank), and
// per step of 16 columns reads its A operands from there, builds its B
// operands from the codes and adds into a 64 x 64 fp32 accumulator (2 x 2 MFMA
// blocks).  The loads of the next window are issued as soon as the registers
// are free, a whole window ahead.  All of them are buffer loads: what lies past
// the last token, past the width or past a wavefront's last window is given an
// offset outside the buffer and comes back as zeros, without a branch or a
// mask.  At the end the partial tiles are added through LDS in wavefront
// order, rounded to bf16 and added onto y in bf16 (reference
// sub1_cuda_kernel.cu:199-200).  The number of wavefronts depends on the matrix
// alone, so a token's result does not depend on the launch it is part of.
//
// Results: each product x * w is exact in fp32 and the sums are fp32, but in
// the matrix cores' own order; they agree with the row-walking kernels and the
// oracle to rounding (the tests hold them to 1e-2 and to the fp32 error bound),
// not to the bit.
#include <hip/hip_runtime.h>

#include <cstring>

#include "sub1_common.h"

namespace {

using sub1::bf16_to_f32;
using sub1::f32_to_bf16;
using sub1::fail;
using sub1::misaligned;

constexpr int kUnitRows = 32;             // rows per unit
constexpr int kRows = 64;                 // rows per workgroup: two units
constexpr int kCols = 128;                // columns per window
constexpr int kTokens = 64;               // tokens per workgroup
constexpr int kSteps = kCols / 16;        // MFMA steps per window
constexpr int kMaxWaves = 8;              // wavefronts per workgroup, at most
constexpr uint32_t kAllZero = 0xaaaaaaaau; // a word of codes of zero weights
constexpr int kPartialBytes = kTokens * kRows * 4;   // one wavefront's scaled tile

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

// The meta block: arrays back to back, each 256-byte aligned.
struct TileLayout {
  int units_down;     // units of 32 rows per matrix, even
  int windows;
  int64_t units;      // of all matrices
  int64_t minmax;     // u32 [count * height]
  int64_t status;     // i32 [4]: [0] rows whose codes do not cover the width
  int64_t bytes;
};

TileLayout tile_layout(int count, int height, int width) {
  TileLayout t;
  t.units_down = (height + kRows - 1) / kRows * (kRows / kUnitRows);
  t.windows = (width + kCols - 1) / kCols;
  t.units = static_cast<int64_t>(count) * t.units_down * t.windows;
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    int64_t o = off;
    off += align256(bytes);
    return o;
  };
  t.minmax = take(static_cast<int64_t>(count) * height * 4);
  t.status = take(16);
  t.bytes = off;
  return t;
}

// Calls nz(column, symbol) for every non-zero weight of a row, in column order,
// and returns the columns the row's codes cover (dictionary layout: reference
// sub1.py:60-72, sub1_cuda_kernel.cu:186-192).
template <class F>
__device__ __forceinline__ int each_nonzero(const uint16_t *codes, int n,
                                            const int32_t *__restrict__ dec, int width, F &&nz) {
  int col = 0;
  for (int i = 0; i < n; i++) {
    const int e = codes[i];
    const uint32_t w0 = static_cast<uint32_t>(dec[2 * e]);
    const uint32_t w1 = static_cast<uint32_t>(dec[2 * e + 1]);
    unsigned long long digits = static_cast<unsigned long long>(w0 >> 4) |
                                (static_cast<unsigned long long>(w1 >> 4) << 28);
    while (digits) {
      const int d = (__ffsll(digits) - 1) >> 1;
      const int sym = static_cast<int>(digits >> (2 * d)) & 3;
      digits &= ~(3ull << (2 * d));
      if (col + d < width && sym != 3) nz(col + d, sym);   // digits past the width are dropped
    }
    col += 2 * static_cast<int>(w0 & 15u);
  }
  return col;
}

struct RowSource {
  const int32_t *dec;
  const uint16_t *w_comp;
  const int64_t *code_base;   // NULL: one matrix, base 0
  const int32_t *row_off;     // [count, height + 1]
  int count, height, width;
};

__device__ __forceinline__ const uint16_t *codes_of(const RowSource &s, int m, int r, int &n) {
  const int32_t *ro = s.row_off + static_cast<int64_t>(m) * (s.height + 1);
  n = ro[r + 1] - ro[r];
  if (n < 1 || n > (s.width + 1) / 2) n = 0;   // counted as a bad row
  return s.w_comp + (s.code_base ? s.code_base[m] : 0) + ro[r];
}

// Where the weight of column c of a window sits in its lane's 16 bytes.
__device__ __forceinline__ void code_place(int c, int &half, int &word, int &shift) {
  const int step = c >> 4, q = c & 7;
  half = (c >> 3) & 1;
  word = step >> 1;
  shift = 16 * (q & 1) + 8 * (step & 1) + 2 * (q >> 1);
}

// One thread per row of every matrix: its codes into the units (all zero
// weights before).
__global__ __launch_bounds__(256) void code_emit_kernel(RowSource s, int units_down, int windows,
                                                        u32x4 *__restrict__ units,
                                                        int32_t *__restrict__ status,
                                                        int64_t rows_total) {
  const int64_t gl = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gl >= rows_total) return;
  const int m = static_cast<int>(gl / s.height);
  const int r = static_cast<int>(gl % s.height);
  u32x4 *mine = units + (static_cast<int64_t>(m) * units_down + r / kUnitRows) * windows * 64 +
                r % kUnitRows;
  uint32_t held[2][4];   // [half][word] of the window at hand
  int w_cur = 0;
  bool dirty = false;
  auto clear = [&]() {
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int d = 0; d < 4; d++) held[h][d] = kAllZero;
    dirty = false;
  };
  auto flush = [&]() {
    if (dirty) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        u32x4 v = {held[h][0], held[h][1], held[h][2], held[h][3]};
        mine[static_cast<int64_t>(w_cur) * 64 + h * kUnitRows] = v;
      }
    }
    clear();
  };
  clear();
  int n;
  const uint16_t *codes = codes_of(s, m, r, n);
  const int covered = each_nonzero(codes, n, s.dec, s.width, [&](int col, int sym) {
    const int w = col / kCols;
    if (w != w_cur) {
      flush();
      w_cur = w;
    }
    int half, word, shift;
    code_place(col % kCols, half, word, shift);
    // symbol 1 (min) is code 0, symbol 2 (max) code 1; the place holds 2 (zero)
    const uint32_t flip = (sym == 2 ? 3u : 2u) << shift;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int d = 0; d < 4; d++)
        if (h == half && d == word) held[h][d] ^= flip;
    dirty = true;
  });
  flush();
  if (covered != ((s.width + 1) & ~1)) atomicAdd(&status[0], 1);
}

// The symbols of one matrix back out of its units, a thread per weight.
__global__ __launch_bounds__(256) void code_decode_kernel(const u32x4 *__restrict__ units,
                                                          uint8_t *__restrict__ out, int matrix,
                                                          int units_down, int windows, int height,
                                                          int width) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<int64_t>(height) * width) return;
  const int r = static_cast<int>(i / width), col = static_cast<int>(i % width);
  int half, word, shift;
  code_place(col % kCols, half, word, shift);
  const u32x4 v = units[((static_cast<int64_t>(matrix) * units_down + r / kUnitRows) * windows +
                         col / kCols) * 64 + half * kUnitRows + r % kUnitRows];
  const uint32_t code = (v[word] >> shift) & 3u;
  out[i] = static_cast<uint8_t>(code == 2 ? 0 : code + 1);
}

__global__ void tile_fill_kernel(uint32_t *p, int64_t n, uint32_t v) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void tile_copy_words_kernel(const uint32_t *src, uint32_t *dst, int64_t n) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

// --------------------------------------------------------------- product ---

struct TileArgs {
  const u32x4 *units;
  const uint32_t *minmax;
  const uint16_t *x;
  uint16_t *y;
  int64_t ldx, ldy;
  int height, width, tokens;
  int units_down, windows, matrix;
};

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// A buffer over `bytes` bytes from base on: loads at offsets from `bytes` on
// return zeros and touch no memory.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_over(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes),
                                           0x00020000);
}
constexpr uint32_t kOutside = 0x80000000u;   // an offset past every buffer here

// Eight activations of one token from byte offset `at` of the buffer on, of
// which the first `inside` lie inside the width (8 or more: all; 0 or less:
// none).  kWide: x rows are 16-byte aligned and the width is a multiple of 8,
// so a piece lies inside or outside as a whole; otherwise element by element.
template <bool kWide>
__device__ __forceinline__ u32x4 load_piece(__amdgpu_buffer_rsrc_t x, uint32_t at, int inside) {
  if (kWide) return __builtin_amdgcn_raw_buffer_load_b128(x, inside > 0 ? at : kOutside, 0, 0);
  uint32_t e[8];
#pragma unroll
  for (int q = 0; q < 8; q++)
    e[q] = __builtin_amdgcn_raw_buffer_load_b16(x, (q < inside ? at : kOutside) + 2 * q, 0, 0);
  u32x4 v = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
  return v;
}

// The bf16 pair of weights of pair k (0..7) of a word of codes: `min_max` is
// the row's (min, max) word.
__device__ __forceinline__ uint32_t weight_pair(uint32_t codes, int k, uint32_t min_max) {
  const uint32_t two = (codes >> (2 * k)) & 0x00030003u;
  const uint32_t pick = two * 0x0202u + 0x01000100u;
  return __builtin_amdgcn_perm(0u, min_max, pick);
}

template <bool kWide>
__global__ __launch_bounds__(64 * kMaxWaves, 1) void matvec_tiles_kernel(TileArgs a) {
  extern __shared__ __align__(16) unsigned char lds[];
  float *partial = reinterpret_cast<float *>(lds);
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int block = blockIdx.x, t0 = blockIdx.y * kTokens;
  // the lane's two rows as the B operand (and as the outputs' column): 32 j + lane % 32
  uint32_t min_max[2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = block * kRows + j * kUnitRows + (lane & 31);
    min_max[j] = row < a.height ? a.minmax[static_cast<int64_t>(a.matrix) * a.height + row] : 0u;
  }
  // The activations of this workgroup's tokens.  Load u of a window brings
  // tokens 4 u + lane / 16; the lane's piece of its token is the one that
  // belongs at its place in LDS, piece (lane % 16) ^ (token % 16), and
  // token % 16 = 4 (u % 4) + lane / 16 takes four values.
  const int rows_here = min(kTokens, a.tokens - t0);
  const __amdgpu_buffer_rsrc_t xb = buffer_over(
      a.x + static_cast<int64_t>(t0) * a.ldx,
      static_cast<uint32_t>((static_cast<int64_t>(rows_here - 1) * a.ldx + a.width) * 2));
  uint32_t x_at[4];      // byte offset of the lane's piece in window 0, loads u = 0..3
  int x_col[4];          // and its first column
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int token = 4 * u + (lane >> 4);
    x_col[u] = 8 * ((lane & 15) ^ token);
    x_at[u] = static_cast<uint32_t>((token * a.ldx + x_col[u]) * 2);
  }
  const uint32_t x_step = static_cast<uint32_t>(16 * a.ldx * 2);   // sixteen tokens on
  unsigned char *xt = lds + wave * kPartialBytes;                   // [64 tokens][16 pieces]
  unsigned char *xt_put = xt + lane * 16;
  // as the A operand the lane has tokens 32 i + lane % 32 and in step s their
  // piece 2 s + half, kept at place (2 s + half) ^ (token % 16)
  const unsigned char *xt_get = xt + (lane & 31) * 256;
  const uint32_t get_z = static_cast<uint32_t>((half ^ (lane & 15)) << 4);
  // the two units of this workgroup's rows, window after window
  const __amdgpu_buffer_rsrc_t ub = buffer_over(
      a.units + (static_cast<int64_t>(a.matrix) * a.units_down + block * 2) * a.windows * 64,
      static_cast<uint32_t>(2 * a.windows * 1024));
  uint32_t unit_at[2];
#pragma unroll
  for (int j = 0; j < 2; j++) unit_at[j] = static_cast<uint32_t>(j * a.windows * 1024 + lane * 16);

  f32x16 acc[2][2];   // [32 tokens][32 rows] blocks
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  if (wave < a.windows) {
    int w = wave;
    u32x4 xv[16], codes[2];
    // The first window's loads, in the order in which the loop renews them: the
    // waits in the loop count the loads issued since, and are only as long as
    // they need to be when the way in and the way round agree.
#pragma unroll
    for (int u = 0; u < 16; u++)
      xv[u] = load_piece<kWide>(xb, x_at[u & 3] + (u >> 2) * x_step + w * (kCols * 2),
                                a.width - w * kCols - x_col[u & 3]);
#pragma unroll
    for (int j = 0; j < 2; j++) codes[j] = __builtin_amdgcn_raw_buffer_load_b128(ub, unit_at[j], w * 1024, 0);
    __builtin_amdgcn_sched_barrier(0);
    for (;;) {
      // this window's activations into LDS (after the last window's reads: the
      // LDS serves a wavefront's operations in order)
#pragma unroll
      for (int u = 0; u < 16; u++) *reinterpret_cast<u32x4 *>(xt_put + u * 1024) = xv[u];
      // what this wavefront takes next; after its last window nothing: every
      // offset outside, zeros that are not used
      const bool more = w + waves < a.windows;
      const int wn = w + waves;
      const int width_next = more ? a.width - wn * kCols : 0;
#pragma unroll
      for (int u = 0; u < 16; u++)
        xv[u] = load_piece<kWide>(xb, x_at[u & 3] + (u >> 2) * x_step + wn * (kCols * 2),
                                  width_next - x_col[u & 3]);
      u32x4 codes_next[2];
#pragma unroll
      for (int j = 0; j < 2; j++)
        codes_next[j] = __builtin_amdgcn_raw_buffer_load_b128(ub, more ? unit_at[j] : kOutside,
                                                              wn * 1024, 0);
      __builtin_amdgcn_sched_barrier(0);   // the loads stay up here, a window ahead
#pragma unroll
      for (int s = 0; s < kSteps; s++) {
        bf16x8 xa[2], wb[2];
        const uint32_t get = get_z ^ (32 * s);
#pragma unroll
        for (int i = 0; i < 2; i++)
          xa[i] = *reinterpret_cast<const bf16x8 *>(xt_get + i * (32 * 256) + get);
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const uint32_t word = codes[j][s >> 1];
          u32x4 v;
#pragma unroll
          for (int k = 0; k < 4; k++) v[k] = weight_pair(word, 4 * (s & 1) + k, min_max[j]);
          wb[j] = __builtin_bit_cast(bf16x8, v);
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[i], wb[j], acc[i][j], 0, 0, 0);
      }
      if (!more) break;
      w = wn;
      codes[0] = codes_next[0];
      codes[1] = codes_next[1];
    }
  }
  __syncthreads();   // the partial tiles take the place of the activations

  // Each wavefront's tile into LDS; then added in wavefront order.  Element
  // (token i, row j) of an accumulator block sits in lane
  // j + 32 * ((i / 4) % 2), register 4 * (i / 8) + i % 4.
  float *mine = partial + wave * (kTokens * kRows);
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int token = i * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
        const int r = j * 32 + (lane & 31);
        mine[token * kRows + r] = acc[i][j][v];
      }
  __syncthreads();
  // The wavefronts share the tokens; a lane has row `lane` of the block.  Eight
  // tokens at a time: their y are all requested before the first is needed
  // (tokens past the last: loads that return zero, stores that are dropped).
  const int row = block * kRows + lane;
  if (row < a.height) {
    const __amdgpu_buffer_rsrc_t yb = buffer_over(
        a.y + static_cast<int64_t>(t0) * a.ldy,
        static_cast<uint32_t>((static_cast<int64_t>(rows_here - 1) * a.ldy + a.height) * 2));
    const uint32_t y_at = static_cast<uint32_t>(row * 2), y_step = static_cast<uint32_t>(a.ldy * 2);
    for (int first = wave; first < rows_here; first += 8 * waves) {
      uint16_t before[8];
#pragma unroll
      for (int k = 0; k < 8; k++)
        before[k] = __builtin_amdgcn_raw_buffer_load_b16(yb, y_at + (first + k * waves) * y_step, 0, 0);
#pragma unroll
      for (int k = 0; k < 8; k++) {
        const int t = first + k * waves;
        const int at = (t & (kTokens - 1)) * kRows + lane;
        float sum = partial[at];
        for (int v = 1; v < waves; v++) sum += partial[v * (kTokens * kRows) + at];
        // reference sub1_cuda_kernel.cu:200: y[row] += bf16(res), the sum in bf16
        __builtin_amdgcn_raw_buffer_store_b16(
            f32_to_bf16(bf16_to_f32(before[k]) + bf16_to_f32(f32_to_bf16(sum))), yb,
            t < kTokens ? y_at + t * y_step : kOutside, 0, 0);
      }
    }
  }
}

// Wavefronts per workgroup for a matrix of `blocks` blocks of 64 rows and
// `windows` windows: 1, 2, 4 or 8, whichever gives the fewest rounds of
// workgroups over the chip times the windows a wavefront walks in a row
// (counting what a workgroup costs besides its windows) at eight tiles of
// tokens.  It depends on the matrix alone, never on the tokens of a launch, so
// a token's result is the same whatever launch it is part of.  A CU holds
// eight of these wavefronts (registers).
int pick_waves(int blocks, int windows) {
  int best = 1;
  double best_cost = 0;
  for (int n = 1; n <= kMaxWaves; n *= 2) {
    const int64_t slots = 256 * (8 / n);
    const int64_t rounds = (8ll * blocks + slots - 1) / slots;
    const double cost = rounds * (2.0 + 0.9 * ((windows + n - 1) / n));
    if (n == 1 || cost < best_cost - 1e-9) {
      best = n;
      best_cost = cost;
    }
  }
  return best;
}

int check_set(const sub1_matrix_set *ms, const char *who) {
  if (!ms) return fail(SUB1_ERR_NULL, "%s: NULL matrix set", who);
  if (!ms->dec || !ms->w_comp || !ms->row_off || !ms->ter_minmax ||
      (ms->count > 1 && !ms->code_base))
    return fail(SUB1_ERR_NULL, "%s: NULL pointer", who);
  if (ms->count < 1 || ms->height < 1 || ms->width < 1 ||
      static_cast<int64_t>(ms->count) * ((ms->height + kRows - 1) / kRows) *
              ((ms->width + kCols - 1) / kCols) > (1 << 28))
    return fail(SUB1_ERR_SHAPE, "%s: %d matrices of %d x %d", who, ms->count, ms->height,
                ms->width);
  if (misaligned(ms->dec, 4) || misaligned(ms->w_comp, 2) || misaligned(ms->row_off, 4) ||
      misaligned(ms->ter_minmax, 4) || misaligned(ms->code_base, 8))
    return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
  return SUB1_OK;
}

RowSource source_of(const sub1_matrix_set *ms) {
  RowSource s;
  s.dec = ms->dec;
  s.w_comp = reinterpret_cast<const uint16_t *>(ms->w_comp);
  s.code_base = ms->code_base;
  s.row_off = ms->row_off;
  s.count = ms->count;
  s.height = ms->height;
  s.width = ms->width;
  return s;
}

int check_tiles(const sub1_tiles *t, const char *who) {
  if (!t || !t->meta || !t->entries) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (t->count < 1 || t->height < 1 || t->width < 1)
    return fail(SUB1_ERR_SHAPE, "%s: %d matrices of %d x %d", who, t->count, t->height, t->width);
  if (misaligned(t->meta, 256) || misaligned(t->entries, 256))
    return fail(SUB1_ERR_ALIGN, "%s: buffers must be 256-byte aligned", who);
  const TileLayout l = tile_layout(t->count, t->height, t->width);
  if (t->meta_bytes < l.bytes) return fail(SUB1_ERR_SHAPE, "%s: meta smaller than its layout", who);
  if (t->total_chunks != l.units || t->entry_bytes < l.units * 1024)
    return fail(SUB1_ERR_SHAPE, "%s: entries buffer smaller than the layout needs", who);
  return SUB1_OK;
}

}  // namespace

// ================================================================ C ABI =====

extern "C" int64_t sub1_tiles_meta_bytes(int count, int height, int width) {
  if (count < 1 || height < 1 || width < 1) return 0;
  return tile_layout(count, height, width).bytes;
}

extern "C" int sub1_tiles_layout(const sub1_matrix_set *ms, void *meta, int64_t meta_bytes,
                                 sub1_tiles *out, void *stream) {
  const char *who = "sub1_tiles_layout";
  (void)stream;
  int rc = check_set(ms, who);
  if (rc) return rc;
  if (!meta || !out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (misaligned(meta, 256)) return fail(SUB1_ERR_ALIGN, "%s: meta must be 256-byte aligned", who);
  const TileLayout t = tile_layout(ms->count, ms->height, ms->width);
  if (meta_bytes < t.bytes)
    return fail(SUB1_ERR_SHAPE, "%s: meta needs %lld bytes", who, static_cast<long long>(t.bytes));
  out->meta = meta;
  out->entries = nullptr;
  out->meta_bytes = t.bytes;
  out->total_chunks = t.units;
  out->entry_bytes = t.units * 1024;
  out->count = ms->count;
  out->height = ms->height;
  out->width = ms->width;
  return SUB1_OK;
}

extern "C" int sub1_tiles_entries(const sub1_matrix_set *ms, const sub1_tiles *t, void *stream) {
  const char *who = "sub1_tiles_entries";
  int rc = check_set(ms, who);
  if (rc) return rc;
  rc = check_tiles(t, who);
  if (rc) return rc;
  if (t->count != ms->count || t->height != ms->height || t->width != ms->width)
    return fail(SUB1_ERR_SHAPE, "%s: the layout belongs to other matrices", who);
  const TileLayout l = tile_layout(t->count, t->height, t->width);
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *base = static_cast<char *>(const_cast<void *>(t->meta));
  int32_t *status = reinterpret_cast<int32_t *>(base + l.status);
  u32x4 *units = static_cast<u32x4 *>(const_cast<void *>(t->entries));
  tile_fill_kernel<<<1, 64, 0, s>>>(reinterpret_cast<uint32_t *>(status), 4, 0u);
  const int64_t unit_words = l.units * 256;
  tile_fill_kernel<<<static_cast<unsigned>((unit_words + 255) / 256), 256, 0, s>>>(
      reinterpret_cast<uint32_t *>(units), unit_words, kAllZero);
  const int64_t rows = static_cast<int64_t>(ms->count) * ms->height;
  code_emit_kernel<<<static_cast<unsigned>((rows + 255) / 256), 256, 0, s>>>(
      source_of(ms), l.units_down, l.windows, units, status, rows);
  tile_copy_words_kernel<<<static_cast<unsigned>((rows + 255) / 256), 256, 0, s>>>(
      static_cast<const uint32_t *>(ms->ter_minmax), reinterpret_cast<uint32_t *>(base + l.minmax),
      rows);
  HIP_TRY(hipGetLastError());
  int32_t bad = 0;
  HIP_TRY(hipMemcpyAsync(&bad, status, 4, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  if (bad) return fail(SUB1_ERR_SHAPE, "%s: the codes of %d rows do not cover the width", who, bad);
  return SUB1_OK;
}

extern "C" int sub1_matvec_tiles(const sub1_tiles *t, int matrix, const void *x, int64_t ldx,
                                 void *y, int64_t ldy, int tokens, void *stream) {
  const char *who = "sub1_matvec_tiles";
  if (tokens == 0) return SUB1_OK;
  int rc = check_tiles(t, who);
  if (rc) return rc;
  if (!x || !y) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (matrix < 0 || matrix >= t->count) return fail(SUB1_ERR_SHAPE, "%s: no matrix %d", who, matrix);
  if (tokens < 0 || tokens > (1 << 22))
    return fail(SUB1_ERR_SHAPE, "%s: tokens %d outside 0..2^22", who, tokens);
  if (ldx < t->width || ldy < t->height)
    return fail(SUB1_ERR_SHAPE, "%s: token strides smaller than the rows", who);
  if (misaligned(x, 2) || misaligned(y, 2)) return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
  const TileLayout l = tile_layout(t->count, t->height, t->width);
  const char *base = static_cast<const char *>(t->meta);
  TileArgs a;
  a.units = static_cast<const u32x4 *>(t->entries);
  a.minmax = reinterpret_cast<const uint32_t *>(base + l.minmax);
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.ldx = ldx;
  a.ldy = ldy;
  a.height = t->height;
  a.width = t->width;
  a.tokens = tokens;
  a.units_down = l.units_down;
  a.windows = l.windows;
  a.matrix = matrix;
  const bool wide = !misaligned(x, 16) && ldx % 8 == 0 && t->width % 8 == 0;
  if (ldx >= (1 << 24) || ldy >= (1 << 24))
    return fail(SUB1_ERR_SHAPE, "%s: token strides of 2^24 elements or more", who);
  const dim3 grid(l.units_down / 2, (tokens + kTokens - 1) / kTokens);
  const int waves = pick_waves(l.units_down / 2, l.windows);
  const size_t lds_bytes = static_cast<size_t>(waves) * kPartialBytes;
  auto kernel = wide ? matvec_tiles_kernel<true> : matvec_tiles_kernel<false>;
  HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kMaxWaves * kPartialBytes)));
  sub1::note_kernel(wide ? "matvec_tiles_kernel<true>" : "matvec_tiles_kernel<false>");
  kernel<<<grid, 64 * waves, lds_bytes, static_cast<hipStream_t>(stream)>>>(a);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_tiles_decode(const sub1_tiles *t, int matrix, void *tern_out, void *stream) {
  const char *who = "sub1_tiles_decode";
  int rc = check_tiles(t, who);
  if (rc) return rc;
  if (!tern_out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (matrix < 0 || matrix >= t->count) return fail(SUB1_ERR_SHAPE, "%s: no matrix %d", who, matrix);
  const TileLayout l = tile_layout(t->count, t->height, t->width);
  const int64_t n = static_cast<int64_t>(t->height) * t->width;
  code_decode_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0,
                        static_cast<hipStream_t>(stream)>>>(
      static_cast<const u32x4 *>(t->entries), static_cast<uint8_t *>(tern_out), matrix,
      l.units_down, l.windows, t->height, t->width);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}
