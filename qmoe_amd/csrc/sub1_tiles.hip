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
// window a wavefront brings the tokens' activations, 64 x 128, into its own
// 16 KB of LDS (16-byte pieces, four tokens an instruction; the pieces of a
// token are XOR-swizzled with the token's number so that neither the arrivals
// nor the operand reads meet in a bank), and per step of 16 columns reads its
// A operands from there, builds its B operands from the codes and adds into a
// 64 x 64 fp32 accumulator (2 x 2 MFMA blocks).  Where x rows are 16-byte
// aligned the loads go straight into LDS, into a second buffer, a whole window
// ahead of the arithmetic (matvec_tiles_kernel); otherwise through registers,
// element by element (matvec_tiles_ragged_kernel).  All of them are buffer
// loads: what lies past the last token, past the width or past a wavefront's
// last window is given an offset outside the buffer (or an empty buffer) and
// reads nothing, without a branch or a mask.  At the end the partial tiles are
// added through LDS in wavefront order, rounded to bf16 and added onto y in
// bf16 (reference sub1_cuda_kernel.cu:199-200).  The number of wavefronts
// depends on the matrix alone, so a token's result does not depend on the
// launch it is part of.
//
// Bound: building the B operands, four plain instructions per pair of weights
// and 64 per step of four MFMAs, takes a wavefront twice as long to issue as
// the matrix core needs for the four; with the one wavefront per SIMD that the
// LDS leaves room for, a window takes 1.25 us where its MFMAs alone take 0.43.
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
constexpr int kMaxWaves = 4;              // wavefronts per workgroup, at most
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

// The bf16 pair of weights of pair k (0..7) of a word of codes: `min_max` is
// the row's (min, max) word.
__device__ __forceinline__ uint32_t weight_pair(uint32_t codes, int k, uint32_t min_max) {
  const uint32_t two = (codes >> (2 * k)) & 0x00030003u;
  const uint32_t pick = two * 0x0202u + 0x01000100u;
  return __builtin_amdgcn_perm(0u, min_max, pick);
}

// What the kernels share.  A workgroup owns rows 64 block .. +64 and tokens
// t0 .. +64; as the B operand (and as an output column) a lane has the rows
// 32 j + lane % 32, as the A operand the tokens 32 i + lane % 32 and in step s
// their piece 2 s + half.  In LDS piece p of token t of a window sits at
// 256 t + 16 (p ^ (t % 16)) of the wavefront's 16 KB.
struct TileLane {
  int lane, half, block, t0, rows_here;
  uint32_t min_max[2];
  uint32_t unit_at[2];   // byte offset of the lane's codes in window 0, per unit
  uint32_t get_at;       // of its A operand of step 0 in the wavefront's tile
};

__device__ __forceinline__ TileLane tile_lane(const TileArgs &a) {
  TileLane l;
  l.lane = threadIdx.x & 63;
  l.half = l.lane >> 5;
  l.block = blockIdx.x;
  l.t0 = blockIdx.y * kTokens;
  l.rows_here = min(kTokens, a.tokens - l.t0);
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = l.block * kRows + j * kUnitRows + (l.lane & 31);
    l.min_max[j] = row < a.height ? a.minmax[static_cast<int64_t>(a.matrix) * a.height + row] : 0u;
    l.unit_at[j] = static_cast<uint32_t>(j * a.windows * 1024 + l.lane * 16);
  }
  l.get_at = static_cast<uint32_t>((l.lane & 31) * 256 + ((l.half ^ (l.lane & 15)) << 4));
  return l;
}

// The codes of this workgroup's two units, window after window.
// (`any` false: an empty buffer, every load from it returns zeros.)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t units_of(const TileArgs &a, int block,
                                                           bool any = true) {
  return buffer_over(
      a.units + (static_cast<int64_t>(a.matrix) * a.units_down + block * 2) * a.windows * 64,
      any ? static_cast<uint32_t>(2 * a.windows * 1024) : 0u);
}

// The activations of this workgroup's tokens.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tokens_of(const TileArgs &a, const TileLane &l,
                                                            bool any = true) {
  return buffer_over(
      a.x + static_cast<int64_t>(l.t0) * a.ldx,
      any ? static_cast<uint32_t>((static_cast<int64_t>(l.rows_here - 1) * a.ldx + a.width) * 2)
          : 0u);
}

// One window: eight steps of four MFMAs on the activations in `tile` (this
// wavefront's 16 KB) and the weights in `codes`.  Each MFMA keeps the matrix
// core busy for as long as eight plain instructions take to issue, so the next
// step's B operands are built a quarter at a time behind the MFMAs of this one
// and its A operands are requested at its start.
__device__ __forceinline__ void window_steps(const unsigned char *tile, const TileLane &l,
                                             const u32x4 (&codes)[2], f32x16 (&acc)[2][2]) {
  const unsigned char *get = tile + l.get_at;
  bf16x8 xa[2];
  u32x4 wv[2];
#pragma unroll
  for (int i = 0; i < 2; i++) xa[i] = *reinterpret_cast<const bf16x8 *>(get + i * (32 * 256));
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int k = 0; k < 4; k++) wv[j][k] = weight_pair(codes[j][0], k, l.min_max[j]);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < kSteps; s++) {
    bf16x8 xa_next[2];
    u32x4 wv_next[2];
    const int sn = s + 1 < kSteps ? s + 1 : s;   // after the last step nothing new
    if (s + 1 < kSteps) {
#pragma unroll
      for (int i = 0; i < 2; i++)
        xa_next[i] = *reinterpret_cast<const bf16x8 *>(
            tile + (l.get_at ^ static_cast<uint32_t>(32 * sn)) + i * (32 * 256));
    }
    const bf16x8 wb0 = __builtin_bit_cast(bf16x8, wv[0]), wb1 = __builtin_bit_cast(bf16x8, wv[1]);
#pragma unroll
    for (int quarter = 0; quarter < 4; quarter++) {
      const int i = quarter >> 1, j = quarter & 1;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[i], j ? wb1 : wb0, acc[i][j], 0, 0, 0);
      if (s + 1 < kSteps) {
        const int jn = quarter >> 1, k0 = 2 * (quarter & 1);
#pragma unroll
        for (int k = k0; k < k0 + 2; k++)
          wv_next[jn][k] = weight_pair(codes[jn][sn >> 1], 4 * (sn & 1) + k, l.min_max[jn]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (s + 1 < kSteps) {
      xa[0] = xa_next[0];
      xa[1] = xa_next[1];
      wv[0] = wv_next[0];
      wv[1] = wv_next[1];
    }
  }
}

// The end of a workgroup: its wavefronts' tiles added in wavefront order,
// rounded to bf16 and added onto y in bf16 (reference sub1_cuda_kernel.cu:199-
// 200).  The wavefronts share the tokens, a lane has row `lane` of the block;
// the y of a lane's tokens are all requested before anything else (tokens past
// the last: loads that return zero, stores that are dropped).  `partial` is
// LDS that no wavefront reads any more.  kPer = 64 / waves.
template <int kPer>
__device__ __forceinline__ void finish_tile(const TileArgs &a, const TileLane &l, int wave,
                                            int waves, float *partial, const f32x16 (&acc)[2][2]) {
  const int row = l.block * kRows + l.lane;
  const __amdgpu_buffer_rsrc_t yb = buffer_over(
      a.y + static_cast<int64_t>(l.t0) * a.ldy,
      static_cast<uint32_t>((static_cast<int64_t>(l.rows_here - 1) * a.ldy + a.height) * 2));
  // rows past the height: outside the buffer
  const uint32_t y_at = row < a.height ? static_cast<uint32_t>(row * 2) : kOutside;
  const uint32_t y_step = static_cast<uint32_t>(a.ldy * 2);
  uint16_t before[kPer];
#pragma unroll
  for (int k = 0; k < kPer; k++)
    before[k] = __builtin_amdgcn_raw_buffer_load_b16(yb, y_at + (wave + k * waves) * y_step, 0, 0);
  // Element (token i, row j) of an accumulator block sits in lane
  // j + 32 * ((i / 4) % 2), register 4 * (i / 8) + i % 4.
  float *mine = partial + wave * (kTokens * kRows);
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int token = i * 32 + 8 * (v >> 2) + 4 * l.half + (v & 3);
        mine[token * kRows + j * 32 + (l.lane & 31)] = acc[i][j][v];
      }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kPer; k++) {
    const int t = wave + k * waves;
    const int at = t * kRows + l.lane;
    float sum = partial[at];
    for (int v = 1; v < waves; v++) sum += partial[v * (kTokens * kRows) + at];
    __builtin_amdgcn_raw_buffer_store_b16(
        f32_to_bf16(bf16_to_f32(before[k]) + bf16_to_f32(f32_to_bf16(sum))), yb, y_at + t * y_step, 0,
        0);
  }
}

// ---- x rows 16-byte aligned, the width a multiple of 8 ----------------------
//
// Activations and codes go from global memory straight into LDS (buffer loads
// with the lds bit, 16 bytes a lane: four tokens of activations, or one unit
// of codes, an instruction).  A wavefront has two buffers (a tile of
// activations of 16 KB and a block of codes of 2 KB each) and asks for the next
// window before it starts on the current one.
//
// Waiting is done by hand.  Left to the compiler, an LDS read behind such
// loads waits for all of them (it cannot tell the two buffers apart), which
// puts the memory latency of every window back in front of its arithmetic.  So
// the loop reads LDS through ds_read_b128 written as inline assembly, which
// the compiler does not see as LDS reads, and counts the loads itself: every
// turn issues exactly kLoadsPerWindow of them (after a wavefront's last window
// from empty buffers: nothing is read, nothing lands), loads complete in the
// order issued, and "all but the newest kLoadsPerWindow have landed" is the
// wait before a window is read.  The LDS reads are waited for with lgkmcnt(0)
// in statements that take the read registers as operands, so nothing uses them
// earlier.

constexpr int kLoadsPerWindow = 18;   // 16 of activations, 2 of codes
constexpr int kTileBytes = 16384;     // a tile of activations
constexpr int kBlockBytes = 2048;     // a window's codes (two units)

// Load u (0..15) of a window brings tokens 4 u + lane / 16, the lane its piece
// (lane % 16) ^ (token % 16): the one that belongs at its place in LDS.  `at`
// holds the lane's byte offsets for u = 0..3 (token % 16 takes four values per
// lane), `col` the first column of each.
struct Fetch {
  uint32_t at[4];
  int col[4];
  uint32_t step;   // sixteen tokens on
};

__device__ __forceinline__ Fetch fetch_of(const TileArgs &a, int lane) {
  Fetch f;
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int token = 4 * u + (lane >> 4);
    f.col[u] = 8 * ((lane & 15) ^ token);
    f.at[u] = static_cast<uint32_t>((token * a.ldx + f.col[u]) * 2);
  }
  f.step = static_cast<uint32_t>(16 * a.ldx * 2);
  return f;
}

typedef __attribute__((address_space(3))) unsigned char *lds_bytes;

// Window w on its way: the activations into the tile at `tile`, the codes into
// the block at `block`.  Pieces from the width on are not fetched (`edge`: this
// window reaches past the width; their places hold zeros or older activations,
// and the weights there are zeros).
__device__ __forceinline__ void fetch_window(__amdgpu_buffer_rsrc_t xb, __amdgpu_buffer_rsrc_t ub,
                                             const Fetch &f, const TileArgs &a, const TileLane &l,
                                             int w, bool edge, lds_bytes tile, lds_bytes block) {
  if (edge) {
    const int inside = a.width - w * kCols;
#pragma unroll
    for (int u = 0; u < 16; u++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          xb, tile + u * 1024, 16,
          f.col[u & 3] < inside ? f.at[u & 3] + (u >> 2) * f.step : kOutside, w * (kCols * 2), 0, 0);
  } else {
#pragma unroll
    for (int u = 0; u < 16; u++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xb, tile + u * 1024, 16,
                                               f.at[u & 3] + (u >> 2) * f.step, w * (kCols * 2), 0, 0);
  }
#pragma unroll
  for (int j = 0; j < 2; j++)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ub, block + j * 1024, 16, l.unit_at[j], w * 1024, 0, 0);
}

// 16 bytes from LDS address `at` and from `at` + kFar, requested only.
template <int kFar>
__device__ __forceinline__ void lds_request(uint32_t at, u32x4 &near, u32x4 &far) {
  asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:%3"
               : "=&v"(near), "=&v"(far)
               : "v"(at), "n"(kFar)
               : "memory");
}
// What was requested has arrived.
__device__ __forceinline__ void lds_arrived(u32x4 &p, u32x4 &q) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(p), "+v"(q)::"memory");
}

// window_steps with the operands read by hand: the tile at LDS address `tile`,
// the codes at `block`.
__device__ __forceinline__ void window_steps_counted(uint32_t tile, uint32_t block,
                                                     const TileLane &l, f32x16 (&acc)[2][2]) {
  const uint32_t get = tile + l.get_at;
  u32x4 xa[2], codes[2], wv[2];
  lds_request<1024>(block + l.lane * 16, codes[0], codes[1]);
  lds_request<32 * 256>(get, xa[0], xa[1]);
  lds_arrived(codes[0], codes[1]);
  lds_arrived(xa[0], xa[1]);
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int k = 0; k < 4; k++) wv[j][k] = weight_pair(codes[j][0], k, l.min_max[j]);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < kSteps; s++) {
    u32x4 xa_next[2], wv_next[2];
    const int sn = s + 1 < kSteps ? s + 1 : s;   // after the last step nothing new
    if (s + 1 < kSteps) lds_request<32 * 256>(get ^ static_cast<uint32_t>(32 * sn), xa_next[0], xa_next[1]);
    const bf16x8 wb0 = __builtin_bit_cast(bf16x8, wv[0]), wb1 = __builtin_bit_cast(bf16x8, wv[1]);
    const bf16x8 xa0 = __builtin_bit_cast(bf16x8, xa[0]), xa1 = __builtin_bit_cast(bf16x8, xa[1]);
#pragma unroll
    for (int quarter = 0; quarter < 4; quarter++) {
      const int i = quarter >> 1, j = quarter & 1;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(i ? xa1 : xa0, j ? wb1 : wb0, acc[i][j], 0, 0, 0);
      if (s + 1 < kSteps) {
        const int jn = quarter >> 1, k0 = 2 * (quarter & 1);
#pragma unroll
        for (int k = k0; k < k0 + 2; k++)
          wv_next[jn][k] = weight_pair(codes[jn][sn >> 1], 4 * (sn & 1) + k, l.min_max[jn]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (s + 1 < kSteps) {
      lds_arrived(xa_next[0], xa_next[1]);
      xa[0] = xa_next[0];
      xa[1] = xa_next[1];
      wv[0] = wv_next[0];
      wv[1] = wv_next[1];
    }
  }
}

template <int kWaves>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(1, 2)))
void matvec_tiles_kernel(TileArgs a) {
  __shared__ __align__(16384) unsigned char tiles[2 * kWaves * kTileBytes];   // [buffer][wavefront]
  __shared__ __align__(1024) unsigned char blocks[2 * kWaves * kBlockBytes];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const TileLane l = tile_lane(a);
  const Fetch f = fetch_of(a, l.lane);
  // (the rows' min and max are waited for here, while nothing else is on its way)
  asm volatile("" ::"v"(l.min_max[0]), "v"(l.min_max[1]));
  const lds_bytes my_tiles = (lds_bytes)tiles + wave * kTileBytes;
  const lds_bytes my_blocks = (lds_bytes)blocks + wave * kBlockBytes;
  const int last = a.windows - 1;
  const bool ragged_edge = (a.width & (kCols - 1)) != 0;
  if (ragged_edge) {
    // places that no fetch writes must not hold what LDS happened to hold
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int u = 0; u < 16; u++)
        *reinterpret_cast<u32x4 *>(tiles + (b * kWaves + wave) * kTileBytes + (u * 64 + l.lane) * 16) =
            zero;
    // these stores and the fetches below go to LDS by different ways: the
    // zeros must have arrived before the first fetch is asked for
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }

  f32x16 acc[2][2];   // [32 tokens][32 rows] blocks
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  if (wave < a.windows) {
    int w = wave;
    int cur = 0;   // the buffer that holds, or is about to hold, window w
    fetch_window(tokens_of(a, l), units_of(a, l.block), f, a, l, w, ragged_edge && w == last,
                 my_tiles, my_blocks);
    for (;;) {
      const int wn = __builtin_amdgcn_readfirstlane(w + kWaves);
      const bool more = wn < a.windows;
      const int next = __builtin_amdgcn_readfirstlane(cur ^ 1);
      // that buffer was read a turn ago, and those reads have been waited for
      fetch_window(tokens_of(a, l, more), units_of(a, l.block, more), f, a, l, wn,
                   ragged_edge && wn == last, my_tiles + next * (kWaves * kTileBytes),
                   my_blocks + next * (kWaves * kBlockBytes));
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerWindow) : "memory");
      window_steps_counted(
          static_cast<uint32_t>(reinterpret_cast<uintptr_t>(my_tiles + cur * (kWaves * kTileBytes))),
          static_cast<uint32_t>(reinterpret_cast<uintptr_t>(my_blocks + cur * (kWaves * kBlockBytes))),
          l, acc);
      if (!more) break;
      w = wn;
      cur = next;
    }
  }
  // nothing is on its way into LDS any more; then the partial tiles take the
  // place of the activations
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  finish_tile<kTokens / kWaves>(a, l, wave, kWaves, reinterpret_cast<float *>(tiles), acc);
}

// ---- any x ------------------------------------------------------------------
//
// The same, the activations read element by element into registers and stored
// into LDS from there (one tile per wavefront, the next window's loads issued
// as soon as the registers are free): for x rows that are not 16-byte aligned
// or a width that is not a multiple of 8.  The same sums in the same order.

// Eight activations of one token from byte offset `at` of the buffer on, of
// which the first `inside` lie inside the width (0 or less: none).
__device__ __forceinline__ u32x4 load_piece(__amdgpu_buffer_rsrc_t x, uint32_t at, int inside) {
  uint32_t e[8];
#pragma unroll
  for (int q = 0; q < 8; q++)
    e[q] = __builtin_amdgcn_raw_buffer_load_b16(x, (q < inside ? at : kOutside) + 2 * q, 0, 0);
  u32x4 v = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
  return v;
}

template <int kWaves>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
void matvec_tiles_ragged_kernel(TileArgs a) {
  __shared__ u32x4 tile[kWaves * 1024];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const TileLane l = tile_lane(a);
  const __amdgpu_buffer_rsrc_t xb = tokens_of(a, l), ub = units_of(a, l.block);
  const Fetch f = fetch_of(a, l.lane);
  u32x4 *mine = tile + wave * 1024;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  for (int w = wave; w < a.windows; w += kWaves) {
    u32x4 codes[2];
#pragma unroll
    for (int j = 0; j < 2; j++) codes[j] = __builtin_amdgcn_raw_buffer_load_b128(ub, l.unit_at[j], w * 1024, 0);
#pragma unroll
    for (int u = 0; u < 16; u++)
      mine[u * 64 + l.lane] = load_piece(xb, f.at[u & 3] + (u >> 2) * f.step + w * (kCols * 2),
                                         a.width - w * kCols - f.col[u & 3]);
    window_steps(reinterpret_cast<const unsigned char *>(mine), l, codes, acc);
  }
  __syncthreads();
  finish_tile<kTokens / kWaves>(a, l, wave, kWaves, reinterpret_cast<float *>(tile), acc);
}

// Wavefronts per workgroup for a matrix of `blocks` blocks of 64 rows and
// `windows` windows: 1, 2 or 4, whichever is estimated fastest at nine tiles of
// tokens (568, the longest sequence of the Switch encoders): rounds of
// workgroups over the chip, each taking 4 us plus 1.25 us per window that a
// wavefront walks (measured on the six Switch shapes).  A wavefront has 36 KB
// of a compute unit's 160 KB of LDS, so a unit holds four.  The choice depends
// on the matrix alone, never on the tokens of a launch, so a token's result is
// the same whatever launch it is part of.
int pick_waves(int blocks, int windows) {
  int best = 1;
  double best_cost = 0;
  for (int n = 1; n <= kMaxWaves; n *= 2) {
    const int64_t slots = 256 * (4 / n);
    const int64_t rounds = (9ll * blocks + slots - 1) / slots;
    const double cost = rounds * (4.0 + 1.25 * ((windows + n - 1) / n));
    if (n == 1 || cost < best_cost - 1e-9) {
      best = n;
      best_cost = cost;
    }
  }
  return best;
}

template <int kWaves>
void launch_tiles(const TileArgs &a, bool wide, dim3 grid, hipStream_t stream) {
  if (wide)
    matvec_tiles_kernel<kWaves><<<grid, 64 * kWaves, 0, stream>>>(a);
  else
    matvec_tiles_ragged_kernel<kWaves><<<grid, 64 * kWaves, 0, stream>>>(a);
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(l.units_down / 2, (tokens + kTokens - 1) / kTokens);
  const int waves = pick_waves(l.units_down / 2, l.windows);
  sub1::note_kernel(wide ? "matvec_tiles_kernel" : "matvec_tiles_ragged_kernel");
  if (waves == 1) launch_tiles<1>(a, wide, grid, s);
  else if (waves == 2) launch_tiles<2>(a, wide, grid, s);
  else launch_tiles<4>(a, wide, grid, s);
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
