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
// Long sequences go through workgroups of four wavefronts that share each
// window of activations in LDS instead (matvec_tiles_shared_kernel, below).
//
// Bound: a wavefront alone on its SIMD issues an MFMA of this shape every
// 18 ns (the matrix core needs 13.4); with the four plain instructions per
// pair of weights that build the B operands behind it, and the LDS reads of
// the A operands, 22 to 24 ns where an operand serves 128 tokens (four
// instructions per MFMA) and 27 to 30 ns where it serves 64 (eight), measured
// on loops of just these instructions; the kernels here take 28 and 35 ns.
// A second wavefront on the SIMD fills part of the gap, and then the issue of
// the decoding instructions is what the SIMD runs out of.
//
// Results: each product x * w is exact in fp32 and the sums are fp32, but in
// the matrix cores' own order; they agree with the row-walking kernels and the
// oracle to rounding (the tests hold them to 1e-2 and to the fp32 error bound),
// not to the bit.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <type_traits>

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

constexpr int kActivationLoads = 16;   // of a window: four tokens each
constexpr int kCodeLoads = 2;          // one per unit of 32 rows
constexpr int kLoadsPerWindow = kActivationLoads + kCodeLoads;   // what fetch_window issues, every time
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
    for (int u = 0; u < kActivationLoads; u++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          xb, tile + u * 1024, 16,
          f.col[u & 3] < inside ? f.at[u & 3] + (u >> 2) * f.step : kOutside, w * (kCols * 2), 0, 0);
  } else {
#pragma unroll
    for (int u = 0; u < kActivationLoads; u++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xb, tile + u * 1024, 16,
                                               f.at[u & 3] + (u >> 2) * f.step, w * (kCols * 2), 0, 0);
  }
#pragma unroll
  for (int j = 0; j < kCodeLoads; j++)
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

// ---- the same alignment, y rows 4-byte aligned, an even height ---------------
//
// Workgroups of four wavefronts that share what they fetch.  The wavefronts
// form kKP parts of the windows (part k takes windows k, k + kKP, ...: the sums
// and their order are those of matvec_tiles_kernel<kKP>) times kRG groups of 64
// rows; a workgroup owns 64 kRG rows and 32 kNB tokens.  The kRG wavefronts of
// a part bring each window of activations into LDS together, once, and every
// one of them multiplies its own rows with it: a window's activations cross the
// L1 once per 64 kRG rows instead of once per 64, and with kNB = 4 a B operand
// serves 128 tokens.  The codes go straight into registers.
//
// The steps of 16 columns form one pipeline across the windows: while the
// MFMAs of a step run, the B operands of the next step are built and its A
// operands read, also from the last step of a window to the first of the
// next.  A part has two tiles and a wavefront two sets of code registers.
// Before the last step of a window a wavefront waits for all it has asked for
// (its share of the next window, asked for a window ago) and meets the others
// at a barrier: then the next window is there whole, and everyone has read
// the last operands of this one, so during that step the window after the
// next is asked for into this window's tile and registers.  Nothing is counted
// by hand: at the barrier nothing of this wavefront is on its way.  Blocks of
// 32 tokens past the last token are neither multiplied nor stored.

template <int kOff>
__device__ __forceinline__ void lds_request_at(uint32_t at, u32x4 &v) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(at), "n"(kOff) : "memory");
}
// The operands of kN blocks of 32 tokens (kStride bytes apart), requested only.
template <int kN, int kStride = 8192>
__device__ __forceinline__ void lds_request_blocks(uint32_t at, u32x4 (&v)[kN]) {
  lds_request_at<0>(at, v[0]);
  if constexpr (kN > 1) lds_request_at<kStride>(at, v[1]);
  if constexpr (kN > 2) lds_request_at<2 * kStride>(at, v[2]);
  if constexpr (kN > 3) lds_request_at<3 * kStride>(at, v[3]);
}
template <int kN>
__device__ __forceinline__ void lds_arrived_blocks(u32x4 (&v)[kN]) {
  static_assert(kN == 1 || kN == 2 || kN == 4, "one, two or four blocks");
  if constexpr (kN == 1) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0])::"memory");
  if constexpr (kN == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1])::"memory");
  if constexpr (kN == 4)
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])::"memory");
}

// What a wavefront carries from one step of 16 columns to the next: the A
// operands of kLive blocks of 32 tokens and the B operands of its two units of
// rows.
template <int kLive>
struct StepOperands {
  u32x4 xa[kLive];
  u32x4 wv[2];
};

// The B operands of a step in the making: the eight pairs of weights of a
// wavefront's two units go through four stages (shift, mask, selector, pick),
// and each stage of a group of pairs is issued together, so that no
// instruction has to wait for the one just before it.
struct PairsInTheMaking {
  uint32_t v[8];
};
template <int kStage, int kE>
__device__ __forceinline__ void pair_stage(PairsInTheMaking &t, int p, uint32_t word0, uint32_t word1,
                                           const uint32_t (&min_max)[2], u32x4 (&wv)[2]) {
  const int q = 4 * kE + (p & 3);   // the pair's place in its word
  if (kStage == 0) t.v[p] = (p >> 2 ? word1 : word0) >> (2 * q);
  if (kStage == 1) t.v[p] &= 0x00030003u;
  if (kStage == 2) t.v[p] = __umul24(t.v[p], 0x0202u) + 0x01000100u;
  if (kStage == 3) wv[p >> 2][p & 3] = __builtin_amdgcn_perm(0u, min_max[p >> 2], t.v[p]);
}
// (keeps a stage where it was written: what it produced is not known before)
__device__ __forceinline__ void settle(PairsInTheMaking &t, int from, int count) {
  if (count == 8)
    asm volatile("" : "+v"(t.v[0]), "+v"(t.v[1]), "+v"(t.v[2]), "+v"(t.v[3]), "+v"(t.v[4]), "+v"(t.v[5]),
                 "+v"(t.v[6]), "+v"(t.v[7]));
  else
    asm volatile("" : "+v"(t.v[from]), "+v"(t.v[from + 1]), "+v"(t.v[from + 2]), "+v"(t.v[from + 3]));
}

// One step: 2 kLive MFMAs on `now`.  Each MFMA is followed by an equal share
// of the work for the step after it, which the matrix core's time covers: the
// B operands from half kE of `word0` and `word1` (the codes of the two units),
// and whatever `extra(m)` issues.  The A operands of that step are requested
// from `next_get` before the first MFMA and waited for after the last.  The
// fences keep every MFMA ahead of the work that hides behind it.
template <int kLive, int kNB, int kE, int kStride = 8192, class Extra>
__device__ __forceinline__ void tile_step(StepOperands<kLive> &now, uint32_t next_get,
                                          uint32_t word0, uint32_t word1,
                                          const uint32_t (&min_max)[2], f32x16 (&acc)[kNB][2],
                                          Extra &&extra) {
  StepOperands<kLive> next;
  PairsInTheMaking t;
  // (nothing that derives from the words is to be computed before this step)
  asm volatile("" : "+v"(word0), "+v"(word1));
  lds_request_blocks<kLive, kStride>(next_get, next.xa);
  const bf16x8 wb0 = __builtin_bit_cast(bf16x8, now.wv[0]), wb1 = __builtin_bit_cast(bf16x8, now.wv[1]);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int m = 0; m < 2 * kLive; m++) {
    const int i = m >> 1, j = m & 1;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, now.xa[i]),
                                                         j ? wb1 : wb0, acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kLive == 4) {
      // eight MFMAs: stage m % 4 of the pairs of unit m / 4
      const int from = 4 * (m >> 2);
#pragma unroll
      for (int p = from; p < from + 4; p++) {
        if ((m & 3) == 0) pair_stage<0, kE>(t, p, word0, word1, min_max, next.wv);
        if ((m & 3) == 1) pair_stage<1, kE>(t, p, word0, word1, min_max, next.wv);
        if ((m & 3) == 2) pair_stage<2, kE>(t, p, word0, word1, min_max, next.wv);
        if ((m & 3) == 3) pair_stage<3, kE>(t, p, word0, word1, min_max, next.wv);
      }
      if ((m & 3) != 3) settle(t, from, 4);
      else asm volatile("" : "+v"(next.wv[m >> 2]));
    } else if constexpr (kLive == 2) {
      // four MFMAs: stage m of all eight pairs
#pragma unroll
      for (int p = 0; p < 8; p++) {
        if (m == 0) pair_stage<0, kE>(t, p, word0, word1, min_max, next.wv);
        if (m == 1) pair_stage<1, kE>(t, p, word0, word1, min_max, next.wv);
        if (m == 2) pair_stage<2, kE>(t, p, word0, word1, min_max, next.wv);
        if (m == 3) pair_stage<3, kE>(t, p, word0, word1, min_max, next.wv);
      }
      if (m != 3) settle(t, 0, 8);
      else asm volatile("" : "+v"(next.wv[0]), "+v"(next.wv[1]));
    } else {
      // two MFMAs: two stages of all eight pairs behind each
#pragma unroll
      for (int p = 0; p < 8; p++) {
        if (m == 0) pair_stage<0, kE>(t, p, word0, word1, min_max, next.wv);
        else pair_stage<2, kE>(t, p, word0, word1, min_max, next.wv);
      }
      settle(t, 0, 8);
#pragma unroll
      for (int p = 0; p < 8; p++) {
        if (m == 0) pair_stage<1, kE>(t, p, word0, word1, min_max, next.wv);
        else pair_stage<3, kE>(t, p, word0, word1, min_max, next.wv);
      }
      if (m == 0) settle(t, 0, 8);
      else asm volatile("" : "+v"(next.wv[0]), "+v"(next.wv[1]));
    }
    extra(m);
    __builtin_amdgcn_sched_barrier(0);
  }
  lds_arrived_blocks<kLive>(next.xa);
  now = next;
}

template <int kRG, int kKP, int kNB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(kNB == 2 || kRG == 4 ? 2 : 1, 4)))
void matvec_tiles_shared_kernel(TileArgs a) {
  static_assert(kRG * kKP == 4 && (kNB == 2 || kNB == 4), "four wavefronts");
  constexpr int kTile = kNB * 32 * 256;        // a window of activations
  constexpr int kLoads = 8 * kNB / kRG;        // of them this wavefront's loads
  static_assert(kLoads % 4 == 0, "whole groups of sixteen tokens per wavefront");
  extern __shared__ __align__(16384) unsigned char shared_tiles[];   // [part][2][kTile]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = wave % kRG, k = wave / kRG;
  const int blocks = a.units_down / 2;
  TileLane l;
  l.lane = threadIdx.x & 63;
  l.half = l.lane >> 5;
  l.block = blockIdx.x * kRG + g;
  const bool has_rows = l.block < blocks;
  l.t0 = blockIdx.y * (32 * kNB);
  l.rows_here = min(32 * kNB, a.tokens - l.t0);
  const int live = (l.rows_here + 31) / 32;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = l.block * kRows + j * kUnitRows + (l.lane & 31);
    l.min_max[j] = row < a.height ? a.minmax[static_cast<int64_t>(a.matrix) * a.height + row] : 0u;
    l.unit_at[j] = static_cast<uint32_t>(j * a.windows * 1024 + l.lane * 16);
  }
  l.get_at = static_cast<uint32_t>((l.lane & 31) * 256 + ((l.half ^ (l.lane & 15)) << 4));
  Fetch f = fetch_of(a, l.lane);
#pragma unroll
  for (int u = 0; u < 4; u++) f.at[u] += static_cast<uint32_t>(g * (kLoads / 4)) * f.step;
  const lds_bytes part_tiles = (lds_bytes)shared_tiles + k * (2 * kTile);
  const int last = a.windows - 1;
  const bool ragged_edge = (a.width & (kCols - 1)) != 0;
  if (ragged_edge) {
    // places that no fetch writes must not hold what LDS happened to hold
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < 2 * kLoads; u++)
      *reinterpret_cast<u32x4 *>(shared_tiles + k * (2 * kTile) + ((g * 2 * kLoads + u) * 64 + l.lane) * 16) =
          zero;
    __syncthreads();
  }

  f32x16 acc[kNB][2];   // [32 tokens][32 rows] blocks
#pragma unroll
  for (int i = 0; i < kNB; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // Load u (0 .. kLoads - 1) of this wavefront's share of window w of the
  // activations, into tile `buffer` of its part; and its own codes of window w.
  auto issue_x = [&](const __amdgpu_buffer_rsrc_t &xb, int w, int buffer, int u) {
    const bool edge = ragged_edge && w == last;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        xb, part_tiles + buffer * kTile + g * (kLoads * 1024) + u * 1024, 16,
        edge && f.col[u & 3] >= a.width - w * kCols ? kOutside : f.at[u & 3] + (u >> 2) * f.step,
        w * (kCols * 2), 0, 0);
  };
  auto issue_codes = [&](int w, u32x4 (&codes)[2]) {
    const __amdgpu_buffer_rsrc_t ub =
        units_of(a, has_rows ? l.block : 0, has_rows && w < a.windows);
#pragma unroll
    for (int j = 0; j < 2; j++)
      codes[j] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(ub, l.unit_at[j], w * 1024, 0));
  };

  // The first two windows of this part are asked for at once; from then on
  // the window after the next is asked for during the last step of a window,
  // into the tile and the registers that this window has just finished with.
  const int turns = (a.windows + kKP - 1) / kKP;
  u32x4 codes_a[2], codes_b[2];
  {
    const __amdgpu_buffer_rsrc_t x0 = tokens_of(a, l, k < a.windows);
    const __amdgpu_buffer_rsrc_t x1 = tokens_of(a, l, k + kKP < a.windows);
#pragma unroll
    for (int u = 0; u < kLoads; u++) issue_x(x0, k, 0, u);
    issue_codes(k, codes_a);
#pragma unroll
    for (int u = 0; u < kLoads; u++) issue_x(x1, k + kKP, 1, u);
    issue_codes(k + kKP, codes_b);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const uint32_t tile_at[2] = {
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part_tiles)) + l.get_at,
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>(part_tiles + kTile)) + l.get_at};

  auto run = [&](auto live_c) {
    constexpr int kLive = decltype(live_c)::value;
    constexpr int kSlots = 2 * kLive;                          // MFMAs of a step
    constexpr int kPerSlot = (kLoads + kSlots - 1) / kSlots;   // loads issued behind each
    StepOperands<kLive> now;
    lds_request_blocks<kLive>(tile_at[0], now.xa);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) now.wv[j][q] = weight_pair(codes_a[j][0], q, l.min_max[j]);
    lds_arrived_blocks<kLive>(now.xa);
    auto nothing = [](int) {};
    // one window: the tile and codes `cur`, then on to `nxt`
    auto turn_of = [&](int turn, int cur, u32x4 (&codes_cur)[2], u32x4 (&codes_nxt)[2]) {
      const int w = __builtin_amdgcn_readfirstlane(k + turn * kKP);
      const int w2 = w + 2 * kKP;
      const __amdgpu_buffer_rsrc_t x2 = tokens_of(a, l, w2 < a.windows);
      if (has_rows && w < a.windows) {
        const uint32_t get = tile_at[cur];
        tile_step<kLive, kNB, 1>(now, get ^ 32u, codes_cur[0][0], codes_cur[1][0], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 0>(now, get ^ 64u, codes_cur[0][1], codes_cur[1][1], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 1>(now, get ^ 96u, codes_cur[0][1], codes_cur[1][1], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 0>(now, get ^ 128u, codes_cur[0][2], codes_cur[1][2], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 1>(now, get ^ 160u, codes_cur[0][2], codes_cur[1][2], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 0>(now, get ^ 192u, codes_cur[0][3], codes_cur[1][3], l.min_max, acc, nothing);
        tile_step<kLive, kNB, 1>(now, get ^ 224u, codes_cur[0][3], codes_cur[1][3], l.min_max, acc, nothing);
        // the next window is there (this wavefront's share of it, and after
        // the barrier everyone's), and everyone has read the last of this one
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const uint32_t word0 = codes_nxt[0][0], word1 = codes_nxt[1][0];
        tile_step<kLive, kNB, 0>(now, tile_at[cur ^ 1], word0, word1, l.min_max, acc, [&](int m) {
#pragma unroll
          for (int u = m * kPerSlot; u < (m + 1) * kPerSlot && u < kLoads; u++) issue_x(x2, w2, cur, u);
          if (m == kSlots - 1) issue_codes(w2, codes_cur);
        });
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kLoads; u++) issue_x(x2, w2, cur, u);
        issue_codes(w2, codes_cur);
      }
    };
    for (int turn = 0; turn < turns; turn += 2) {
      turn_of(turn, 0, codes_a, codes_b);
      if (turn + 1 < turns) turn_of(turn + 1, 1, codes_b, codes_a);
    }
  };
  if (live > kNB / 2)
    run(std::integral_constant<int, kNB>{});
  else
    run(std::integral_constant<int, kNB / 2>{});
  // nothing is on its way into LDS any more and everyone has read its last
  // window; then the sums take the place of the activations, 32 tokens at a time
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  float *sums = reinterpret_cast<float *>(shared_tiles);   // [wavefront][32 tokens][64 rows]
  const int pair = l.lane & 31;                            // rows 2 pair, 2 pair + 1 of the group
  const int row = l.block * kRows + 2 * pair;
  const __amdgpu_buffer_rsrc_t yb = buffer_over(
      a.y + static_cast<int64_t>(l.t0) * a.ldy,
      static_cast<uint32_t>((static_cast<int64_t>(l.rows_here - 1) * a.ldy + a.height) * 2));
  const uint32_t y_at = has_rows && row < a.height ? static_cast<uint32_t>(row * 2) : kOutside;
  const uint32_t y_step = static_cast<uint32_t>(a.ldy * 2);
  constexpr int kMine = 16 / kKP;   // pairs of tokens of a block that this wavefront finishes
#pragma unroll
  for (int i = 0; i < kNB; i++) {
    if (i >= live) break;
    uint32_t before[kMine];
#pragma unroll
    for (int n = 0; n < kMine; n++)
      before[n] = __builtin_amdgcn_raw_buffer_load_b32(
          yb, y_at + (32 * i + k * (32 / kKP) + 2 * n + l.half) * y_step, 0, 0);
    // Element (token t, row r) of an accumulator block sits in lane
    // r + 32 * ((t / 4) % 2), register 4 * (t / 8) + t % 4.
    float *mine = sums + wave * (32 * kRows);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++)
        mine[(8 * (v >> 2) + 4 * l.half + (v & 3)) * kRows + j * 32 + (l.lane & 31)] = acc[i][j][v];
    if (kKP > 1) __syncthreads();
#pragma unroll
    for (int n = 0; n < kMine; n++) {
      const int t = k * (32 / kKP) + 2 * n + l.half;
      const float *at = sums + g * (32 * kRows) + t * kRows + 2 * pair;
      float lo = at[0], hi = at[1];
#pragma unroll
      for (int part = 1; part < kKP; part++) {
        lo += at[part * kRG * (32 * kRows)];
        hi += at[part * kRG * (32 * kRows) + 1];
      }
      const uint32_t was = before[n];
      const uint32_t now =
          static_cast<uint32_t>(f32_to_bf16(bf16_to_f32(static_cast<uint16_t>(was & 0xffffu)) +
                                            bf16_to_f32(f32_to_bf16(lo)))) |
          static_cast<uint32_t>(f32_to_bf16(bf16_to_f32(static_cast<uint16_t>(was >> 16)) +
                                            bf16_to_f32(f32_to_bf16(hi)))) << 16;
      __builtin_amdgcn_raw_buffer_store_b32(now, yb, y_at + (32 * i + t) * y_step, 0, 0);
    }
    if (kKP > 1) __syncthreads();
  }
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

// Estimated microseconds of a launch on `tiles` blocks of 64 tokens, for a
// matrix of `blocks` blocks of 64 rows and `windows` windows cut into n parts
// (fitted to measurements on the six Switch shapes at 64 to 2272 tokens).
// matvec_tiles_kernel<n>: rounds of workgroups over the chip, four wavefronts a
// compute unit (36 KB of LDS each), each round 4 us plus 1.25 us per window that
// a wavefront walks.
double cost_own_tiles(int blocks, int windows, int n, int64_t tiles) {
  const int64_t slots = 256 * (kMaxWaves / n);
  const int64_t rounds = (blocks * tiles + slots - 1) / slots;
  return rounds * (4.0 + 1.25 * ((windows + n - 1) / n));
}
// matvec_tiles_shared_kernel<4 / n, n, 2>: 1.35 us per window of a part; a
// compute unit holds three such workgroups with one part and two with two, and
// each one beyond the first slows the others by 0.6 of its time; more
// workgroups than that follow as the first ones end.
double cost_shared_tiles(int blocks, int windows, int n, int64_t tiles) {
  const int groups = kMaxWaves / n, cap = n == 1 ? 3 : 2;
  const int64_t workgroups = (blocks + groups - 1) / groups * tiles;
  const int64_t per_unit = std::min<int64_t>(cap, (workgroups + 255) / 256);
  const double fill = static_cast<double>(workgroups) / (256.0 * cap);
  const double rounds = fill <= 1.0 ? 1.0 : 0.5 * (std::ceil(fill) + fill);
  return rounds * (4.0 + 1.35 * ((windows + n - 1) / n) * (1.0 + 0.6 * (per_unit - 1)));
}

// Parts that the windows of a matrix are cut into: 1, 2 or 4, whichever is
// estimated fastest at nine blocks of tokens (568, the longest sequence of the
// Switch encoders) by the better of the two kernels.  The choice depends on
// the matrix alone, never on the tokens of a launch, and the parts are added in
// the same order by both kernels: a token's result is the same whatever launch
// it is part of.
std::atomic<int> g_forced_kernel{0};   // sub1_test_tiles_kernel

int pick_waves(int blocks, int windows) {
  int best = 1;
  double best_cost = 0;
  for (int n = 1; n <= kMaxWaves; n *= 2) {
    double cost = cost_own_tiles(blocks, windows, n, 9);
    if (n <= 2) cost = std::min(cost, cost_shared_tiles(blocks, windows, n, 9));
    if (n == 1 || cost < best_cost - 1e-9) {
      best = n;
      best_cost = cost;
    }
  }
  return best;
}

template <int kRG, int kKP, int kNB>
int launch_shared_as(const TileArgs &a, int blocks, hipStream_t stream) {
  constexpr int lds = kKP * 2 * kNB * 32 * 256;
  static_assert(lds >= 4 * 32 * kRows * 4 && lds <= 160 * 1024, "tiles, then the sums of four wavefronts");
  HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(matvec_tiles_shared_kernel<kRG, kKP, kNB>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  const dim3 grid((blocks + kRG - 1) / kRG, (a.tokens + 32 * kNB - 1) / (32 * kNB));
  matvec_tiles_shared_kernel<kRG, kKP, kNB><<<grid, 256, lds, stream>>>(a);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

int launch_shared(const TileArgs &a, int parts, int token_blocks, int blocks, hipStream_t stream) {
  sub1::note_kernel(token_blocks == 4 ? "matvec_tiles_shared_kernel<128>" : "matvec_tiles_shared_kernel<64>");
  if (parts == 1) return token_blocks == 4 ? launch_shared_as<4, 1, 4>(a, blocks, stream)
                                           : launch_shared_as<4, 1, 2>(a, blocks, stream);
  if (parts == 2) return token_blocks == 4 ? launch_shared_as<2, 2, 4>(a, blocks, stream)
                                           : launch_shared_as<2, 2, 2>(a, blocks, stream);
  return launch_shared_as<1, 4, 2>(a, blocks, stream);
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
  if (tokens < 0 || tokens > 65535 * kTokens)   // (a grid's second dimension)
    return fail(SUB1_ERR_SHAPE, "%s: tokens %d outside 0..%d", who, tokens, 65535 * kTokens);
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ldx >= (1 << 24) || ldy >= (1 << 24))
    return fail(SUB1_ERR_SHAPE, "%s: token strides of 2^24 elements or more", who);
  const int waves = pick_waves(l.units_down / 2, l.windows);
  const bool shared_ok = wide && !misaligned(y, 4) && ldy % 2 == 0 && t->height % 2 == 0 &&
                         ldx < (1 << 22) && ldy < (1 << 22);
  // Which kernel: the one estimated faster for this many tokens (the sums and
  // their order are the same).  Workgroups that share their activations take
  // over where those of one wavefront's own tiles no longer fit the chip at
  // once (20 to 35% less time on the Switch shapes from there on); with four
  // parts they are no faster and are not used.  Blocks of 128 tokens where
  // blocks of 64 would make more such workgroups than the chip holds at once.
  const int blocks = l.units_down / 2;
  const int64_t tiles_of_64 = (tokens + kTokens - 1) / kTokens;
  const int forced = g_forced_kernel.load(std::memory_order_relaxed);
  if (shared_ok && forced >= 2) return launch_shared(a, waves, forced == 3 && waves < 4 ? 4 : 2, blocks, s);
  if (shared_ok && !forced && waves <= 2 &&
      cost_shared_tiles(blocks, l.windows, waves, tiles_of_64) <
          cost_own_tiles(blocks, l.windows, waves, tiles_of_64)) {
    const int groups = kMaxWaves / waves;
    const bool wide_blocks = waves == 1 && (blocks + groups - 1) / groups * tiles_of_64 > 3 * 256;
    return launch_shared(a, waves, wide_blocks ? 4 : 2, blocks, s);
  }
  const dim3 grid(l.units_down / 2, (tokens + kTokens - 1) / kTokens);
  sub1::note_kernel(wide ? "matvec_tiles_kernel" : "matvec_tiles_ragged_kernel");
  if (waves == 1) launch_tiles<1>(a, wide, grid, s);
  else if (waves == 2) launch_tiles<2>(a, wide, grid, s);
  else launch_tiles<4>(a, wide, grid, s);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_test_tiles_kernel(int which) {
  if (which < 0 || which > 3) return fail(SUB1_ERR_SHAPE, "sub1_test_tiles_kernel: no kernel %d", which);
  g_forced_kernel.store(which, std::memory_order_relaxed);
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
