// Many tokens through one compressed matrix on the matrix cores.
//
// Sub1Linear.forward on a sequence (reference sub1.py:132-143 launches one
// product per token and calls that "naive") is a skinny GEMM Y += X W^T: the
// weights are decoded ONCE per tile of 64 tokens into a dense bf16 tile in LDS
// and multiplied with the tokens' activations by v_mfma_f32_32x32x16_bf16,
// instead of walking the non-zeros once per token (or per four tokens) as the
// row-walking kernels do; the work no longer grows with tokens x non-zeros.
//
// The tile form of a matrix (sub1_tiles_*) is made for that, once, from the
// packed codes:
//   * rows stay in their own order, in blocks of 64 (a lane per row), so a
//     tile's outputs are 64 consecutive rows of y: coalesced read-modify-writes;
//   * columns are cut into windows of 128; a (block, window) segment lists, per
//     lane, the row's non-zero weights inside the window as one byte each,
//     (column in the window) * 2 + (symbol - 1), eight to a chunk of 8 bytes,
//     chunk c of lane l at ((segment base + c) * 64 + l) * 8 bytes as in the
//     prepared stream; a segment is as long as its fullest lane, each lane's
//     own count says where its bytes end;
//   * (min, max) per row, copied.
// Segments are independent, so a wavefront decodes a window with no state
// carried over from the windows before it.
//
// Kernel: a workgroup of four wavefronts owns 64 rows x 64 tokens.  Wavefront v
// takes the windows v, v + 4, ...: it zeroes its weight tile, writes the window's
// weights into it (bf16 values of the row's min or max), copies the tokens'
// activations of the same 128 columns next to it, and multiplies the two
// 64 x 128 tiles into its own 64 x 64 fp32 accumulators (2 x 2 MFMA blocks, one
// LDS read per MFMA).  The wavefronts never wait for each other inside the
// loop; at the end the four partial tiles are added through LDS in wavefront
// order, rounded to bf16 and added onto y in bf16 (reference
// sub1_cuda_kernel.cu:199-200).  The loads of a wavefront's next window (its
// chunks, its counts, the activations) are requested before it works on the
// current one.
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

constexpr int kRows = 64;                 // rows per block, a lane each
constexpr int kCols = 128;                // columns per window
constexpr int kPerChunk = 8;              // entries (bytes) per chunk
constexpr int kTokens = 64;               // tokens per workgroup
constexpr int kWaves = 4;                 // wavefronts per workgroup
// bf16 elements per LDS row of a tile: 272 bytes, so that the 16-byte operand
// reads of 32 consecutive rows fall into all banks evenly
constexpr int kStride = kCols + 8;
constexpr int kTileElems = kRows * kStride;
constexpr size_t kTilesLds = static_cast<size_t>(kWaves) * 2 * kTileElems * sizeof(uint16_t);
constexpr int kAhead = 4;                 // chunks of the next window requested ahead

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

// One block of device memory, arrays back to back, each 256-byte aligned.
struct TileLayout {
  int blocks, windows;
  int64_t segments;
  int64_t seg_base;   // i32 [segments + 1]: chunk counts, scanned in place
  int64_t cnt;        // u8  [segments * 64]: entries of every lane
  int64_t minmax;     // u32 [count * height]
  int64_t status;     // i32 [4]: [0] rows whose codes do not cover the width
  int64_t bytes;
};

TileLayout tile_layout(int count, int height, int width) {
  TileLayout t;
  t.blocks = (height + kRows - 1) / kRows;
  t.windows = (width + kCols - 1) / kCols;
  t.segments = static_cast<int64_t>(count) * t.blocks * t.windows;
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    int64_t o = off;
    off += align256(bytes);
    return o;
  };
  t.seg_base = take((t.segments + 1) * 4);
  t.cnt = take(t.segments * kRows);
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

// One thread per lane of every block: the entries of its row in every window.
__global__ __launch_bounds__(256) void tile_count_kernel(RowSource s, int blocks, int windows,
                                                         uint8_t *__restrict__ cnt,
                                                         int32_t *__restrict__ status,
                                                         int64_t lanes_total) {
  const int64_t gl = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gl >= lanes_total) return;
  const int lane = static_cast<int>(gl & 63);
  const int64_t mb = gl >> 6;                 // matrix * blocks + block
  const int m = static_cast<int>(mb / blocks);
  const int r = static_cast<int>(mb % blocks) * kRows + lane;
  uint8_t *mine = cnt + mb * windows * kRows + lane;   // [window * 64]
  int w_cur = 0, n_cur = 0;
  auto flush_to = [&](int w) {
    while (w_cur < w) {
      mine[static_cast<int64_t>(w_cur) * kRows] = static_cast<uint8_t>(n_cur);
      n_cur = 0;
      w_cur++;
    }
  };
  if (r < s.height) {
    int n;
    const uint16_t *codes = codes_of(s, m, r, n);
    const int covered = each_nonzero(codes, n, s.dec, s.width, [&](int col, int) {
      flush_to(col / kCols);
      n_cur++;
    });
    if (covered != ((s.width + 1) & ~1)) atomicAdd(&status[0], 1);
  }
  flush_to(windows);
}

// One thread per segment: its chunks are those of its fullest lane.
__global__ __launch_bounds__(256) void tile_segments_kernel(const uint8_t *__restrict__ cnt,
                                                            int32_t *__restrict__ counts,
                                                            int64_t segments) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= segments) return;
  const uint4 *p = reinterpret_cast<const uint4 *>(cnt + g * kRows);
  uint32_t most = 0;
  for (int i = 0; i < kRows / 16; i++) {
    const uint4 v = p[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    for (int j = 0; j < 4; j++)
      for (int k = 0; k < 4; k++) most = max(most, (w[j] >> (8 * k)) & 255u);
  }
  counts[g + 1] = static_cast<int32_t>((most + kPerChunk - 1) / kPerChunk);
}

// In-place inclusive prefix sum over v[1..n], v[0] = 0; one workgroup.
__global__ __launch_bounds__(1024) void tile_scan_kernel(int32_t *__restrict__ v, int64_t n) {
  __shared__ int32_t part[1024];
  const int tid = threadIdx.x;
  const int64_t seg = (n + 1023) / 1024;
  const int64_t lo = 1 + tid * seg;
  const int64_t hi = min(n + 1, lo + seg);
  int32_t s = 0;
  for (int64_t i = lo; i < hi; i++) s += v[i];
  part[tid] = s;
  __syncthreads();
  for (int d = 1; d < 1024; d *= 2) {
    int32_t t = tid >= d ? part[tid - d] : 0;
    __syncthreads();
    part[tid] += t;
    __syncthreads();
  }
  int32_t run = tid ? part[tid - 1] : 0;
  if (tid == 0) v[0] = 0;
  for (int64_t i = lo; i < hi; i++) {
    run += v[i];
    v[i] = run;
  }
}

// One thread per lane of every block: its entries into the segments.
__global__ __launch_bounds__(256) void tile_emit_kernel(RowSource s, int blocks, int windows,
                                                        const int32_t *__restrict__ seg_base,
                                                        uint8_t *__restrict__ dst,
                                                        int64_t lanes_total) {
  const int64_t gl = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gl >= lanes_total) return;
  const int lane = static_cast<int>(gl & 63);
  const int64_t mb = gl >> 6;
  const int m = static_cast<int>(mb / blocks);
  const int r = static_cast<int>(mb % blocks) * kRows + lane;
  if (r >= s.height) return;
  int n;
  const uint16_t *codes = codes_of(s, m, r, n);
  int w_cur = -1, i = 0;
  int64_t base = 0;
  each_nonzero(codes, n, s.dec, s.width, [&](int col, int sym) {
    const int w = col / kCols;
    if (w != w_cur) {
      w_cur = w;
      i = 0;
      base = seg_base[mb * windows + w];
    }
    dst[((base + i / kPerChunk) * kRows + lane) * 8 + i % kPerChunk] =
        static_cast<uint8_t>(((col - w * kCols) << 1) | (sym - 1));
    i++;
  });
}

// The symbols of one matrix back out of its tile form: out[row, column] = 1 or
// 2 at every entry; out is zero before.
__global__ __launch_bounds__(256) void tile_decode_kernel(const uint8_t *__restrict__ entries,
                                                          const int32_t *__restrict__ seg_base,
                                                          const uint8_t *__restrict__ cnt,
                                                          uint8_t *__restrict__ out, int matrix,
                                                          int blocks, int windows, int height,
                                                          int width) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= blocks * kRows) return;
  const int lane = t & 63, r = t;
  if (r >= height) return;
  const int64_t mb = static_cast<int64_t>(matrix) * blocks + (t >> 6);
  for (int w = 0; w < windows; w++) {
    const int64_t g = mb * windows + w;
    const int n = cnt[g * kRows + lane];
    const int64_t base = seg_base[g];
    for (int i = 0; i < n; i++) {
      const uint8_t e = entries[((base + i / kPerChunk) * kRows + lane) * 8 + i % kPerChunk];
      const int col = w * kCols + (e >> 1);
      if (col < width) out[static_cast<int64_t>(r) * width + col] = static_cast<uint8_t>((e & 1) + 1);
    }
  }
}

__global__ void tile_fill_kernel(uint8_t *p, int64_t n, uint8_t v) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void tile_copy_words_kernel(const uint32_t *src, uint32_t *dst, int64_t n) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

// --------------------------------------------------------------- product ---

struct TileArgs {
  const uint2 *entries;
  const int32_t *seg_base;
  const uint8_t *cnt;
  const uint32_t *minmax;
  const uint16_t *x;
  uint16_t *y;
  int64_t ldx, ldy;
  int height, width, tokens;
  int blocks, windows, matrix;
  int x_wide;   // x rows can be read 16 bytes at a time
};

// What a wavefront has requested for a window before it works on it.
struct WindowLoads {
  int32_t base, nch;          // the same in every lane
  int cnt;                    // this lane's entries
  uint2 chunk[kAhead];        // the segment's first chunks of this lane
  uint4 xv[kTokens * kCols / 8 / 64];   // this lane's 16-byte pieces of the activations
};

__device__ __forceinline__ WindowLoads request_window(const TileArgs &a, int64_t seg0, int w,
                                                      int t0) {
  const int lane = threadIdx.x & 63;
  WindowLoads l;
  const int64_t g = seg0 + w;
  l.base = a.seg_base[g];
  l.nch = a.seg_base[g + 1];
  l.cnt = a.cnt[g * kRows + lane];
  l.base = __builtin_amdgcn_readfirstlane(l.base);
  l.nch = __builtin_amdgcn_readfirstlane(l.nch) - l.base;
  const uint2 *p = a.entries + static_cast<int64_t>(l.base) * kRows + lane;
#pragma unroll
  for (int c = 0; c < kAhead; c++)
    l.chunk[c] = c < l.nch ? p[c * kRows] : make_uint2(0u, 0u);
  // 64 tokens x 128 columns = 1024 pieces of 8 elements; lane takes piece
  // i = lane + 64 * u: token i / 16, columns (i % 16) * 8 ...
  const int k0 = w * kCols;
#pragma unroll
  for (int u = 0; u < kTokens * kCols / 8 / 64; u++) {
    const int i = lane + 64 * u;
    const int t = t0 + (i >> 4), col = k0 + (i & 15) * 8;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (t < a.tokens && col < a.width) {
      const uint16_t *src = a.x + static_cast<int64_t>(t) * a.ldx + col;
      if (a.x_wide && col + 8 <= a.width) {
        v = *reinterpret_cast<const uint4 *>(src);
      } else {
        uint16_t e[8];
#pragma unroll
        for (int q = 0; q < 8; q++) e[q] = col + q < a.width ? src[q] : static_cast<uint16_t>(0);
        v = make_uint4(e[0] | (static_cast<uint32_t>(e[1]) << 16), e[2] | (static_cast<uint32_t>(e[3]) << 16),
                       e[4] | (static_cast<uint32_t>(e[5]) << 16), e[6] | (static_cast<uint32_t>(e[7]) << 16));
      }
    }
    l.xv[u] = v;
  }
  return l;
}

__global__ __launch_bounds__(64 * kWaves) void matvec_tiles_kernel(TileArgs a) {
  extern __shared__ __align__(16) uint16_t lds[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  uint16_t *wt = lds + wave * (2 * kTileElems);   // [64 rows][kStride]: the window's weights
  uint16_t *xt = wt + kTileElems;                 // [64 tokens][kStride]: its activations
  const int block = blockIdx.x, t0 = blockIdx.y * kTokens;
  const int row = block * kRows + lane;
  const uint32_t mm = row < a.height ? a.minmax[static_cast<int64_t>(a.matrix) * a.height + row] : 0u;
  const uint16_t w_min = static_cast<uint16_t>(mm & 0xffffu), w_max = static_cast<uint16_t>(mm >> 16);
  const int64_t seg0 = (static_cast<int64_t>(a.matrix) * a.blocks + block) * a.windows;
  f32x16 acc[2][2];   // [32 tokens][32 rows] blocks
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  WindowLoads cur;
  if (wave < a.windows) cur = request_window(a, seg0, wave, t0);
  for (int w = wave; w < a.windows; w += kWaves) {
    WindowLoads nxt;
    const bool more = w + kWaves < a.windows;
    if (more) nxt = request_window(a, seg0, w + kWaves, t0);
    // a clean tile; the LDS serves a wavefront's operations in order, so these
    // stores come before the decoded weights and after the last window's reads
    uint4 *wz = reinterpret_cast<uint4 *>(wt);
    for (int i = lane; i < kTileElems / 8; i += 64) wz[i] = make_uint4(0u, 0u, 0u, 0u);
    // the window's weights
    uint16_t *my_row = wt + lane * kStride;
    const int nch = __builtin_amdgcn_readfirstlane(cur.nch);   // uniform: scalar loop control
    const uint2 *p = a.entries +
                     static_cast<int64_t>(__builtin_amdgcn_readfirstlane(cur.base)) * kRows + lane;
    for (int c = 0; c < nch; c += kAhead) {
      uint2 cw[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; u++)
        cw[u] = c == 0 ? cur.chunk[u] : (c + u < nch ? p[(c + u) * kRows] : make_uint2(0u, 0u));
#pragma unroll
      for (int u = 0; u < kAhead; u++) {
        if (c + u < nch) {
#pragma unroll
          for (int j = 0; j < kPerChunk; j++) {
            const uint32_t word = j < 4 ? cw[u].x : cw[u].y;
            const uint32_t e = (word >> (8 * (j & 3))) & 255u;
            if ((c + u) * kPerChunk + j < cur.cnt) my_row[e >> 1] = (e & 1u) ? w_max : w_min;
          }
        }
      }
    }
    // the tokens' activations of the same columns
#pragma unroll
    for (int u = 0; u < kTokens * kCols / 8 / 64; u++) {
      const int i = lane + 64 * u;
      *reinterpret_cast<uint4 *>(xt + (i >> 4) * kStride + (i & 15) * 8) = cur.xv[u];
    }
    // 64 tokens x 64 rows += activations x weights^T over the 128 columns
#pragma unroll
    for (int kk = 0; kk < kCols; kk += 16) {
      const int at = (lane & 31) * kStride + kk + 8 * (lane >> 5);
      bf16x8 xa[2], wb[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        xa[i] = *reinterpret_cast<const bf16x8 *>(xt + i * 32 * kStride + at);
        wb[i] = *reinterpret_cast<const bf16x8 *>(wt + i * 32 * kStride + at);
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[i], wb[j], acc[i][j], 0, 0, 0);
    }
    if (more) cur = nxt;
  }

  // The four wavefronts' partial tiles, added in wavefront order.  Element
  // (token i, row j) of an accumulator block sits in lane j + 32 * ((i / 4) % 2),
  // register 4 * (i / 8) + i % 4.
  __syncthreads();   // every wavefront is done with its tiles
  float *red = reinterpret_cast<float *>(lds) + wave * (kTokens * kRows);
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int token = i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int r = j * 32 + (lane & 31);
        red[token * kRows + r] = acc[i][j][v];
      }
  __syncthreads();
  if (row < a.height) {
    const float *all = reinterpret_cast<const float *>(lds);
    for (int t = wave; t < kTokens && t0 + t < a.tokens; t += kWaves) {
      const int at = t * kRows + lane;
      const float sum = ((all[at] + all[kTokens * kRows + at]) + all[2 * kTokens * kRows + at]) +
                        all[3 * kTokens * kRows + at];
      uint16_t *dst = a.y + static_cast<int64_t>(t0 + t) * a.ldy + row;
      // reference sub1_cuda_kernel.cu:200: y[row] += bf16(res), the sum in bf16
      *dst = f32_to_bf16(bf16_to_f32(*dst) + bf16_to_f32(f32_to_bf16(sum)));
    }
  }
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
  if (t->meta_bytes < tile_layout(t->count, t->height, t->width).bytes)
    return fail(SUB1_ERR_SHAPE, "%s: meta smaller than its layout", who);
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
  int rc = check_set(ms, who);
  if (rc) return rc;
  if (!meta || !out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (misaligned(meta, 256)) return fail(SUB1_ERR_ALIGN, "%s: meta must be 256-byte aligned", who);
  const TileLayout t = tile_layout(ms->count, ms->height, ms->width);
  if (meta_bytes < t.bytes)
    return fail(SUB1_ERR_SHAPE, "%s: meta needs %lld bytes", who, static_cast<long long>(t.bytes));
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *base = static_cast<char *>(meta);
  int32_t *counts = reinterpret_cast<int32_t *>(base + t.seg_base);
  uint8_t *cnt = reinterpret_cast<uint8_t *>(base + t.cnt);
  int32_t *status = reinterpret_cast<int32_t *>(base + t.status);
  tile_fill_kernel<<<1, 64, 0, s>>>(reinterpret_cast<uint8_t *>(status), 16, 0);
  const int64_t lanes = static_cast<int64_t>(ms->count) * t.blocks * kRows;
  tile_count_kernel<<<static_cast<unsigned>((lanes + 255) / 256), 256, 0, s>>>(
      source_of(ms), t.blocks, t.windows, cnt, status, lanes);
  tile_segments_kernel<<<static_cast<unsigned>((t.segments + 255) / 256), 256, 0, s>>>(cnt, counts,
                                                                                        t.segments);
  tile_scan_kernel<<<1, 1024, 0, s>>>(counts, t.segments);
  const int64_t words = static_cast<int64_t>(ms->count) * ms->height;
  tile_copy_words_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, s>>>(
      static_cast<const uint32_t *>(ms->ter_minmax), reinterpret_cast<uint32_t *>(base + t.minmax),
      words);
  HIP_TRY(hipGetLastError());
  int32_t bad = 0, total = 0;
  HIP_TRY(hipMemcpyAsync(&bad, status, 4, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipMemcpyAsync(&total, counts + t.segments, 4, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  if (bad) return fail(SUB1_ERR_SHAPE, "%s: the codes of %d rows do not cover the width", who, bad);
  if (total < 0) return fail(SUB1_ERR_SHAPE, "%s: too many entries", who);
  out->meta = meta;
  out->entries = nullptr;
  out->meta_bytes = t.bytes;
  out->total_chunks = total;
  out->entry_bytes = align256(static_cast<int64_t>(total) * kRows * 8 + 256);
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
  if (t->total_chunks < 0 || t->entry_bytes < t->total_chunks * kRows * 8)
    return fail(SUB1_ERR_SHAPE, "%s: entries buffer smaller than the layout needs", who);
  const TileLayout l = tile_layout(t->count, t->height, t->width);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const char *base = static_cast<const char *>(t->meta);
  const int64_t lanes = static_cast<int64_t>(ms->count) * l.blocks * kRows;
  tile_emit_kernel<<<static_cast<unsigned>((lanes + 255) / 256), 256, 0, s>>>(
      source_of(ms), l.blocks, l.windows, reinterpret_cast<const int32_t *>(base + l.seg_base),
      static_cast<uint8_t *>(const_cast<void *>(t->entries)), lanes);
  HIP_TRY(hipGetLastError());
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
  a.entries = static_cast<const uint2 *>(t->entries);
  a.seg_base = reinterpret_cast<const int32_t *>(base + l.seg_base);
  a.cnt = reinterpret_cast<const uint8_t *>(base + l.cnt);
  a.minmax = reinterpret_cast<const uint32_t *>(base + l.minmax);
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.ldx = ldx;
  a.ldy = ldy;
  a.height = t->height;
  a.width = t->width;
  a.tokens = tokens;
  a.blocks = l.blocks;
  a.windows = l.windows;
  a.matrix = matrix;
  a.x_wide = !misaligned(x, 16) && ldx % 8 == 0;
  HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(matvec_tiles_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kTilesLds)));
  const dim3 grid(l.blocks, (tokens + kTokens - 1) / kTokens);
  sub1::note_kernel("matvec_tiles_kernel");
  matvec_tiles_kernel<<<grid, 64 * kWaves, kTilesLds, static_cast<hipStream_t>(stream)>>>(a);
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
  const char *base = static_cast<const char *>(t->meta);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = static_cast<int64_t>(t->height) * t->width;
  tile_fill_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(
      static_cast<uint8_t *>(tern_out), n, 0);
  tile_decode_kernel<<<(l.blocks * kRows + 255) / 256, 256, 0, s>>>(
      static_cast<const uint8_t *>(t->entries), reinterpret_cast<const int32_t *>(base + l.seg_base),
      reinterpret_cast<const uint8_t *>(base + l.cnt), static_cast<uint8_t *>(tern_out), matrix,
      l.blocks, l.windows, t->height, t->width);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}
