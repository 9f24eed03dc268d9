// Prepared expert stack: the fast form of the grouped expert launch.
//
// sub1_moe_prepare_* turn an expert stack in the reference's packed layout
// (reference sub1.py:114-130: one row-major code stream per matrix plus
// row_off) into a form the GPU can stream at full width:
//
//   * every row's dictionary codes are decoded once and its non-zero weights
//     written as a gap-coded stream: 7-bit entries, each the distance to the
//     next non-zero in units of the LDS activation array (2 dwords per column:
//     the activation for a row-min weight and for a row-max weight; every 17th
//     column is a zero column), so an entry names the column and the symbol at
//     once; gaps beyond 127 units step over zero columns.  At 10% non-zeros
//     this is 0.72 bit per weight against 0.69 for the dictionary codes, and
//     the kernel needs no decode table;
//   * rows of every matrix are ordered by entry count and cut into slices of
//     64 rows (one wavefront lane each);
//   * a slice's entries are interleaved in chunks of 9 (8 bytes) per lane:
//     chunk c of lane l sits at slice_base*512 + (c*64 + l)*8 bytes, so one
//     wavefront load fetches 512 contiguous bytes and every byte of a cache
//     line is used; lanes are padded to the slice's longest row with entries
//     that stay on a zero dword.
//
// The kernels then walk 64 rows per wavefront: per entry one address add, one
// LDS read of a bf16 pair (x, 0) or (0, x), and one v_dot2c_f32_bf16 with the
// row's (min, max) pair, which adds x * min or x * max onto the row's fp32 sum;
// no cross-lane traffic at all.  They compute what reference
// sub1_cuda_kernel.cu:163-201 computes per row.
// Four kernels share that loop and give the same bits:
// moe_prepared_fused_kernel streams whole tokens (wi, ReLU, wo in one
// workgroup, h kept in LDS) when there is at least a token per compute unit;
// moe_prepared_shared_kernel lets several workgroups share a token, each in
// both projections, when there are fewer tokens than half the compute units;
// moe_prepared_kernel streams tiles of one matrix (persistent grid, a wavefront
// per slice, the next slice's loads in flight) for the batches in between and
// for single matrices; moe_prepared_small_kernel is the latency form for a
// handful of tokens through single matrices (wavefronts share a slice from
// position checkpoints).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

#include "sub1_common.h"

namespace {

using sub1::bf16_to_f32;
using sub1::f32_to_bf16;
using sub1::fail;
using sub1::misaligned;

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kMaxThreads = 1024;    // 16 wavefronts per workgroup
constexpr int kFields = 9;           // entries per lane per chunk (7 bits each in 8 bytes)
constexpr int kFieldBits = 7;
constexpr int kMaxStep = 127;        // the largest entry
constexpr int kRing = 4;             // chunks in flight per lane (2 KB per wavefront)
constexpr int kGroupChunks = 8;      // chunks (72 entries) per partial sum, a multiple of kRing
constexpr int kSplitRing = 8;        // chunks in flight per lane where wavefronts share a slice
constexpr int kMaxRowEntries = 16383; // entries per row the row ordering can count (widths to 12288)
using sub1::kCtrlBadIds;
using sub1::kCtrlGaveUp;
using sub1::kCtrlHeader;
using sub1::kCtrlTicket;
using sub1::kCtrlTiles;

// ------------------------------------------------------------- meta layout --
//
// One block of device memory, arrays back to back, each 256-byte aligned.
// Kind 0 = wi (rows d_ff, width d_model), kind 1 = wo.
struct KindMeta {
  int64_t slice_base;   // u32 [E*S] (+1): this kind's part of the scanned counts
  int64_t slice_len;    // u16 [E*S]: entries of the slice's longest row
  int64_t row_len;      // u16 [E*H]: entries of every row, in the matrix's own row order
  int64_t row_idx;      // u16 [E*S*64]
  int64_t minmax;       // u32 [E*S*64]
  int slices;           // S
  int height, width;
};

struct MetaLayout {
  KindMeta k[2];
  int kinds;
  int64_t counts;       // i32 [all slices + 1] chunk counts, scanned in place
  int64_t status;       // i32 [4]: [0] rows whose codes do not cover the width, [1], [2]
                        // longest slice of kind 0 / 1 in chunks
  int64_t bytes;
};

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

// kinds = 2: an expert stack (kind 0 = wi, rows d_ff; kind 1 = wo);
// kinds = 1: `experts` matrices of one shape.
MetaLayout meta_layout(int experts, int kinds, const int height[2], const int width[2]) {
  MetaLayout m;
  m.kinds = kinds;
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    int64_t o = off;
    off += align256(bytes);
    return o;
  };
  int64_t nslices = 0;
  int64_t first[2] = {0, 0};
  for (int i = 0; i < kinds; i++) {
    KindMeta &k = m.k[i];
    k.height = height[i];
    k.width = width[i];
    k.slices = (height[i] + 63) / 64;
    int64_t es = static_cast<int64_t>(experts) * k.slices;
    first[i] = nslices;
    nslices += es;
    k.slice_len = take(es * 2);
    k.row_len = take(static_cast<int64_t>(experts) * height[i] * 2);
    k.row_idx = take(es * 64 * 2);
    k.minmax = take(es * 64 * 4);
  }
  m.counts = take((nslices + 1) * 4);
  for (int i = 0; i < kinds; i++) m.k[i].slice_base = m.counts + first[i] * 4;
  m.status = take(16);
  m.bytes = off;
  return m;
}

MetaLayout moe_layout(int experts, int d_model, int d_ff) {
  const int h[2] = {d_ff, d_model}, w[2] = {d_model, d_ff};
  return meta_layout(experts, 2, h, w);
}

MetaLayout matrix_layout(int count, int height, int width) {
  const int h[2] = {height, 0}, w[2] = {width, 0};
  return meta_layout(count, 1, h, w);
}

// ---------------------------------------------------------- prepare kernels --

// Calls nz(column, symbol) for every non-zero weight of a row, in column order,
// and returns the columns the row's codes cover.  Digit d of dictionary entry e
// is (dec[2e + d/14] >> (4 + 2 (d % 14))) & 3, the low nibble of dec[2e] the
// entry's pair count (reference sub1.py:60-72, sub1_cuda_kernel.cu:186-192).
template <class F>
__device__ __forceinline__ int for_each_nonzero(const uint16_t *codes, int n,
                                                const int32_t *__restrict__ dec, int width,
                                                F &&nz) {
  int col = 0;
  // the code after next and the next code's entry are asked for before this
  // code's digits are walked: a row is a chain of dependent loads otherwise
  int e_next = n > 1 ? codes[1] : 0;
  const int e_first = n > 0 ? codes[0] : 0;
  int32_t next0 = dec[2 * e_first], next1 = dec[2 * e_first + 1];
  for (int i = 0; i < n; i++) {
    const uint32_t w0 = static_cast<uint32_t>(next0);
    const uint32_t w1 = static_cast<uint32_t>(next1);
    if (i + 1 < n) {
      next0 = dec[2 * e_next];
      next1 = dec[2 * e_next + 1];
    }
    if (i + 2 < n) e_next = codes[i + 2];
    unsigned long long digits = static_cast<unsigned long long>(w0 >> 4) |
                                (static_cast<unsigned long long>(w1 >> 4) << 28);
    while (digits) {
      const int d = (__ffsll(digits) - 1) >> 1;
      const int sym = static_cast<int>(digits >> (2 * d)) & 3;
      digits &= ~(3ull << (2 * d));
      if (col + d < width) nz(col + d, sym);   // digits past the width are dropped
    }
    col += 2 * static_cast<int>(w0 & 15u);
  }
  return col;
}

// A slice is as long as its longest row, counted in ENTRIES; its chunks, and how
// many entries of the last one are walked (1..9; the rest of that chunk is
// padding nobody reads).
__host__ __device__ constexpr int chunks_of(int len) { return (len + kFields - 1) / kFields; }
__host__ __device__ constexpr int last_entries_of(int len) { return len - kFields * (chunks_of(len) - 1); }

// Positions.  The kernels keep the activations in LDS by physical column: real
// column c is physical column q = c + c/16 + 1, so that every 17th physical
// column (0, 17, 34, ...) is a zero column; a physical column is two dwords,
// and position p = 2q + (symbol - 1) is the dword a weight with that symbol
// reads: (x, 0) for a row-min weight, (0, x) for a row-max weight, zero in a
// zero column.  The low bit of a position is the symbol, the rest the column.
constexpr int kZeroPeriod = 17;                  // physical columns from one zero column to the next
__host__ __device__ constexpr int physical_column(int c) { return c + (c >> 4) + 1; }
__host__ __device__ constexpr int position_of(int c, int sym) {
  return 2 * physical_column(c) + (sym - 1);
}
// Physical columns an array for `width` real columns needs: up to and including
// the zero column that follows the last real one.
__host__ __device__ constexpr int physical_columns(int width) {
  return (physical_column(width - 1) / kZeroPeriod + 1) * kZeroPeriod + 1;
}

// Non-zeros to entries.  An entry is the step from the row's position (0 at
// the start) to the next, 0..127.  A longer gap goes over zero columns, as far
// as each step reaches; after the last non-zero the row parks on the next zero
// column, where steps of 0 pad it to the length of its slice.
struct EntryWriter {
  int j = 0;
  template <class E>
  __device__ __forceinline__ void nonzero(int col, int sym, E &&emit) {
    const int target = position_of(col, sym);
    while (target - j > kMaxStep) {
      const int z = (j + kMaxStep) / (2 * kZeroPeriod) * (2 * kZeroPeriod);
      emit(z - j, j);
      j = z;
    }
    emit(target - j, j);
    j = target;
  }
  template <class E>
  __device__ __forceinline__ void park(E &&emit) {
    if ((j >> 1) % kZeroPeriod == 0) return;
    const int z = (j + 2 * kZeroPeriod - 1) / (2 * kZeroPeriod) * (2 * kZeroPeriod);
    emit(z - j, j);
    j = z;
  }
};

// Where the matrices of one kind come from: one buffer of codes with a base
// offset per matrix and [count, height + 1] / [count, height] arrays of row
// offsets and (min, max) - an expert stack - or, with the *_of tables set, a
// device array of device pointers per buffer, one entry per matrix - the
// layers' own tensors, wherever they lie.
struct KindSource {
  const uint16_t *w_comp;
  const int64_t *code_base;      // NULL with one matrix: its codes start at w_comp
  const int32_t *row_off;
  const uint32_t *minmax;
  const uint16_t *const *w_comp_of;
  const int32_t *const *row_off_of;
  const uint32_t *const *minmax_of;
};

__device__ __forceinline__ const uint16_t *row_codes(const KindSource &ks, int e, int r,
                                                     int height, int width, int &n) {
  const int32_t *ro = ks.row_off_of ? ks.row_off_of[e]
                                    : ks.row_off + static_cast<int64_t>(e) * (height + 1);
  n = ro[r + 1] - ro[r];
  if (n < 1 || n > (width + 1) / 2) n = 0;   // counted as a bad row by count_entries_kernel
  const uint16_t *codes = ks.w_comp_of ? ks.w_comp_of[e]
                                       : ks.w_comp + (ks.code_base ? ks.code_base[e] : 0);
  return codes + ro[r];
}

// One thread per row: how many entries its non-zeros take (the step onto a zero
// column that a padded row makes after them is not counted: it fits the padding).
__global__ __launch_bounds__(256) void count_entries_kernel(
    KindSource ks, const int32_t *__restrict__ dec, uint16_t *__restrict__ row_len,
    int32_t *__restrict__ status, int height, int width, int64_t rows_total) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= rows_total) return;
  const int e = static_cast<int>(g / height);
  const int r = static_cast<int>(g % height);
  int n;
  const uint16_t *codes = row_codes(ks, e, r, height, width, n);
  int entries = 0;
  auto emit = [&](int, int) { entries++; };
  EntryWriter wr;
  const int covered =
      for_each_nonzero(codes, n, dec, width, [&](int col, int sym) { wr.nonzero(col, sym, emit); });
  // a row's codes cover its width rounded up to a whole pair, exactly
  if (covered != ((width + 1) & ~1)) atomicAdd(&status[0], 1);
  row_len[g] = static_cast<uint16_t>(min(entries, kMaxRowEntries));
}

// One workgroup per matrix: order the rows by entry count, longest first, and
// describe the 64-row slices.  The order is a counting sort carried out by one
// thread, so it is the same on every run.  Dynamic LDS: the histogram
// (kMaxRowEntries + 2 counters), then the entry count of the first row of up to
// 1024 slices.
constexpr size_t kOrderRowsLds = (kMaxRowEntries + 2 + 1024) * sizeof(int);
__global__ __launch_bounds__(256) void order_rows_kernel(
    const uint16_t *__restrict__ row_len_all, KindSource ks,
    uint16_t *__restrict__ row_idx, uint32_t *__restrict__ minmax_sorted,
    uint16_t *__restrict__ slice_len, int32_t *__restrict__ counts,
    int32_t *__restrict__ status, int height, int slices, int kind) {
  extern __shared__ int order_lds[];
  int *hist = order_lds;
  int *first_len = order_lds + kMaxRowEntries + 2;
  const int e = blockIdx.x;
  const uint16_t *rl = row_len_all + static_cast<int64_t>(e) * height;
  const uint32_t *mm = ks.minmax_of ? ks.minmax_of[e] : ks.minmax + static_cast<int64_t>(e) * height;
  const int64_t lane0 = static_cast<int64_t>(e) * slices * 64;
  for (int i = threadIdx.x; i < kMaxRowEntries + 2; i += blockDim.x) hist[i] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < height; r += blockDim.x)
    atomicAdd(&hist[min(static_cast<int>(rl[r]), kMaxRowEntries)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;  // rows with a larger count come first
    for (int len = kMaxRowEntries; len >= 0; len--) {
      int n = hist[len];
      hist[len] = run;
      run += n;
    }
    for (int r = 0; r < height; r++) {
      const int len = min(static_cast<int>(rl[r]), kMaxRowEntries);
      int p = hist[len]++;
      row_idx[lane0 + p] = static_cast<uint16_t>(r);
      minmax_sorted[lane0 + p] = mm[r];
      if ((p & 63) == 0 && (p >> 6) < 1024) first_len[p >> 6] = len;
    }
  }
  for (int p = height + threadIdx.x; p < slices * 64; p += blockDim.x) {
    row_idx[lane0 + p] = 0xffffu;
    minmax_sorted[lane0 + p] = 0u;
  }
  __syncthreads();
  for (int s = threadIdx.x; s < slices; s += blockDim.x) {
    // a slice is as long as its first row, and at least one entry
    int len = s < 1024 ? first_len[s] : static_cast<int>(rl[row_idx[lane0 + 64 * s]]);
    len = max(len, 1);
    int64_t g = static_cast<int64_t>(e) * slices + s;
    slice_len[g] = static_cast<uint16_t>(len);
    counts[g + 1] = chunks_of(len);
    atomicMax(&status[1 + kind], chunks_of(len));
  }
}

// In-place inclusive prefix sum over v[1..n], v[0] = 0; one workgroup.
__global__ __launch_bounds__(1024) void scan_counts_kernel(int32_t *__restrict__ v, int n) {
  __shared__ int32_t part[1024];
  const int tid = threadIdx.x;
  const int seg = (n + 1023) / 1024;
  const int lo = 1 + tid * seg;
  const int hi = min(n + 1, lo + seg);
  int32_t s = 0;
  for (int i = lo; i < hi; i++) s += v[i];
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
  for (int i = lo; i < hi; i++) {
    run += v[i];
    v[i] = run;
  }
}

// Position checkpoints.  For every slice and every group of kGroupChunks chunks,
// the position at which each lane's row stands when the group begins: 64 x u16
// per group, groups of slice g stored from entry slice_base[g]/kGroupChunks + g
// on.  With them a wavefront can start in the middle of a slice, which is how a
// small batch is spread over the GPU.
__device__ __forceinline__ int64_t checkpoint_entry(uint32_t slice_base, int64_t slice) {
  return static_cast<int64_t>(slice_base / kGroupChunks) + slice;
}

// One thread per lane of every slice: the row's entries into the interleaved
// stream, nine to a chunk; a row shorter than its slice then steps onto the
// next zero column and stays there (steps of 0) to the end of the slice's last
// chunk; and the row's position at the start of every group of chunks into the
// checkpoints.
__global__ __launch_bounds__(256) void emit_entries_kernel(
    KindSource ks, const int32_t *__restrict__ dec,
    const uint32_t *__restrict__ slice_base, const uint16_t *__restrict__ slice_len,
    const uint16_t *__restrict__ row_idx, uint2 *__restrict__ dst, uint16_t *__restrict__ ckpt,
    int height, int width, int slices, int64_t first_slice, int64_t lanes_total) {
  const int64_t gl = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gl >= lanes_total) return;
  const int64_t slice = gl >> 6;
  const int ln = static_cast<int>(gl & 63);
  const int e = static_cast<int>(slice / slices);
  const int ridx = row_idx[gl];
  const uint32_t base = slice_base[slice];
  const int len = slice_len[slice];
  const int nch = chunks_of(len);
  uint2 *d = dst + static_cast<int64_t>(base) * 64 + ln;
  uint16_t *ck = ckpt + checkpoint_entry(base, first_slice + slice) * 64 + ln;
  int c = 0, q = 0;
  unsigned long long w = 0;
  auto emit = [&](int step, int from) {
    if (c >= nch) return;   // the slice is as long as its longest row: not reached
    if (q == 0 && c % kGroupChunks == 0) ck[(c / kGroupChunks) * 64] = static_cast<uint16_t>(from);
    w |= static_cast<unsigned long long>(step) << (kFieldBits * q);
    if (++q == kFields) {
      d[c * 64] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
      c++;
      q = 0;
      w = 0;
    }
  };
  EntryWriter wr;
  if (ridx != 0xffff) {
    int n;
    const uint16_t *codes = row_codes(ks, e, ridx, height, width, n);
    for_each_nonzero(codes, n, dec, width, [&](int col, int sym) { wr.nonzero(col, sym, emit); });
    if (c * kFields + q < len) wr.park(emit);   // padding follows: it must read zeros
  }
  while (c < nch) emit(0, wr.j);
}

// The symbols of one prepared matrix back out of the stream: out[row, column]
// = 1 or 2 at every entry that stands on an activation; out is zero before.
__global__ __launch_bounds__(256) void decode_entries_kernel(
    const uint2 *__restrict__ stream, const uint32_t *__restrict__ slice_base,
    const uint16_t *__restrict__ slice_len, const uint16_t *__restrict__ row_idx,
    uint8_t *__restrict__ out, int64_t first, int slices, int width) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= slices * 64) return;
  const int64_t sl = first + (t >> 6);
  const int ridx = row_idx[sl * 64 + (t & 63)];
  if (ridx == 0xffff) return;
  const uint2 *p = stream + static_cast<int64_t>(slice_base[sl]) * 64 + (t & 63);
  const int len = slice_len[sl];
  const int nch = chunks_of(len);
  int j = 0;
  for (int c = 0; c < nch; c++) {
    const uint2 cw = p[c * 64];
    const unsigned long long w = (static_cast<unsigned long long>(cw.y) << 32) | cw.x;
    for (int q = 0; q < kFields && c * kFields + q < len; q++) {
      j += static_cast<int>(w >> (kFieldBits * q)) & kMaxStep;
      const int pc = j >> 1;   // physical column
      const int col = pc - 1 - pc / kZeroPeriod;
      if (pc % kZeroPeriod != 0 && col < width)
        out[static_cast<int64_t>(ridx) * width + col] = static_cast<uint8_t>((j & 1) + 1);
    }
  }
}

__global__ void fill_bytes_kernel(uint8_t *p, int64_t n, uint8_t v) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void zero_words_kernel(int32_t *p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ------------------------------------------------------------- main kernel --

struct KindArgs {
  const uint32_t *slice_base;
  const uint16_t *slice_len;
  const uint16_t *row_idx;
  const uint32_t *minmax;
  int slices, height, width, parts;
  int split;            // wavefronts that share one slice (1 = a slice per wavefront)
  int groups_max;       // most groups of chunks in a slice of this kind
  int64_t first_slice;  // global index of the kind's first slice (checkpoint addressing)
  int tail_split;       // fused kernel: wavefronts per slice of a short last pass (0: none)
};

struct PreparedArgs {
  const uint2 *stream;        // the interleaved entries
  const uint16_t *ckpt;       // position checkpoints, behind the stream
  KindArgs k[2];
  const int32_t *token_expert;   // NULL: every token uses matrix 0
  const int32_t *order;          // fused kernel, tokens grouped by expert: token ids by expert,
  const int2 *groups;            // and tiles (expert or -1, first index into order * 8 + tokens)
  const uint16_t *x;
  uint16_t *y;
  uint16_t *h;                   // kinds == 2 only
  int32_t *ctrl;                 // NULL: no dependencies between tiles, static tile order
  int64_t ldx, ldy;              // element strides between tokens of x and y
  int kinds;                     // 2: y = wo(relu(wi x));  1: y += W x
  int tokens, experts;
  int xdwords;                   // LDS dwords reserved for the activations
  int hdwords;                   // fused kernel: LDS dwords of h (wo's activations)
  int tail_room;                 // persistent kernel: partial sums (groups x 64 lanes) LDS has room for
  int wi_expect;                 // workgroups of a token's wi a wait expects (k[0].parts outside tests)
  int by_ticket;                 // shared-token kernel: a workgroup's place comes from the ticket
  unsigned long long *tagged;    // shared-token kernel: h is handed over by tag (NULL: by count)
  int lane_parts;                // one-token kernel with wo in workgroups of its own: these share a slice by lanes
  int64_t wait_ticks;            // longest wait between workgroups, ticks of wall_clock64
  int32_t *sticky;               // fault flags in pinned host memory
};

// Activations in LDS: two dwords per physical column, A = (x, 0) and B = (0, x)
// as bf16 pairs, zeros in the zero columns (see "Positions" above).  Rounded up
// to whole 16 bytes (what follows in LDS stays aligned).
__host__ __device__ constexpr int activation_dwords(int width) {
  return (2 * physical_columns(width) + 3) / 4 * 4;
}

// Every load of a thread is in flight before its first LDS store, so a tile
// pays one memory round trip for its activations, not one per pass.  In two
// steps, so that a kernel can ask for the activations long before it needs
// them: stage_request issues a thread's first four loads (all of them up to a
// width of eight times the workgroup), stage_finish stores them and does the
// rest.
struct StagedPairs {
  uint32_t v[4];
};

__device__ __forceinline__ uint32_t load_pair(const uint16_t *x, int m, int width, bool aligned) {
  uint32_t v = 0u;
  if (aligned && 2 * m + 1 < width) {
    v = *reinterpret_cast<const uint32_t *>(x + 2 * m);
  } else {
    if (2 * m < width) v = x[2 * m];
    if (2 * m + 1 < width) v |= static_cast<uint32_t>(x[2 * m + 1]) << 16;
  }
  return v;
}

__device__ __forceinline__ void store_pair(uint32_t *xa, int m, int width, uint32_t v) {
  if (2 * m >= width) return;
  // columns 2m and 2m+1 are neighbours among the physical columns too
  uint32_t *p = xa + 2 * physical_column(2 * m);
  p[0] = v & 0xffffu;
  p[1] = v << 16;
  if (2 * m + 1 < width) {
    p[2] = v >> 16;
    p[3] = v & 0xffff0000u;
  }
}

__device__ __forceinline__ StagedPairs stage_request(const uint16_t *x, int width) {
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 3u) == 0;
  StagedPairs s;
#pragma unroll
  for (int u = 0; u < 4; u++)
    s.v[u] = load_pair(x, threadIdx.x + u * blockDim.x, width, aligned);
  return s;
}

__device__ __forceinline__ void stage_finish(uint32_t *xa, const uint16_t *x, int width,
                                             const StagedPairs &s) {
  const int npairs = (width + 1) / 2;
  const int step = blockDim.x;
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 3u) == 0;
  for (int z = threadIdx.x * kZeroPeriod; z < physical_columns(width); z += step * kZeroPeriod) {
    xa[2 * z] = 0u;
    xa[2 * z + 1] = 0u;
  }
#pragma unroll
  for (int u = 0; u < 4; u++) store_pair(xa, threadIdx.x + u * step, width, s.v[u]);
  for (int m0 = threadIdx.x + 4 * step; m0 < npairs; m0 += 4 * step) {
    uint32_t v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = load_pair(x, m0 + u * step, width, aligned);
#pragma unroll
    for (int u = 0; u < 4; u++) store_pair(xa, m0 + u * step, width, v[u]);
  }
}

__device__ __forceinline__ void stage_activations(uint32_t *xa, const uint16_t *x, int width) {
  const StagedPairs s = stage_request(x, width);
  stage_finish(xa, x, width, s);
}

typedef __attribute__((address_space(3))) const uint32_t lds_word;

// The LDS byte address of a dword of the activation array.
__device__ __forceinline__ uint32_t lds_address(const uint32_t *xa) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_word *)xa));
}

// The nine entries of a chunk: each moves the row's LDS address `at` (bytes)
// and adds the bf16 pair found there, times the row's (min, max), onto acc.
// v_bfe_u32 and v_lshl_add_u32 are written out because the compiler expands the
// same arithmetic into three instructions per entry instead of two.
__device__ __forceinline__ void add_chunk(uint2 cw, uint32_t &at, float &acc, bf16x2 minmax) {
  const uint32_t mid = __builtin_amdgcn_alignbit(cw.y, cw.x, 28);   // bits 28..59: entries 4..7
  uint32_t f[kFields];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[q]) : "v"(cw.x), "n"(kFieldBits * q));
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[4 + q]) : "v"(mid), "n"(kFieldBits * q));
  }
  asm("v_bfe_u32 %0, %1, 24, 7" : "=v"(f[8]) : "v"(cw.y));           // bits 56..62
#pragma unroll
  for (int q = 0; q < kFields; q++) {
    asm("v_lshl_add_u32 %0, %1, 2, %0" : "+v"(at) : "v"(f[q]));
    const bf16x2 v = __builtin_bit_cast(bf16x2, *(lds_word *)static_cast<uintptr_t>(at));
    acc = __builtin_amdgcn_fdot2_f32_bf16(v, minmax, acc, false);
  }
}

// The same sums in the same order with all nine LDS reads of the chunk asked
// for before the first is used: where a compute unit has few wavefronts at work
// (a handful of tokens), a walk is a chain of LDS round trips, and this makes it
// one per chunk instead of one per entry.  (With sixteen wavefronts at it the
// LDS is busy either way, and the registers are better spent elsewhere.)
__device__ __forceinline__ void add_chunk_ahead(uint2 cw, uint32_t &at, float &acc,
                                                bf16x2 minmax) {
  const uint32_t mid = __builtin_amdgcn_alignbit(cw.y, cw.x, 28);
  uint32_t f[kFields], where[kFields];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[q]) : "v"(cw.x), "n"(kFieldBits * q));
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[4 + q]) : "v"(mid), "n"(kFieldBits * q));
  }
  asm("v_bfe_u32 %0, %1, 24, 7" : "=v"(f[8]) : "v"(cw.y));
#pragma unroll
  for (int q = 0; q < kFields; q++) {
    asm("v_lshl_add_u32 %0, %1, 2, %2" : "=v"(where[q]) : "v"(f[q]), "v"(q ? where[q - 1] : at));
  }
  at = where[kFields - 1];
  bf16x2 v[kFields];
#pragma unroll
  for (int q = 0; q < kFields; q++)
    v[q] = __builtin_bit_cast(bf16x2, *(lds_word *)static_cast<uintptr_t>(where[q]));
#pragma unroll
  for (int q = 0; q < kFields; q++) acc = __builtin_amdgcn_fdot2_f32_bf16(v[q], minmax, acc, false);
}

// A chunk of the stream.  kOnce: the launch reads more of the stream than the
// caches hold and every chunk exactly once, and the load says so (a
// non-temporal load; measured 2% faster on the Switch-c-2048 sweep, 2% slower
// where the same few matrices are read over and over from the caches).
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <bool kOnce>
__device__ __forceinline__ uint2 load_chunk(const uint2 *p) {
  if (kOnce) {
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
    return make_uint2(v.x, v.y);
  }
  return *p;
}

// The first n entries of a chunk, n the same in every lane: the last chunk of a
// slice, which is walked only as far as the slice's longest row goes.
__device__ __forceinline__ void add_entries(uint2 cw, int n, uint32_t &at, float &acc,
                                            bf16x2 minmax) {
  if (n == kFields) {
    add_chunk(cw, at, acc, minmax);
    return;
  }
  unsigned long long w = (static_cast<unsigned long long>(cw.y) << 32) | cw.x;
  for (int q = 0; q < n; q++) {
    at += (static_cast<uint32_t>(w) & static_cast<uint32_t>(kMaxStep)) << 2;
    w >>= kFieldBits;
    const bf16x2 v = __builtin_bit_cast(bf16x2, *(lds_word *)static_cast<uintptr_t>(at));
    acc = __builtin_amdgcn_fdot2_f32_bf16(v, minmax, acc, false);
  }
}

// The same with the reads asked for together (see add_chunk_ahead).
__device__ __forceinline__ void add_entries_ahead(uint2 cw, int n, uint32_t &at, float &acc,
                                                  bf16x2 minmax) {
  if (n == kFields) {
    add_chunk_ahead(cw, at, acc, minmax);
    return;
  }
  unsigned long long w = (static_cast<unsigned long long>(cw.y) << 32) | cw.x;
  uint32_t where[kFields - 1];
  bf16x2 v[kFields - 1];
#pragma unroll
  for (int q = 0; q < kFields - 1; q++) {
    where[q] = (q ? where[q - 1] : at) + ((static_cast<uint32_t>(w) & static_cast<uint32_t>(kMaxStep)) << 2);
    w >>= kFieldBits;
  }
#pragma unroll
  for (int q = 0; q < kFields - 1; q++)
    if (q < n) v[q] = __builtin_bit_cast(bf16x2, *(lds_word *)static_cast<uintptr_t>(where[q]));
#pragma unroll
  for (int q = 0; q < kFields - 1; q++)
    if (q < n) acc = __builtin_amdgcn_fdot2_f32_bf16(v[q], minmax, acc, false);
  if (n > 0) {
    uint32_t last = where[0];
#pragma unroll
    for (int q = 1; q < kFields - 1; q++)
      if (q < n) last = where[q];
    at = last;
  }
}

// This lane's chunk 0 of the slice that starts at chunk `base` of the stream.
__device__ __forceinline__ const uint2 *chunk_pointer(const uint2 *stream, uint32_t base) {
  return stream + static_cast<int64_t>(base) * 64 + (threadIdx.x & 63);
}

// What a lane needs to walk its row of one slice; load_slice issues the loads
// of the first chunks, so calling it for the NEXT slice before walking the
// current one hides their latency.
template <int R, bool kOnce = false>
struct Walk {
  uint32_t base;     // the slice's first chunk, in chunks; the same in every lane,
  int nch;           // like the chunk count (where this wavefront stops),
  int last;          // the entries of chunk nch - 1 that are walked (9 unless it ends the slice)
  int c0;            // and the chunk this wavefront starts at (0 unless it shares the slice)
  int j0;            // this lane's position at chunk c0
  int ridx;
  uint32_t minmax;
  uint2 ring[R];
};
typedef Walk<kRing> SliceWalk;

// g_lo, g_hi: the run of chunk groups to walk, for a wavefront that shares the
// slice with others (it then starts from the position checkpoint of group g_lo).
// (len, base: the slice's description, where the caller has read it already.)
template <int R = kRing, bool kOnce = false>
__device__ __forceinline__ Walk<R, kOnce> load_slice_described(const PreparedArgs &a,
                                                               const KindArgs &k, int64_t sl,
                                                               int len, uint32_t base, int g_lo,
                                                               int g_hi) {
  const int lane = threadIdx.x & 63;
  Walk<R, kOnce> w;
  const int nch_all = chunks_of(len);
  w.nch = min(g_hi * kGroupChunks, nch_all);
  w.last = w.nch == nch_all ? last_entries_of(len) : kFields;
  w.c0 = g_lo * kGroupChunks;
  w.ridx = k.row_idx[sl * 64 + lane];
  w.minmax = k.minmax[sl * 64 + lane];
  w.base = base;
  w.j0 = 0;
  if (g_lo)
    w.j0 = a.ckpt[(checkpoint_entry(w.base, k.first_slice + sl) + g_lo) * 64 + lane];
  const uint2 *p = chunk_pointer(a.stream, w.base);
#pragma unroll
  for (int i = 0; i < R; i++) w.ring[i] = load_chunk<kOnce>(p + min(w.c0 + i, w.nch - 1) * 64);
  return w;
}

template <int R = kRing, bool kOnce = false>
__device__ __forceinline__ Walk<R, kOnce> load_slice(const PreparedArgs &a, const KindArgs &k,
                                                     int64_t sl, int g_lo = 0,
                                                     int g_hi = 1 << 20) {
  const int len_word = k.slice_len[sl];
  const uint32_t base_word = k.slice_base[sl];
  return load_slice_described<R, kOnce>(a, k, sl, __builtin_amdgcn_readfirstlane(len_word),
                                        __builtin_amdgcn_readfirstlane(base_word), g_lo, g_hi);
}

// R chunks (the depth of the walk's ring) starting at chunk c added onto the
// partial sum; all of them whole (c + R <= nch - 1), each replaced in the ring
// by the chunk R further on.
// kChecked: the walk's last chunks, fewer than R whole ones and then chunk
// nch - 1 with its `last` entries; nothing is requested any more.
template <bool kChecked, int R, bool kOnce>
__device__ __forceinline__ void run_chunks(Walk<R, kOnce> &w, const uint2 *p, int c, uint32_t &at,
                                           float &part, bf16x2 minmax) {
  const int nch = w.nch;
  // the deep ring is the one of the walks built for latency
  constexpr bool kAhead = R == kSplitRing;
#pragma unroll
  for (int i = 0; i < R; i++) {
    if (!kChecked) {
      const uint2 cw = w.ring[i];
      // unconditional, clamped to the last chunk: the load can target the ring
      // register itself and the loop needs no wait for it
      w.ring[i] = load_chunk<kOnce>(p + min(c + i + R, nch - 1) * 64);
      if (kAhead) add_chunk_ahead(cw, at, part, minmax);
      else add_chunk(cw, at, part, minmax);
    } else if (c + i < nch - 1) {
      if (kAhead) add_chunk_ahead(w.ring[i], at, part, minmax);
      else add_chunk(w.ring[i], at, part, minmax);
    } else if (c + i == nch - 1) {
      if (kAhead) add_entries_ahead(w.ring[i], w.last, at, part, minmax);
      else add_entries(w.ring[i], w.last, at, part, minmax);
    }
  }
}

// The hardware serves the oldest wavefront of a SIMD first; left alone, the
// wavefronts of a workgroup drift apart and the last ones finish a phase on an
// idle compute unit.  A wavefront therefore lowers its priority as it gets
// through its share of the phase, in steps that get finer towards the end
// (`done` of `total`: below 5/8 priority 3, below 13/16 2, below 15/16 1, then
// 0), so that the laggards catch up and all finish together.
__device__ __forceinline__ void progress_priority(int done, int total) {
  const int p = done * 16 / total;
  if (p < 10) {
    __builtin_amdgcn_s_setprio(3);
  } else if (p < 13) {
    __builtin_amdgcn_s_setprio(2);
  } else if (p < 15) {
    __builtin_amdgcn_s_setprio(1);
  } else {
    __builtin_amdgcn_s_setprio(0);
  }
}

// The sum of this lane's row, in the library's canonical order: groups of 72
// entries (kGroupChunks chunks), a partial sum per group from zero, the partial
// sums added first group first.
// With `part` the wavefront shares its slice: it leaves each group's partial
// sum at part[group * 64 + lane] for the wavefront that adds them up.
// pass / passes (passes != 0): this slice is the wavefront's pass-th of `passes`
// about equal ones in the current phase; sets the priority by progress.
template <int R, bool kOnce>
__device__ __forceinline__ float run_slice(Walk<R, kOnce> &w, const uint2 *stream,
                                           const uint32_t *xa, float *part = nullptr,
                                           int pass = 0, int passes = 0) {
  static_assert(kGroupChunks % R == 0, "a group of chunks is a whole number of ring turns");
  // a walk that went through `cur = nxt` may sit in vector registers: put what
  // is the same in all lanes back into scalar ones, for scalar loop control
  // and scalar address arithmetic
  w.nch = __builtin_amdgcn_readfirstlane(w.nch);
  w.last = __builtin_amdgcn_readfirstlane(w.last);
  const uint2 *p = chunk_pointer(stream, __builtin_amdgcn_readfirstlane(w.base));
  const int lane = threadIdx.x & 63;
  const bf16x2 minmax = __builtin_bit_cast(bf16x2, w.minmax);
  float sum = 0.f, partial = 0.f;
  uint32_t at = lds_address(xa) + 4u * static_cast<uint32_t>(w.j0);
  int c = __builtin_amdgcn_readfirstlane(w.c0);
  if (passes) progress_priority(pass, passes);
  auto group_done = [&]() {
    if (passes) progress_priority(pass * w.nch + c + R, passes * w.nch);
    if (part) {
      part[((c + R) / kGroupChunks - 1) * 64 + lane] = partial;
    } else {
      sum += partial;
    }
    partial = 0.f;
  };
  for (; c + R <= w.nch - 1; c += R) {
    run_chunks<false>(w, p, c, at, partial, minmax);
    if ((c + R) % kGroupChunks == 0) group_done();
  }
  // fewer than R whole chunks are left, and the last chunk
  run_chunks<true>(w, p, c, at, partial, minmax);
  if ((c + R) % kGroupChunks == 0) group_done();
  c += R;
  if (part) {
    // the slice's last group, unless the loop has just closed it
    if (c % kGroupChunks) part[(c / kGroupChunks) * 64 + lane] = partial;
  } else {
    sum += partial;   // the last, partial group (+0 if it was just folded)
  }
  return sum;
}

// The slice a wavefront takes in its pass-th turn through `count` slices that
// are ordered longest first: back and forth, so that every wavefront gets
// about the same number of chunks.  >= count: no slice left in this pass.
__device__ __forceinline__ int slice_of_pass(int pass, int wave, int waves, int count) {
  const int s = pass * waves + ((pass & 1) ? waves - 1 - wave : wave);
  return s < count ? s : count;
}

// How a row's result leaves the kernel.
enum OutMode { kStoreRelu = 0, kStore = 1, kAccumulate = 2 };

__device__ __forceinline__ void write_row(uint16_t *dst, int ridx, float res, int mode) {
  if (ridx == 0xffff) return;   // padding lane
  uint16_t out = f32_to_bf16(res);
  if (mode == kStoreRelu) {
    if (out & 0x8000u) out = 0;   // relu between the projections, on the bf16 value
    // h in the workspace, read by other workgroups: written through to where
    // every compute unit sees it (see publish_h)
    __hip_atomic_store(&dst[ridx], out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  } else if (mode == kAccumulate) {
    // reference sub1_cuda_kernel.cu:200: y[row] += bf16(res), the sum in bf16
    out = f32_to_bf16(bf16_to_f32(dst[ridx]) + bf16_to_f32(out));
  }
  dst[ridx] = out;
}

// ----------------------------------------------------- four tokens per walk --
//
// Where several tokens go through the same matrix, the stream is walked once
// for four of them.  The activation array then holds, per physical column, the
// two dwords (x0, x1) and (x2, x3) of tokens 0..3 as bf16 pairs (zeros in the
// zero columns), and an entry costs one address, one 8-byte LDS read and four
// v_dot2c_f32_bf16: the weight, picked by the position's low bit, sits in one
// half of the second operand so that each instruction adds one token's term.
// (Two 4-byte reads from separate arrays measured 10% slower in this kernel.)
// Every token's sum is taken in the same order as when it is walked alone, so
// the results are the same to the bit (for finite activations: a token's
// infinity or NaN also spoils the sum of the token it shares a dword with).
constexpr int kGroupTokens = 4;

struct GroupSums {
  float v[kGroupTokens];
};

struct GroupRows {
  const uint16_t *row[kGroupTokens];   // NULL: no token in this place
};

__device__ __forceinline__ void stage_group(uint32_t *xa, const GroupRows &rows, int width) {
  const int npairs = (width + 1) / 2;
  const int step = blockDim.x;
  for (int z = threadIdx.x * kZeroPeriod; z < physical_columns(width); z += step * kZeroPeriod) {
    xa[2 * z] = 0u;
    xa[2 * z + 1] = 0u;
  }
  for (int m = threadIdx.x; m < npairs; m += step) {
    uint32_t v[kGroupTokens];
#pragma unroll
    for (int t = 0; t < kGroupTokens; t++) {
      v[t] = 0u;
      const uint16_t *row = rows.row[t];
      if (row) {
        if ((reinterpret_cast<uintptr_t>(row) & 3u) == 0 && 2 * m + 1 < width) {
          v[t] = *reinterpret_cast<const uint32_t *>(row + 2 * m);
        } else {
          v[t] = row[2 * m];
          if (2 * m + 1 < width) v[t] |= static_cast<uint32_t>(row[2 * m + 1]) << 16;
        }
      }
    }
    uint32_t *p = xa + 2 * physical_column(2 * m);
    p[0] = (v[0] & 0xffffu) | (v[1] << 16);
    p[1] = (v[2] & 0xffffu) | (v[3] << 16);
    if (2 * m + 1 < width) {
      p[2] = (v[0] >> 16) | (v[1] & 0xffff0000u);
      p[3] = (v[2] >> 16) | (v[3] & 0xffff0000u);
    }
  }
}

// The nine entries of a chunk for four tokens.  `at` is the position's LDS byte
// address as in add_chunk (the array starts on an 8-byte boundary): bit 2 is
// the symbol, the rest the physical column's two dwords.
__device__ __forceinline__ void add_chunk_group(uint2 cw, uint32_t &at, GroupSums &acc,
                                                uint32_t w_min, uint32_t w_max) {
  const uint32_t mid = __builtin_amdgcn_alignbit(cw.y, cw.x, 28);
  uint32_t f[kFields];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[q]) : "v"(cw.x), "n"(kFieldBits * q));
    asm("v_bfe_u32 %0, %1, %2, 7" : "=v"(f[4 + q]) : "v"(mid), "n"(kFieldBits * q));
  }
  asm("v_bfe_u32 %0, %1, 24, 7" : "=v"(f[8]) : "v"(cw.y));
#pragma unroll
  for (int q = 0; q < kFields; q++) {
    asm("v_lshl_add_u32 %0, %1, 2, %0" : "+v"(at) : "v"(f[q]));
    const uint32_t is_max = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(at), 2, 1));
    const uint32_t k_lo = (w_max & is_max) | (w_min & ~is_max);   // (w, 0): one v_bfi_b32
    const uint32_t k_hi = k_lo << 16;                             // (0, w)
    lds_word *col = (lds_word *)static_cast<uintptr_t>(at & ~7u);
    const bf16x2 v01 = __builtin_bit_cast(bf16x2, col[0]);
    const bf16x2 v23 = __builtin_bit_cast(bf16x2, col[1]);
    acc.v[0] = __builtin_amdgcn_fdot2_f32_bf16(v01, __builtin_bit_cast(bf16x2, k_lo), acc.v[0], false);
    acc.v[1] = __builtin_amdgcn_fdot2_f32_bf16(v01, __builtin_bit_cast(bf16x2, k_hi), acc.v[1], false);
    acc.v[2] = __builtin_amdgcn_fdot2_f32_bf16(v23, __builtin_bit_cast(bf16x2, k_lo), acc.v[2], false);
    acc.v[3] = __builtin_amdgcn_fdot2_f32_bf16(v23, __builtin_bit_cast(bf16x2, k_hi), acc.v[3], false);
  }
}

// The first n entries of a chunk for four tokens (see add_entries).
__device__ __forceinline__ void add_entries_group(uint2 cw, int n, uint32_t &at, GroupSums &acc,
                                                  uint32_t w_min, uint32_t w_max) {
  if (n == kFields) {
    add_chunk_group(cw, at, acc, w_min, w_max);
    return;
  }
  unsigned long long w = (static_cast<unsigned long long>(cw.y) << 32) | cw.x;
  for (int q = 0; q < n; q++) {
    at += (static_cast<uint32_t>(w) & static_cast<uint32_t>(kMaxStep)) << 2;
    w >>= kFieldBits;
    const uint32_t is_max = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(at), 2, 1));
    const uint32_t k_lo = (w_max & is_max) | (w_min & ~is_max);
    const uint32_t k_hi = k_lo << 16;
    lds_word *col = (lds_word *)static_cast<uintptr_t>(at & ~7u);
    const bf16x2 v01 = __builtin_bit_cast(bf16x2, col[0]);
    const bf16x2 v23 = __builtin_bit_cast(bf16x2, col[1]);
    acc.v[0] = __builtin_amdgcn_fdot2_f32_bf16(v01, __builtin_bit_cast(bf16x2, k_lo), acc.v[0], false);
    acc.v[1] = __builtin_amdgcn_fdot2_f32_bf16(v01, __builtin_bit_cast(bf16x2, k_hi), acc.v[1], false);
    acc.v[2] = __builtin_amdgcn_fdot2_f32_bf16(v23, __builtin_bit_cast(bf16x2, k_lo), acc.v[2], false);
    acc.v[3] = __builtin_amdgcn_fdot2_f32_bf16(v23, __builtin_bit_cast(bf16x2, k_hi), acc.v[3], false);
  }
}

// run_slice for four tokens: the same groups of 72 entries per token.  With
// `part` the wavefront shares its slice and leaves each group's four partial
// sums at part[group * 64 + lane].
__device__ __forceinline__ GroupSums run_slice_group(SliceWalk &w, const uint2 *stream,
                                                     const uint32_t *xa, GroupSums *part,
                                                     int pass, int passes) {
  w.nch = __builtin_amdgcn_readfirstlane(w.nch);
  w.last = __builtin_amdgcn_readfirstlane(w.last);
  const uint2 *p = chunk_pointer(stream, __builtin_amdgcn_readfirstlane(w.base));
  const int lane = threadIdx.x & 63;
  const uint32_t w_min = w.minmax & 0xffffu, w_max = w.minmax >> 16;
  GroupSums sum = {{0.f, 0.f, 0.f, 0.f}}, partial = {{0.f, 0.f, 0.f, 0.f}};
  uint32_t at = lds_address(xa) + 4u * static_cast<uint32_t>(w.j0);
  int c = __builtin_amdgcn_readfirstlane(w.c0);
  if (passes) progress_priority(pass, passes);
  auto group_done = [&](int g) {
    if (part) {
      part[g * 64 + lane] = partial;
    } else {
#pragma unroll
      for (int t = 0; t < kGroupTokens; t++) sum.v[t] += partial.v[t];
    }
#pragma unroll
    for (int t = 0; t < kGroupTokens; t++) partial.v[t] = 0.f;
  };
  for (; c < w.nch; c += kRing) {
#pragma unroll
    for (int i = 0; i < kRing; i++) {
      if (c + i < w.nch - 1) {
        const uint2 cw = w.ring[i];
        w.ring[i] = p[min(c + i + kRing, w.nch - 1) * 64];
        add_chunk_group(cw, at, partial, w_min, w_max);
      } else if (c + i == w.nch - 1) {
        add_entries_group(w.ring[i], w.last, at, partial, w_min, w_max);   // the walk's last chunk
      }
    }
    if ((c + kRing) % kGroupChunks == 0) {
      if (passes) progress_priority(pass * w.nch + c + kRing, passes * w.nch);
      group_done((c + kRing) / kGroupChunks - 1);
    }
  }
  // the last, partial group, unless the loop has just closed it
  if (c % kGroupChunks) group_done(c / kGroupChunks);
  return sum;
}

// Small-batch form of a tile: `split` wavefronts share each slice, every one
// taking a run of the slice's chunk groups (it starts from the position
// checkpoint of its first group) and leaving one partial sum per group in LDS;
// after a barrier the slice's first wavefront adds the groups in order, which
// is the canonical order, so the result is the same to the bit as with a
// wavefront per slice.  Built for latency: split_begin puts the loads of a
// whole group in flight, and the kernel calls it before it waits for and
// stages the activations.
struct SplitWalk {
  Walk<kSplitRing> w;   // w.nch: this wavefront's last chunk + 1
  int g_lo, g_hi, ngroups;
  int64_t sl;
  bool mine;
};

// Everything but the position and the ring is the same in all lanes and is kept
// in scalar registers (the wavefront index goes through readfirstlane).  The
// ring loads are unconditional, with the chunk index clamped to the wavefront's
// last chunk, so that they all leave at once.
__device__ __forceinline__ SplitWalk split_begin(const PreparedArgs &a, const KindArgs &k, int e,
                                                 int s0, int s_hi) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int sub = wave % k.split;
  const int s = s0 + wave / k.split;
  SplitWalk r;
  r.mine = s < s_hi;
  r.ngroups = 0;
  r.g_lo = 0;
  r.g_hi = 0;
  r.sl = static_cast<int64_t>(e) * k.slices + s;
  r.w.base = 0;
  r.w.j0 = 0;
  r.w.nch = 0;
  r.w.last = kFields;
  r.w.minmax = 0u;
  r.w.ridx = 0xffff;
  // both words of the slice's description in one round trip (a slice that
  // exists is read also where this wavefront has none)
  const int64_t described = r.mine ? r.sl : static_cast<int64_t>(e) * k.slices + s0;
  const int len_word = k.slice_len[described];
  const uint32_t base_word = k.slice_base[described];
  if (r.mine) {
    const int len = __builtin_amdgcn_readfirstlane(len_word);
    const int nch_all = chunks_of(len);
    r.ngroups = (nch_all + kGroupChunks - 1) / kGroupChunks;
    r.g_lo = sub * r.ngroups / k.split;
    r.g_hi = (sub + 1) * r.ngroups / k.split;
    r.w.minmax = k.minmax[r.sl * 64 + lane];
    if (sub == 0) r.w.ridx = k.row_idx[r.sl * 64 + lane];   // it will write the slice's rows
    if (r.g_lo < r.g_hi) {
      const uint32_t base = __builtin_amdgcn_readfirstlane(base_word);
      r.w.base = base;
      const uint2 *p = chunk_pointer(a.stream, base);
      const int c_lo = r.g_lo * kGroupChunks;
      r.w.nch = min(r.g_hi * kGroupChunks, nch_all);
      r.w.last = r.w.nch == nch_all ? last_entries_of(len) : kFields;
      if (r.g_lo)
        r.w.j0 = a.ckpt[(checkpoint_entry(base, k.first_slice + r.sl) + r.g_lo) * 64 + lane];
#pragma unroll
      for (int i = 0; i < kSplitRing; i++)
        r.w.ring[i] = p[min(c_lo + i, r.w.nch - 1) * 64];
    }
  }
  return r;
}

// The groups of a tile; contains a workgroup barrier.  A wavefront that
// has its slice to itself (split 1) adds the groups in registers, in the same
// order, and leaves the partial-sum area alone.
__device__ __forceinline__ void split_run(const PreparedArgs &a, const KindArgs &k, SplitWalk &r,
                                          const uint32_t *xa, uint16_t *dst, int mode) {
  float *part = reinterpret_cast<float *>(const_cast<uint32_t *>(xa) + a.xdwords);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int local = wave / k.split;
  const bool alone = k.split == 1;
  const bf16x2 minmax = __builtin_bit_cast(bf16x2, r.w.minmax);
  uint32_t at = lds_address(xa) + 4u * static_cast<uint32_t>(r.w.j0);
  float sum = 0.f;
  const uint2 *p = chunk_pointer(a.stream, r.w.base);
  for (int g = r.g_lo; g < r.g_hi; g++) {
    float partial = 0.f;
    const int c_end = min((g + 1) * kGroupChunks, r.w.nch);
    for (int c = g * kGroupChunks; c < c_end; c += kSplitRing) {
      if (c + kSplitRing <= r.w.nch - 1)      // whole chunks only, and more to come
        run_chunks<false>(r.w, p, c, at, partial, minmax);
      else                                    // the run that ends with this wavefront's last chunk
        run_chunks<true>(r.w, p, c, at, partial, minmax);
    }
    if (alone) {
      sum += partial;
    } else {
      part[(local * k.groups_max + g) * 64 + lane] = partial;
    }
  }
  __syncthreads();
  if (r.mine && wave % k.split == 0) {
    if (!alone)
      for (int g = 0; g < r.ngroups; g++) sum += part[(local * k.groups_max + g) * 64 + lane];
    write_row(dst, r.w.ridx, sum, mode);
  }
}

// A wo tile waits until its token's wi tiles have published h (bounded spin of
// one lane, then a barrier that extends its acquire to the workgroup); then the
// tile's activations go into LDS.  Ends with a barrier.  The tile says that it
// has waited (done_waiting) once its work is done: that takes a round trip to
// memory, which does not belong between the wait and the walk.
__device__ __forceinline__ void await_activations(const PreparedArgs &a, const KindArgs &k,
                                                  int kind, int t, uint32_t *xa) {
  if (kind == 1) {
    if (threadIdx.x == 0)
      sub1::bounded_wait(&a.ctrl[sub1::token_word(t)], a.wi_expect, a.wait_ticks, a.sticky,
                         &a.ctrl[kCtrlGaveUp]);
    __syncthreads();
  }
  const uint16_t *src = kind ? a.h + static_cast<int64_t>(t) * k.width
                             : a.x + static_cast<int64_t>(t) * a.ldx;
  stage_activations(xa, src, k.width);
  __syncthreads();
}

__device__ __forceinline__ void done_waiting(const PreparedArgs &a, int t) {
  if (threadIdx.x == 0) sub1::waited_on(&a.ctrl[sub1::token_word(t)], a.k[1].parts);
}

// What a ticket stands for.  Every field is the same in all lanes.
struct Tile {
  int kind, t, s_lo, s_hi, e;   // e < 0: no matrix (token dropped or index out of range)
};

__device__ __forceinline__ Tile decode_tile(const PreparedArgs &a, int ticket, bool count_faults) {
  const int n_wi = a.tokens * a.k[0].parts;
  Tile tile;
  tile.kind = ticket < n_wi ? 0 : 1;
  const KindArgs &k = a.k[tile.kind];
  const int rel = tile.kind ? ticket - n_wi : ticket;
  tile.t = rel / k.parts;
  const int part = rel - tile.t * k.parts;
  // slices [s_lo, s_hi) of the matrix
  tile.s_lo = static_cast<int>(static_cast<int64_t>(k.slices) * part / k.parts);
  tile.s_hi = static_cast<int>(static_cast<int64_t>(k.slices) * (part + 1) / k.parts);
  tile.e = a.token_expert ? __builtin_amdgcn_readfirstlane(a.token_expert[tile.t]) : 0;
  if (tile.e >= a.experts) {
    if (count_faults && tile.kind == a.kinds - 1 && part == 0 && threadIdx.x == 0)
      __hip_atomic_fetch_add(&a.ctrl[kCtrlBadIds], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    tile.e = -1;
  }
  return tile;
}

// A dropped token keeps its input (reference sub1.py:312).
__device__ __forceinline__ void pass_through(const PreparedArgs &a, const KindArgs &k, int t,
                                             int s_lo, int s_hi) {
  const int r_lo = min(64 * s_lo, k.height), r_hi = min(64 * s_hi, k.height);
  for (int i = r_lo + threadIdx.x; i < r_hi; i += blockDim.x)
    a.y[static_cast<int64_t>(t) * a.ldy + i] = a.x[static_cast<int64_t>(t) * a.ldx + i];
}

__device__ __forceinline__ uint16_t *tile_output(const PreparedArgs &a, const KindArgs &k,
                                                 int kind, int t, int &mode) {
  if (a.kinds == 2 && kind == 0) {
    mode = kStoreRelu;
    return a.h + static_cast<int64_t>(t) * k.height;
  }
  mode = a.kinds == 2 ? kStore : kAccumulate;
  return a.y + static_cast<int64_t>(t) * a.ldy;
}

// h of a token's wi tile becomes visible to the wo tiles.  The rows of h are
// stored at agent scope (write_row), i.e. written through the L2 of this
// wavefront's die; every wavefront waits until its own stores are acknowledged,
// the barrier collects the wavefronts, and one lane counts the tile as done.
// A release fence instead of the write-through stores would write back the
// whole L2 (measured 8 us per tile with all compute units at it).
__device__ __forceinline__ void publish_h(const PreparedArgs &a, int t) {
  sub1::drain_stores();
  __syncthreads();
  if (threadIdx.x == 0)
    __hip_atomic_fetch_add(&a.ctrl[sub1::token_word(t)], 1, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}

// The wavefronts of a workgroup walk `all` slices of one matrix: slice `first`
// of the stream's slices and every `stride`-th after it.  `before()` runs once
// the first loads of the stream are out (it stages the activations `act` and
// ends with a barrier); `out(row, sum, slice)` takes every row's result.  A short last
// pass (at most half the wavefronts busy) is shared out: `split` wavefronts per
// slice, each a run of its chunk groups, partial sums in `partials`
// (a.tail_room groups of 64 lanes).
template <class Before, class Out>
__device__ __forceinline__ void walk_tile(const PreparedArgs &a, const KindArgs &k, int64_t first,
                                          int stride, int all, const uint32_t *act,
                                          float *partials, Before &&before, Out &&out,
                                          bool active = true) {
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int split = 1;
  const int rest = all % waves;
  if (rest > 0 && rest * 2 <= waves && rest * k.groups_max <= a.tail_room)
    split = min(waves / rest, k.groups_max);
  const int count = split > 1 ? all - rest : all;
  const int passes = (count + waves - 1) / waves + (split > 1);
  // the shared last pass: slice `tail_sl` of the tile, this wavefront its
  // groups g_lo .. g_hi - 1 of `groups`
  const int tail_sl = count + wave / split;
  const int sub = wave % split;
  const int64_t tail_slice = first + static_cast<int64_t>(tail_sl) * stride;
  // With a few tokens that pass is the whole walk, and the walk a chain of
  // memory round trips: its loads (the slice's description, then a whole group
  // of chunks) go out before the wait and the staging like the first loads of
  // any other walk.
  const bool tail_only = split > 1 && count == 0;
  int groups = 0, g_lo = 0, g_hi = 0, tail_len = 0;
  uint32_t tail_base = 0;
  auto tail_groups = [&]() {
    if (tail_sl < all) {
      // both words of the slice's description in one round trip
      const int len_word = k.slice_len[tail_slice];
      const uint32_t base_word = k.slice_base[tail_slice];
      tail_len = __builtin_amdgcn_readfirstlane(len_word);
      tail_base = __builtin_amdgcn_readfirstlane(base_word);
      groups = (chunks_of(tail_len) + kGroupChunks - 1) / kGroupChunks;
      g_lo = sub * groups / split;
      g_hi = (sub + 1) * groups / split;
    }
  };
  Walk<kSplitRing> tail_ahead;
  int tail_ridx = 0xffff;   // the rows of the shared slice, in the wavefront that adds them up
  if (tail_only) {
    if (sub == 0 && tail_sl < all && active) tail_ridx = k.row_idx[tail_slice * 64 + (threadIdx.x & 63)];
    tail_groups();
    if (g_lo < g_hi && active)
      tail_ahead = load_slice_described<kSplitRing>(a, k, tail_slice, tail_len, tail_base, g_lo, g_hi);
  }
  int s = slice_of_pass(0, wave, waves, count);
  SliceWalk cur;
  // the first loads of the stream go out before the wait and the staging
  if (s < count && active) cur = load_slice(a, k, first + static_cast<int64_t>(s) * stride);
  before();
  for (int pass = 0; s < count; pass++) {
    const int s_next = slice_of_pass(pass + 1, wave, waves, count);
    SliceWalk nxt;
    if (active) {
      if (s_next < count) nxt = load_slice(a, k, first + static_cast<int64_t>(s_next) * stride);
      const float res = run_slice(cur, a.stream, act, nullptr, pass, passes);
      out(cur.ridx, res, first + static_cast<int64_t>(s) * stride);
      if (s_next < count) cur = nxt;
    }
    s = s_next;
  }
  if (split > 1) {
    __builtin_amdgcn_s_setprio(0);
    const int lane = threadIdx.x & 63;
    float *mine = partials + (wave / split) * k.groups_max * 64;
    if (tail_only) {
      if (g_lo < g_hi && active) run_slice(tail_ahead, a.stream, act, mine);
    } else {
      if (sub == 0 && tail_sl < all && active) tail_ridx = k.row_idx[tail_slice * 64 + lane];
      tail_groups();
      if (g_lo < g_hi && active) {
        SliceWalk tail = load_slice_described(a, k, tail_slice, tail_len, tail_base, g_lo, g_hi);
        run_slice(tail, a.stream, act, mine);
      }
    }
    __syncthreads();
    if (sub == 0 && tail_sl < all && active) {
      float sum = 0.f;
      for (int g = 0; g < groups; g++) sum += mine[g * 64 + lane];
      out(tail_ridx, sum, tail_slice);
    }
  }
}

// Persistent grid.  A tile is (token, projection, part): the slices of one
// matrix, or of one of `parts` equal ranges of them when there are too few
// tokens to occupy the GPU otherwise; a workgroup stages the token's
// activations once per tile and its wavefronts take the tile's slices in turn.
// All wi tiles are numbered before all wo tiles and handed out by an atomic
// ticket.  A wo tile waits for the wi tiles of its token, which hold smaller
// tickets and so are running or done: the wait always ends.  h is published by
// ONE agent-scope release per tile (thread 0, after every wavefront drained its
// stores and the workgroup barrier) and picked up by one acquire; an agent-scope
// fence costs an L2 write-back on this part, which is why the lanes do not fence
// individually.
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  __shared__ int s_ticket;
  uint32_t *xa = lds;
  const int n_wi = a.tokens * a.k[0].parts;
  const int n_all = n_wi + (a.kinds == 2 ? a.tokens * a.k[1].parts : 0);
  const bool dynamic = a.ctrl != nullptr;
  // dynamic order: thread 0 asks for the next ticket when its own part of the
  // tile is done, so that the atomic's round trip overlaps the tile's tail (any
  // earlier and the workgroups that start first take tiles away from the last
  // ones); static order: tile = workgroup index + k * grid
  int static_ticket = blockIdx.x;   // the same in every lane, unlike thread 0's next_ticket
  int next_ticket = 0;
  auto fetch_next = [&]() {
    if (dynamic && threadIdx.x == 0)
      next_ticket = __hip_atomic_fetch_add(&a.ctrl[0], 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
  };
  fetch_next();
  for (;;) {
    __syncthreads();
    int ticket;
    if (dynamic) {
      if (threadIdx.x == 0) s_ticket = next_ticket;
      __syncthreads();
      ticket = __builtin_amdgcn_readfirstlane(s_ticket);   // the same in every lane: scalar
    } else {
      ticket = static_ticket;
      static_ticket += gridDim.x;
    }
    if (ticket >= n_all) break;
    const Tile tile = decode_tile(a, ticket, dynamic);
    const int kind = tile.kind, t = tile.t, s_lo = tile.s_lo, s_hi = tile.s_hi, e = tile.e;
    const KindArgs &k = a.k[kind];
    if (a.kinds == 2 && kind == 1 && e < 0) {
      pass_through(a, k, t, s_lo, s_hi);
      fetch_next();
      continue;
    }
    if (e >= 0) {
      int mode;
      uint16_t *dst = tile_output(a, k, kind, t, mode);
      walk_tile(a, k, static_cast<int64_t>(e) * k.slices + s_lo, 1, s_hi - s_lo, xa,
                reinterpret_cast<float *>(xa + a.xdwords),
                [&]() { await_activations(a, k, kind, t, xa); },
                [&](int ridx, float res, int64_t) { write_row(dst, ridx, res, mode); });
    }
    fetch_next();
    if (a.kinds == 2 && kind == 0 && e >= 0) publish_h(a, t);   // a dropped token's word stays untouched
    if (a.kinds == 2 && kind == 1 && e >= 0) done_waiting(a, t);
  }
  if (dynamic && threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
}

// Tokens by expert, for the fused kernel when experts receive several tokens
// each.  One workgroup: counts per expert (tokens that name no expert in a
// bucket of their own), prefix sums, then every token takes a place among its
// expert's tokens and, if its place starts one, writes a tile: four tokens of
// an expert walk the stream together, three too; one or two left over go one
// by one (a walk for four costs about as much as 2.3 single ones).
//   tab: int32 [4, experts + 1]: counts, first place, first tile, next place
// ctrl[3] receives the number of tiles, ctrl[2] the tokens whose expert id is
// too large.  Which tokens share a walk depends on the order in which they
// take their places (atomics) and may differ from run to run; each token's
// result does not depend on it.
__device__ __forceinline__ int32_t load_l2(const int32_t *p) {   // past the L1: atomics update L2 only
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__host__ __device__ constexpr int tiles_of(int n) {
  return n / kGroupTokens + (n % kGroupTokens == 3 ? 1 : n % kGroupTokens);
}

__global__ __launch_bounds__(1024) void group_tokens_kernel(
    const int32_t *__restrict__ token_expert, int tokens, int experts, int32_t *__restrict__ tab,
    int32_t *__restrict__ order, int2 *__restrict__ groups, int32_t *__restrict__ ctrl) {
  __shared__ int32_t seg_tokens[1024], seg_tiles[1024];
  const int tid = threadIdx.x;
  const int buckets = experts + 1;
  int32_t *count = tab, *first = tab + buckets, *tile0 = tab + 2 * buckets,
          *next = tab + 3 * buckets;
  for (int b = tid; b < buckets; b += 1024) count[b] = 0;
  __syncthreads();
  int faults = 0;
  for (int t = tid; t < tokens; t += 1024) {
    const int e = token_expert[t];
    if (e >= experts) faults++;
    atomicAdd(&count[e < 0 || e >= experts ? experts : e], 1);
  }
  if (faults) atomicAdd(&ctrl[2], faults);
  __syncthreads();
  // prefix sums over the buckets: a run of buckets per thread, then the runs
  const int seg = (buckets + 1023) / 1024;
  const int lo = min(tid * seg, buckets), hi = min(lo + seg, buckets);
  int32_t n_tok = 0, n_tile = 0;
  for (int b = lo; b < hi; b++) {
    const int n = load_l2(&count[b]);
    n_tok += n;
    n_tile += b == experts ? n : tiles_of(n);
  }
  seg_tokens[tid] = n_tok;
  seg_tiles[tid] = n_tile;
  __syncthreads();
  for (int d = 1; d < 1024; d *= 2) {
    const int32_t a0 = tid >= d ? seg_tokens[tid - d] : 0, a1 = tid >= d ? seg_tiles[tid - d] : 0;
    __syncthreads();
    seg_tokens[tid] += a0;
    seg_tiles[tid] += a1;
    __syncthreads();
  }
  int32_t run_tok = tid ? seg_tokens[tid - 1] : 0, run_tile = tid ? seg_tiles[tid - 1] : 0;
  for (int b = lo; b < hi; b++) {
    const int n = load_l2(&count[b]);
    first[b] = run_tok;
    next[b] = run_tok;
    tile0[b] = run_tile;
    run_tok += n;
    run_tile += b == experts ? n : tiles_of(n);
  }
  if (tid == 1023) ctrl[3] = seg_tiles[1023];
  __syncthreads();
  for (int t = tid; t < tokens; t += 1024) {
    const int e = token_expert[t];
    const int b = e < 0 || e >= experts ? experts : e;
    const int place = atomicAdd(&next[b], 1);
    order[place] = t;
    const int i = place - load_l2(&first[b]), n = load_l2(&count[b]);
    const int t0 = load_l2(&tile0[b]);
    const int whole = b == experts ? 0 : n / kGroupTokens * kGroupTokens;   // tokens in tiles of four
    const int rest = n - whole;
    if (i < whole) {
      if (i % kGroupTokens == 0) groups[t0 + i / kGroupTokens] = make_int2(e, place * 8 + kGroupTokens);
    } else if (b != experts && rest == 3) {
      if (i == whole) groups[t0 + whole / kGroupTokens] = make_int2(e, place * 8 + 3);
    } else {
      groups[t0 + whole / kGroupTokens + (i - whole)] = make_int2(b == experts ? -1 : e, place * 8 + 1);
    }
  }
}

// A tile of the fused kernel with three or four tokens of one expert: the
// same two phases, both walked once for all of them (see "four tokens per
// walk").  order[place ..] are the tokens; h sits in LDS as (h0, h1), (h2, h3)
// per physical column.  Ends before the loop's barrier.
template <class FetchNext>
__device__ __forceinline__ void fused_group_tile(const PreparedArgs &a, uint32_t *xa, uint32_t *ha,
                                                 int e, int place, int n, FetchNext &&fetch_next) {
  const KindArgs &ki = a.k[0];
  const KindArgs &ko = a.k[1];
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  int tok[kGroupTokens];
  GroupRows rows;
#pragma unroll
  for (int k = 0; k < kGroupTokens; k++) {
    tok[k] = k < n ? __builtin_amdgcn_readfirstlane(a.order[place + k]) : -1;
    rows.row[k] = k < n ? a.x + static_cast<int64_t>(tok[k]) * a.ldx : nullptr;
  }
  // wi: x -> relu(h) into LDS
  const int64_t first_i = static_cast<int64_t>(e) * ki.slices;
  int s = slice_of_pass(0, wave, waves, ki.slices);
  SliceWalk cur;
  if (s < ki.slices) cur = load_slice(a, ki, first_i + s);
  stage_group(xa, rows, ki.width);
  __syncthreads();
  for (int pass = 0; s < ki.slices; pass++) {
    const int s_next = slice_of_pass(pass + 1, wave, waves, ki.slices);
    SliceWalk nxt;
    if (s_next < ki.slices) nxt = load_slice(a, ki, first_i + s_next);
    const GroupSums res = run_slice_group(cur, a.stream, xa, nullptr, pass,
                                          (ki.slices + waves - 1) / waves);
    if (cur.ridx != 0xffff) {
      uint32_t out[kGroupTokens];
#pragma unroll
      for (int k = 0; k < kGroupTokens; k++) {
        out[k] = f32_to_bf16(res.v[k]);
        if (out[k] & 0x8000u) out[k] = 0;   // relu between the projections, on the bf16 value
      }
      uint32_t *p = ha + 2 * physical_column(cur.ridx);
      p[0] = out[0] | (out[1] << 16);
      p[1] = out[2] | (out[3] << 16);
    }
    if (s_next < ki.slices) cur = nxt;
    s = s_next;
  }
  fetch_next();
  // wo: h -> y, the short last pass shared out as for a single token
  const int whole = ko.tail_split ? ko.slices - ko.slices % waves : ko.slices;
  const int64_t first = static_cast<int64_t>(e) * ko.slices;
  s = slice_of_pass(0, wave, waves, whole);
  if (s < whole) cur = load_slice(a, ko, first + s);
  __syncthreads();
  auto write_rows = [&](int ridx, const GroupSums &res) {
#pragma unroll
    for (int k = 0; k < kGroupTokens; k++)
      if (k < n) write_row(a.y + static_cast<int64_t>(tok[k]) * a.ldy, ridx, res.v[k], kStore);
  };
  for (int pass = 0; s < whole; pass++) {
    const int s_next = slice_of_pass(pass + 1, wave, waves, whole);
    SliceWalk nxt;
    if (s_next < whole) nxt = load_slice(a, ko, first + s_next);
    const GroupSums res = run_slice_group(cur, a.stream, ha, nullptr, pass, (whole + waves - 1) / waves);
    write_rows(cur.ridx, res);
    if (s_next < whole) cur = nxt;
    s = s_next;
  }
  __builtin_amdgcn_s_setprio(0);
  if (ko.tail_split) {
    const int sl = whole + wave / ko.tail_split;
    const int sub = wave % ko.tail_split;
    GroupSums *mine = reinterpret_cast<GroupSums *>(xa) + (wave / ko.tail_split) * ko.groups_max * 64;
    int groups = 0;
    if (sl < ko.slices) {
      groups = (chunks_of(__builtin_amdgcn_readfirstlane(ko.slice_len[first + sl])) +
                kGroupChunks - 1) / kGroupChunks;
      const int g_lo = sub * groups / ko.tail_split, g_hi = (sub + 1) * groups / ko.tail_split;
      if (g_lo < g_hi) {
        SliceWalk tail = load_slice(a, ko, first + sl, g_lo, g_hi);
        run_slice_group(tail, a.stream, ha, mine, 0, 0);
      }
    }
    __syncthreads();
    if (sub == 0 && sl < ko.slices) {
      GroupSums sum = {{0.f, 0.f, 0.f, 0.f}};
      for (int g = 0; g < groups; g++) {
        const GroupSums v = mine[g * 64 + lane];
#pragma unroll
        for (int k = 0; k < kGroupTokens; k++) sum.v[k] += v.v[k];
      }
      write_rows(ko.row_idx[(first + sl) * 64 + lane], sum);
    }
  }
}

// Streaming form for batches of at least one token per compute unit: a tile is
// a token, and the workgroup runs wi, ReLU and wo back to back with h kept in
// LDS, already in the layout wo reads its activations from.  No workspace
// traffic for h, no waiting between workgroups; tickets only balance the load.
// LDS: x (wi's activations) | h (wo's activations).
// kOnce: see load_chunk.
template <bool kGrouped, bool kOnce>
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_fused_kernel(PreparedArgs a) {
  typedef Walk<kRing, kOnce> TokenWalk;
  extern __shared__ __align__(16) uint32_t lds[];
  __shared__ int s_ticket;
  uint32_t *xa = lds;
  uint32_t *ha = xa + a.xdwords;
  const int threads = blockDim.x;
  const int waves = threads >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const KindArgs &ki = a.k[0];
  const KindArgs &ko = a.k[1];
  // h: the lanes overwrite the two value dwords of their rows; the zeros between
  // them stay for the whole launch
  for (int i = threadIdx.x; i < a.hdwords; i += threads) ha[i] = 0u;
  // tokens grouped by expert: the tiles are in a.groups, ctrl[3] of them
  const int n_tiles = kGrouped ? __builtin_amdgcn_readfirstlane(a.ctrl[3]) : a.tokens;
  int next_ticket = 0;
  auto fetch_next = [&]() {
    if (threadIdx.x == 0)
      next_ticket = __hip_atomic_fetch_add(&a.ctrl[0], 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
  };
  fetch_next();
  for (;;) {
    __syncthreads();   // the previous token's wo has read h; s_ticket is free
    if (threadIdx.x == 0) s_ticket = next_ticket;
    __syncthreads();
    const int tile = __builtin_amdgcn_readfirstlane(s_ticket);
    if (tile >= n_tiles) break;
    int t = tile, e, n = 1, place = 0;
    if (kGrouped) {
      const int2 rec = a.groups[tile];
      e = __builtin_amdgcn_readfirstlane(rec.x);
      place = __builtin_amdgcn_readfirstlane(rec.y >> 3);
      n = __builtin_amdgcn_readfirstlane(rec.y & 7);
      t = __builtin_amdgcn_readfirstlane(a.order[place]);
    } else {
      e = __builtin_amdgcn_readfirstlane(a.token_expert[t]);
      if (e >= a.experts) {
        if (threadIdx.x == 0)
          __hip_atomic_fetch_add(&a.ctrl[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        e = -1;
      }
    }
    if (e < 0) {
      pass_through(a, ko, t, 0, ko.slices);
      fetch_next();
      continue;
    }
    if (kGrouped && n > 2) {
      fused_group_tile(a, xa, ha, e, place, n, fetch_next);
      continue;
    }
    // wi: x -> relu(h) into LDS
    const int64_t first_i = static_cast<int64_t>(e) * ki.slices;
    int s = slice_of_pass(0, wave, waves, ki.slices);
    TokenWalk cur;
    if (s < ki.slices) cur = load_slice<kRing, kOnce>(a, ki, first_i + s);
    stage_activations(xa, a.x + static_cast<int64_t>(t) * a.ldx, ki.width);
    __syncthreads();
    for (int pass = 0; s < ki.slices; pass++) {
      const int s_next = slice_of_pass(pass + 1, wave, waves, ki.slices);
      TokenWalk nxt;
      if (s_next < ki.slices) nxt = load_slice<kRing, kOnce>(a, ki, first_i + s_next);
      const float res = run_slice(cur, a.stream, xa, nullptr, pass,
                                  (ki.slices + waves - 1) / waves);
      if (cur.ridx != 0xffff) {
        uint32_t out = f32_to_bf16(res);
        if (out & 0x8000u) out = 0;   // relu between the projections, on the bf16 value
        uint32_t *p = ha + 2 * physical_column(cur.ridx);
        p[0] = out;
        p[1] = out << 16;
      }
      if (s_next < ki.slices) cur = nxt;
      s = s_next;
    }
    // the next token is asked for halfway through this one: early enough to
    // hide the round trip, late enough that the workgroups that started first
    // do not take the last tokens away from the others
    fetch_next();
    // wo: h -> y; its first loads go out before the barrier.  A short last pass
    // (tail_split != 0) is shared out: tail_split wavefronts per slice, each a
    // run of its chunk groups, partial sums into the LDS that held x.
    const int whole = ko.tail_split ? ko.slices - ko.slices % waves : ko.slices;
    const int64_t first = static_cast<int64_t>(e) * ko.slices;
    s = slice_of_pass(0, wave, waves, whole);
    if (s < whole) cur = load_slice<kRing, kOnce>(a, ko, first + s);
    __syncthreads();
    uint16_t *dst = a.y + static_cast<int64_t>(t) * a.ldy;
    for (int pass = 0; s < whole; pass++) {
      const int s_next = slice_of_pass(pass + 1, wave, waves, whole);
      TokenWalk nxt;
      if (s_next < whole) nxt = load_slice<kRing, kOnce>(a, ko, first + s_next);
      const float res = run_slice(cur, a.stream, ha, nullptr, pass, (whole + waves - 1) / waves);
      write_row(dst, cur.ridx, res, kStore);
      if (s_next < whole) cur = nxt;
      s = s_next;
    }
    __builtin_amdgcn_s_setprio(0);
    if (ko.tail_split) {
      const int lane = threadIdx.x & 63;
      const int sl = whole + wave / ko.tail_split;
      const int sub = wave % ko.tail_split;
      float *mine = reinterpret_cast<float *>(xa) + (wave / ko.tail_split) * ko.groups_max * 64;
      int groups = 0;
      if (sl < ko.slices) {
        groups = (chunks_of(__builtin_amdgcn_readfirstlane(ko.slice_len[first + sl])) +
                  kGroupChunks - 1) / kGroupChunks;
        const int g_lo = sub * groups / ko.tail_split, g_hi = (sub + 1) * groups / ko.tail_split;
        if (g_lo < g_hi) {
          TokenWalk tail = load_slice<kRing, kOnce>(a, ko, first + sl, g_lo, g_hi);
          run_slice(tail, a.stream, ha, mine);
        }
      }
      __syncthreads();
      if (sub == 0 && sl < ko.slices) {
        // the slice's first wavefront adds the groups in order and writes the rows
        float sum = 0.f;
        for (int g = 0; g < groups; g++) sum += mine[g * 64 + lane];
        write_row(dst, ko.row_idx[(first + sl) * 64 + lane], sum, kStore);
      }
    }
  }
  if (threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
}

// ---- h by tag ----------------------------------------------------------------
//
// A row of relu(h) into the tagged copy: value and tag in one 64-bit store,
// written through like the plain rows of h.
__device__ __forceinline__ void write_tagged(unsigned long long *dst, int ridx, float res,
                                             unsigned long long tag) {
  if (ridx == 0xffff) return;   // padding lane
  uint16_t out = f32_to_bf16(res);
  if (out & 0x8000u) out = 0;   // relu between the projections, on the bf16 value
  __hip_atomic_store(&dst[ridx], (tag << 16) | out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The same into a copy kept in wi's row order: `where` is the row's place in
// that order, so that a wavefront's 64 results are 512 consecutive bytes.
__device__ __forceinline__ void write_tagged_placed(unsigned long long *dst, int ridx, int where,
                                                    float res, unsigned long long tag) {
  if (ridx == 0xffff) return;   // padding lane
  uint16_t out = f32_to_bf16(res);
  if (out & 0x8000u) out = 0;   // relu between the projections, on the bf16 value
  __hip_atomic_store(&dst[where], (tag << 16) | out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The activations of wo from the tagged copy into LDS: a thread reads its
// entries, all in flight at once, until each carries `want` (the value then
// belongs to this launch: no count, no fence).  Bounded in time like the other
// waits; a thread that gives up raises the flag, counts itself and stages what
// it has.  Ends with a barrier.  The launch runs 1024 threads a workgroup.
constexpr int kTaggedWidthPerThread = sub1::kTaggedWidth / kMaxThreads;
__device__ __forceinline__ void await_tagged(const PreparedArgs &a, const KindArgs &k,
                                             const unsigned long long *src,
                                             unsigned long long want, uint32_t *xa) {
  constexpr int kMine = kTaggedWidthPerThread;   // entries a thread may have (width / 1024)
  const int width = k.width;
  const int step = blockDim.x;
  for (int z = threadIdx.x * kZeroPeriod; z < physical_columns(width); z += step * kZeroPeriod) {
    xa[2 * z] = 0u;
    xa[2 * z + 1] = 0u;
  }
  unsigned long long v[kMine];
#pragma unroll
  for (int u = 0; u < kMine; u++) v[u] = 0;
  int looks = 0;
  int64_t t0 = 0;
  for (;;) {
    bool all = true;
#pragma unroll
    for (int u = 0; u < kMine; u++) {
      const int i = threadIdx.x + u * step;
      if (i < width && (v[u] >> 16) != want) {
        v[u] = __hip_atomic_load(&src[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        all = all && (v[u] >> 16) == want;
      }
    }
    if (all) break;
    if ((++looks & 15) == 1) {
      const int64_t now = static_cast<int64_t>(wall_clock64());
      if (looks == 1) t0 = now;
      if (now - t0 > a.wait_ticks) {
        sub1::raise_fault(a.sticky, sub1::kFaultWait);
        __hip_atomic_fetch_add(&a.ctrl[kCtrlGaveUp], 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
    __builtin_amdgcn_s_sleep(1);
  }
#pragma unroll
  for (int u = 0; u < kMine; u++) {
    const int i = threadIdx.x + u * step;
    if (i < width) {
      uint32_t *p = xa + 2 * physical_column(i);
      const uint32_t value = static_cast<uint32_t>(v[u]) & 0xffffu;
      p[0] = value;
      p[1] = value << 16;
    }
  }
  __syncthreads();
}

// The same from a copy kept in wi's row order (write_tagged_placed): entry p
// belongs to row `order[p]` of h (0xffff: a padding lane, never written).  A
// thread asks for its part of `order` first - the workgroups that call this
// have nothing else to do until h is there - and then reads its entries, all
// in flight at once, until each
// carries `want` (the value then belongs to this launch: no count, no fence).
// Bounded in time like the other waits; a thread that gives up raises the flag,
// counts itself and stages what it has.  Ends with a barrier.  The launch runs
// 1024 threads a workgroup.
__device__ __forceinline__ void await_tagged_placed(const PreparedArgs &a, const KindArgs &k,
                                             const unsigned long long *src,
                                             const uint16_t *order, int places,
                                             unsigned long long want, uint32_t *xa) {
  constexpr int kMine = kTaggedWidthPerThread;   // entries a thread may have (places / 1024)
  static_assert(kMine % 2 == 0, "rows and values are kept two to a register");
  const int width = k.width;
  const int step = blockDim.x;
  // two 16-bit row indices, and later two bf16 values, to a register: the
  // wavefronts of this workgroup hold their chunks of wo in registers meanwhile
  uint32_t rows[kMine / 2], vals[kMine / 2];
  uint32_t pending = 0;   // bit u: entry u is a row of h and has not been seen with the tag yet
#pragma unroll
  for (int u = 0; u < kMine; u++) {
    const int i = threadIdx.x + u * step;
    const uint32_t r = i < places ? static_cast<uint32_t>(order[i]) : 0xffffu;
    if (u & 1) rows[u / 2] |= r << 16;
    else rows[u / 2] = r;
    if (r != 0xffffu) pending |= 1u << u;
  }
#pragma unroll
  for (int u = 0; u < kMine / 2; u++) vals[u] = 0u;
  for (int z = threadIdx.x * kZeroPeriod; z < physical_columns(width); z += step * kZeroPeriod) {
    xa[2 * z] = 0u;
    xa[2 * z + 1] = 0u;
  }
  int looks = 0;
  int64_t t0 = 0;
  while (pending) {
#pragma unroll
    for (int u = 0; u < kMine; u++) {
      if (pending & (1u << u)) {
        const unsigned long long v = __hip_atomic_load(&src[threadIdx.x + u * step], __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        if ((v >> 16) == want) {
          pending &= ~(1u << u);
          vals[u / 2] |= (static_cast<uint32_t>(v) & 0xffffu) << (16 * (u & 1));
        }
      }
    }
    if (!pending) break;
    if ((++looks & 15) == 1) {
      const int64_t now = static_cast<int64_t>(wall_clock64());
      if (looks == 1) t0 = now;
      if (now - t0 > a.wait_ticks) {
        sub1::raise_fault(a.sticky, sub1::kFaultWait);
        __hip_atomic_fetch_add(&a.ctrl[kCtrlGaveUp], 1, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
    __builtin_amdgcn_s_sleep(1);
  }
#pragma unroll
  for (int u = 0; u < kMine; u++) {
    const uint32_t r = (rows[u / 2] >> (16 * (u & 1))) & 0xffffu;
    if (r != 0xffffu) {
      uint32_t *p = xa + 2 * physical_column(static_cast<int>(r));
      const uint32_t value = (vals[u / 2] >> (16 * (u & 1))) & 0xffffu;
      p[0] = value;
      p[1] = value << 16;
    }
  }
  __syncthreads();
}

// Thread 0 of a workgroup that leaves a launch of the tagged kind: the last one
// out makes the next launch's tag.
__device__ __forceinline__ void leave_tagged(int32_t *ctrl, int workgroups) {
  const int32_t before = __hip_atomic_fetch_add(&ctrl[sub1::kCtrlExits], 1, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
  if (before + 1 == workgroups) {
    __hip_atomic_store(&ctrl[sub1::kCtrlExits], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_fetch_add(reinterpret_cast<unsigned long long *>(ctrl + sub1::kCtrlLaunch), 1ull,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Between the latency form and a token per workgroup: with fewer tokens than
// half the compute units, `parts` workgroups share a token.  Each takes every
// parts-th slice of wi (the slices are ordered longest first, so the shares are
// even), writes its rows of relu(h) to the workspace, counts itself done, waits
// for the others of its token, stages the whole of h and takes every parts-th
// slice of wo.  Unlike tiles of one projection handed out by ticket, every
// workgroup works in both phases, the token's activations are staged once per
// phase and workgroup, and h crosses memory once.
// The workgroups of a token wait for each other.  A grid (tokens x parts) of at
// most one workgroup per compute unit runs all at once on a GPU that does
// nothing else, whatever order the hardware starts them in, and a workgroup's
// place in it is its index: no round trip before the work starts, which
// measured 1.5 to 2.0 us per launch against places by ticket (c-2048 shapes: 4
// tokens 15.9 against 17.4 us, 16 tokens 22.5 against 24.6, 64 tokens 43.0
// against 45.0, 128 tokens 75.9 against 77.9).  Where other work holds compute
// units, the missing workgroups start when that work ends, and the waits are
// bounded in any case.
// A larger grid cannot be on the GPU at once, and there a workgroup takes its
// place by ticket when it starts (by_ticket): the workgroups that are running
// then hold the lowest places, the places of a token are consecutive, so at
// most one token is partly on the GPU whatever order the hardware starts
// workgroups in; all others run to completion and make room.
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_shared_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  __shared__ int s_place;
  uint32_t *xa = lds;
  float *partials = reinterpret_cast<float *>(xa + a.xdwords);
  const KindArgs &ki = a.k[0];
  const KindArgs &ko = a.k[1];
  const int parts = ki.parts;
  int place = blockIdx.x;
  if (a.by_ticket) {
    if (threadIdx.x == 0)
      s_place = __hip_atomic_fetch_add(&a.ctrl[kCtrlTicket], 1, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    place = __builtin_amdgcn_readfirstlane(s_place);
  }
  const int t = place / parts;
  const int part = place - t * parts;
  // the token's activations are asked for before anything else is known
  const uint16_t *x = a.x + static_cast<int64_t>(t) * a.ldx;
  const StagedPairs x_ahead = stage_request(x, ki.width);
  int e = __builtin_amdgcn_readfirstlane(a.token_expert[t]);
  if (e >= a.experts) {
    if (part == 0 && threadIdx.x == 0)
      __hip_atomic_fetch_add(&a.ctrl[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    e = -1;
  }
  if (e < 0) {
    if (part == 0) pass_through(a, ko, t, 0, ko.slices);
    if (a.by_ticket && threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
    return;
  }
  uint16_t *h = a.h + static_cast<int64_t>(t) * ki.height;
  walk_tile(a, ki, static_cast<int64_t>(e) * ki.slices + part, parts,
            (ki.slices - part + parts - 1) / parts, xa, partials,
            [&]() {
              stage_finish(xa, x, ki.width, x_ahead);
              __syncthreads();
            },
            [&](int ridx, float res, int64_t) { write_row(h, ridx, res, kStoreRelu); });
  publish_h(a, t);
  uint16_t *y = a.y + static_cast<int64_t>(t) * a.ldy;
  walk_tile(a, ko, static_cast<int64_t>(e) * ko.slices + part, parts,
            (ko.slices - part + parts - 1) / parts, xa, partials,
            [&]() { await_activations(a, ko, 1, t, xa); },
            [&](int ridx, float res, int64_t) { write_row(y, ridx, res, kStore); });
  done_waiting(a, t);
  if (a.by_ticket && threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
}

// The shared-token kernel for a token or two, h handed over by tag (see
// await_tagged): no drain, no barrier, no count between the projections, and no
// word to give back at the end.  A workgroup's place is its index: the grid is
// at most 64 workgroups.
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_tagged_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *xa = lds;
  float *partials = reinterpret_cast<float *>(xa + a.xdwords);
  const KindArgs &ki = a.k[0];
  const KindArgs &ko = a.k[1];
  const int parts = ki.parts;
  const int t = blockIdx.x / parts;
  const int part = blockIdx.x - t * parts;
  // the token's activations and this launch's tag (one more than the launches
  // so far) are asked for before anything else is known
  const uint16_t *x = a.x + static_cast<int64_t>(t) * a.ldx;
  const StagedPairs x_ahead = stage_request(x, ki.width);
  const unsigned long long tag =
      __hip_atomic_load(reinterpret_cast<unsigned long long *>(a.ctrl + sub1::kCtrlLaunch),
                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
  int e = __builtin_amdgcn_readfirstlane(a.token_expert[t]);
  if (e >= a.experts) {
    if (part == 0 && threadIdx.x == 0)
      __hip_atomic_fetch_add(&a.ctrl[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    e = -1;
  }
  if (e < 0) {
    if (part == 0) pass_through(a, ko, t, 0, ko.slices);
    if (threadIdx.x == 0) leave_tagged(a.ctrl, gridDim.x);
    return;
  }
  unsigned long long *ht = a.tagged + static_cast<int64_t>(t) * sub1::kTaggedWidth;
  walk_tile(a, ki, static_cast<int64_t>(e) * ki.slices + part, parts,
            (ki.slices - part + parts - 1) / parts, xa, partials,
            [&]() {
              stage_finish(xa, x, ki.width, x_ahead);
              __syncthreads();
            },
            [&](int ridx, float res, int64_t) { write_tagged(ht, ridx, res, tag); });
  __syncthreads();   // every wavefront is done with x before h takes its place
  uint16_t *y = a.y + static_cast<int64_t>(t) * a.ldy;
  // (a test that overstates the wait looks for a tag that nobody writes)
  const unsigned long long want = a.wi_expect == parts ? tag : tag + 1;
  walk_tile(a, ko, static_cast<int64_t>(e) * ko.slices + part, parts,
            (ko.slices - part + parts - 1) / parts, xa, partials,
            [&]() { await_tagged(a, ko, ht, want, xa); },
            [&](int ridx, float res, int64_t) { write_row(y, ridx, res, kStore); });
  if (threadIdx.x == 0) leave_tagged(a.ctrl, gridDim.x);
}

// The same with workgroups of its own for wo (one token; two through shapes
// whose wo rows are long).  The first k[0].parts of a token's workgroups walk wi
// (every k[0].parts-th slice from their own; they wait for nobody, so there is
// one per slice where the chip has room) and leave; the others belong to wo and
// ask for all they need of the stream - the descriptions of their slices, the
// row indices and every chunk they will walk (a wavefront's share is one group
// of chunks, which its ring holds) - while wi is still being walked elsewhere.
// Between the last row of h and the first row of y then lie the hand-over and
// a walk whose chunks are in registers already.  For one token a.lane_parts = 2
// workgroups share each slice of wo, 32 lanes (rows) each: the 9 to 14
// wavefronts of a slice gather from one LDS, which takes 32 lanes a pass.
// One token through a c-2048 expert: 13.4 -> 11.9 us (a different expert every
// launch 14.8 -> 12.2), two tokens 15.4 -> 12.8; one token through a base
// expert 11.5 -> 10.7, a large one 11.7 -> 11.5.
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_tagged_split_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *xa = lds;
  float *partials = reinterpret_cast<float *>(xa + a.xdwords);
  const KindArgs &ki = a.k[0];
  const KindArgs &ko = a.k[1];
  const int per_token = ki.parts + ko.parts * a.lane_parts;
  const int t = blockIdx.x / per_token;
  const int place = blockIdx.x - t * per_token;
  const bool for_wo = place >= ki.parts;
  // this launch's tag (one more than the launches so far), and for wi the
  // token's activations, are asked for before anything else is known
  const uint16_t *x = a.x + static_cast<int64_t>(t) * a.ldx;
  StagedPairs x_ahead;
  if (!for_wo) x_ahead = stage_request(x, ki.width);
  const unsigned long long tag =
      __hip_atomic_load(reinterpret_cast<unsigned long long *>(a.ctrl + sub1::kCtrlLaunch),
                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
  int e = __builtin_amdgcn_readfirstlane(a.token_expert[t]);
  if (e >= a.experts) {
    if (place == 0 && threadIdx.x == 0)
      __hip_atomic_fetch_add(&a.ctrl[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    e = -1;
  }
  if (e < 0) {
    if (place == 0) pass_through(a, ko, t, 0, ko.slices);
    if (threadIdx.x == 0) leave_tagged(a.ctrl, gridDim.x);
    return;
  }
  unsigned long long *ht = a.tagged + static_cast<int64_t>(t) * sub1::kTaggedWidth;
  if (!for_wo) {
    walk_tile(a, ki, static_cast<int64_t>(e) * ki.slices + place, ki.parts,
              (ki.slices - place + ki.parts - 1) / ki.parts, xa, partials,
              [&]() {
                stage_finish(xa, x, ki.width, x_ahead);
                __syncthreads();
              },
              [&](int ridx, float res, int64_t slice) {
                const int where = static_cast<int>(slice - static_cast<int64_t>(e) * ki.slices) * 64 +
                                  (threadIdx.x & 63);
                write_tagged_placed(ht, ridx, where, res, tag);
              });
  } else {
    // a.lane_parts workgroups share a slice of wo, each with its part of the
    // lanes (rows): the others do nothing in its walk
    const int part = (place - ki.parts) / a.lane_parts;
    const int lanes_of = (place - ki.parts) % a.lane_parts;
    const bool active = static_cast<int>((threadIdx.x & 63) * a.lane_parts) >> 6 == lanes_of;
    uint16_t *y = a.y + static_cast<int64_t>(t) * a.ldy;
    // (a test that overstates the wait looks for a tag that nobody writes)
    const unsigned long long want = a.wi_expect == ki.parts ? tag : tag + 1;
    walk_tile(a, ko, static_cast<int64_t>(e) * ko.slices + part, ko.parts,
              (ko.slices - part + ko.parts - 1) / ko.parts, xa, partials,
              [&]() {
                await_tagged_placed(a, ko, ht,
                                    ki.row_idx + static_cast<int64_t>(e) * ki.slices * 64,
                                    ki.slices * 64, want, xa);
              },
              [&](int ridx, float res, int64_t) { write_row(y, ridx, res, kStore); }, active);
  }
  if (threadIdx.x == 0) leave_tagged(a.ctrl, gridDim.x);
}

// For the batches too small to occupy the GPU with a wavefront per slice: built
// for latency.  `split` wavefronts share a slice (split_begin / split_run) and
// all of a wavefront's loads leave before anything waits.  With no more tiles
// than compute units every workgroup runs one tile; beyond that the grid is
// persistent.  Tiles are taken by ticket like in the streaming kernel, so a wo
// tile's wait for its token's wi tiles ends for the same reason.
__global__ __launch_bounds__(kMaxThreads) void moe_prepared_small_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  __shared__ int s_ticket;
  uint32_t *xa = lds;
  const bool dynamic = a.ctrl != nullptr;
  const int n_all = a.tokens * (a.k[0].parts + (a.kinds == 2 ? a.k[1].parts : 0));
  int static_ticket = blockIdx.x;
  int next_ticket = 0;
  if (dynamic && threadIdx.x == 0)
    next_ticket = __hip_atomic_fetch_add(&a.ctrl[0], 1, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
  for (;;) {
    int ticket;
    if (dynamic) {
      __syncthreads();   // the previous tile is done with s_ticket, x and the partial sums
      if (threadIdx.x == 0) s_ticket = next_ticket;
      __syncthreads();
      ticket = __builtin_amdgcn_readfirstlane(s_ticket);
    } else {
      __syncthreads();
      ticket = static_ticket;
      static_ticket += gridDim.x;
    }
    if (ticket >= n_all) break;
    const Tile tile = decode_tile(a, ticket, dynamic);
    const int kind = tile.kind, t = tile.t, e = tile.e;
    const KindArgs &k = a.k[kind];
    // the next ticket is asked for late (see the streaming kernel), and not at
    // all when every workgroup has exactly one tile
    auto fetch_next = [&]() {
      if (dynamic && threadIdx.x == 0)
        next_ticket = n_all > static_cast<int>(gridDim.x)
                          ? __hip_atomic_fetch_add(&a.ctrl[0], 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT)
                          : n_all;
    };
    if (a.kinds == 2 && kind == 1 && e < 0) {
      pass_through(a, k, t, tile.s_lo, tile.s_hi);
      fetch_next();
      continue;
    }
    if (e >= 0) {
      int mode;
      uint16_t *dst = tile_output(a, k, kind, t, mode);
      // the launch cuts the matrices so that a tile has at most waves / split slices
      SplitWalk walk = split_begin(a, k, e, tile.s_lo, tile.s_hi);
      await_activations(a, k, kind, t, xa);
      split_run(a, k, walk, xa, dst, mode);
    }
    fetch_next();
    if (a.kinds == 2 && kind == 0 && e >= 0) publish_h(a, t);
    if (a.kinds == 2 && kind == 1 && e >= 0) done_waiting(a, t);
  }
  if (dynamic && threadIdx.x == 0) sub1::leave_launch(a.ctrl, gridDim.x);
}

// y[t] += W x[t] for many tokens through ONE matrix (matrix 0 of the prepared
// set): a tile is (four tokens, part of the matrix), static order, persistent
// grid; the stream of a tile's slices is walked once for its four tokens.
__global__ __launch_bounds__(kMaxThreads) void matvec_group_kernel(PreparedArgs a) {
  extern __shared__ __align__(16) uint32_t lds[];
  uint32_t *xa = lds;
  const KindArgs &k = a.k[0];
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int groups = (a.tokens + kGroupTokens - 1) / kGroupTokens;
  const int n_all = groups * k.parts;
  for (int tile = blockIdx.x; tile < n_all; tile += gridDim.x) {
    const int g = tile / k.parts;
    const int part = tile - g * k.parts;
    const int s_lo = static_cast<int>(static_cast<int64_t>(k.slices) * part / k.parts);
    const int s_hi = static_cast<int>(static_cast<int64_t>(k.slices) * (part + 1) / k.parts);
    const int count = s_hi - s_lo;
    const int passes = (count + waves - 1) / waves;
    const int t0 = g * kGroupTokens;
    const int left = min(a.tokens - t0, kGroupTokens);
    int s = slice_of_pass(0, wave, waves, count);
    SliceWalk cur;
    if (s < count) cur = load_slice(a, k, s_lo + s);
    __syncthreads();   // the previous tile has read its activations
    GroupRows rows;
#pragma unroll
    for (int t = 0; t < kGroupTokens; t++)
      rows.row[t] = t < left ? a.x + static_cast<int64_t>(t0 + t) * a.ldx : nullptr;
    stage_group(xa, rows, k.width);
    __syncthreads();
    for (int pass = 0; s < count; pass++) {
      const int s_next = slice_of_pass(pass + 1, wave, waves, count);
      SliceWalk nxt;
      if (s_next < count) nxt = load_slice(a, k, s_lo + s_next);
      const GroupSums res = run_slice_group(cur, a.stream, xa, nullptr, pass, passes);
#pragma unroll
      for (int t = 0; t < kGroupTokens; t++)
        if (t < left)
          write_row(a.y + static_cast<int64_t>(t0 + t) * a.ldy, cur.ridx, res.v[t], kAccumulate);
      if (s_next < count) cur = nxt;
      s = s_next;
    }
  }
}

// ------------------------------------------------------------ host side --

// The prepare kernels read dec as the fixed dictionary's table (symbols 0..2,
// unused digits zero): refuse any other.  Compared in full on every call (a
// 512 KB copy and a synchronisation; preparing is a load-time step).
int check_dec(const int32_t *dec, hipStream_t stream) {
  std::vector<int32_t> want(SUB1_DEC_WORDS), got(SUB1_DEC_WORDS);
  int rc = sub1_build_tables(want.data(), nullptr);
  if (rc) return fail(rc, "sub1_build_tables failed");
  HIP_TRY(hipMemcpyAsync(got.data(), dec, got.size() * sizeof(int32_t), hipMemcpyDeviceToHost,
                         stream));
  HIP_TRY(hipStreamSynchronize(stream));
  if (std::memcmp(want.data(), got.data(), want.size() * sizeof(int32_t)) != 0)
    return fail(SUB1_ERR_SHAPE,
                "sub1_moe_prepare: dec is not the fixed dictionary; use sub1_moe_grouped");
  return SUB1_OK;
}

// What the prepare passes read: `kinds` groups of `count` matrices each.
struct Source {
  const int32_t *dec;
  KindSource k[2];
  int kinds, count;
  int height[2], width[2];
};

// Pointer tables are copied to the host once and looked at entry by entry.
int check_pointer_table(const void *const *table, int count, size_t align, const char *what,
                        const char *who, hipStream_t s) {
  if (!table) return fail(SUB1_ERR_NULL, "%s: NULL table of %s pointers", who, what);
  if (misaligned(table, 8)) return fail(SUB1_ERR_ALIGN, "%s: misaligned table of %s pointers", who, what);
  std::vector<const void *> host(count);
  HIP_TRY(hipMemcpyAsync(host.data(), table, sizeof(void *) * count, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  for (int i = 0; i < count; i++) {
    if (!host[i]) return fail(SUB1_ERR_NULL, "%s: %s of matrix %d is NULL", who, what, i);
    if (misaligned(host[i], align))
      return fail(SUB1_ERR_ALIGN, "%s: %s of matrix %d is not %zu-byte aligned", who, what, i, align);
  }
  return SUB1_OK;
}

int check_source(const Source &src, const char *who, hipStream_t s = nullptr) {
  if (!src.dec) return fail(SUB1_ERR_NULL, "%s: NULL pointer", who);
  if (src.count < 1) return fail(SUB1_ERR_SHAPE, "%s: %d matrices", who, src.count);
  int64_t slices = 0;
  for (int i = 0; i < src.kinds; i++) {
    const KindSource &k = src.k[i];
    if (src.height[i] < 1 || src.height[i] > 65534 || src.width[i] < 1 ||
        src.width[i] > SUB1_PREPARED_MAX_WIDTH)
      return fail(SUB1_ERR_SHAPE, "%s: matrix %d x %d (height 1..65534, width 1..%d)", who,
                  src.height[i], src.width[i], SUB1_PREPARED_MAX_WIDTH);
    if (k.w_comp_of || k.row_off_of || k.minmax_of) {
      int rc = check_pointer_table(reinterpret_cast<const void *const *>(k.w_comp_of), src.count, 2,
                                   "w_comp", who, s);
      if (!rc)
        rc = check_pointer_table(reinterpret_cast<const void *const *>(k.row_off_of), src.count, 4,
                                 "row_off", who, s);
      if (!rc)
        rc = check_pointer_table(reinterpret_cast<const void *const *>(k.minmax_of), src.count, 4,
                                 "ter_minmax", who, s);
      if (rc) return rc;
    } else {
      if (!k.w_comp || !k.row_off || !k.minmax || (src.count > 1 && !k.code_base))
        return fail(SUB1_ERR_NULL, "%s: NULL pointer", who);
      if (misaligned(k.row_off, 4) || misaligned(k.minmax, 4) || misaligned(k.code_base, 8) ||
          misaligned(k.w_comp, 2))
        return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
    }
    slices += static_cast<int64_t>(src.count) * ((src.height[i] + 63) / 64);
  }
  if (slices > (1 << 24)) return fail(SUB1_ERR_SHAPE, "%s: too many 64-row slices", who);
  if (misaligned(src.dec, 4)) return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
  return SUB1_OK;
}

KindSource stacked(const void *w_comp, const int64_t *code_base, const int32_t *row_off,
                   const void *minmax) {
  return KindSource{static_cast<const uint16_t *>(w_comp), code_base, row_off,
                    static_cast<const uint32_t *>(minmax), nullptr, nullptr, nullptr};
}

KindSource scattered(const void *const *w_comp, const void *const *row_off,
                     const void *const *minmax) {
  return KindSource{nullptr, nullptr, nullptr, nullptr,
                    reinterpret_cast<const uint16_t *const *>(w_comp),
                    reinterpret_cast<const int32_t *const *>(row_off),
                    reinterpret_cast<const uint32_t *const *>(minmax)};
}

Source moe_source(const sub1_moe_stack *st) {
  Source src;
  src.dec = st->dec;
  src.k[0] = stacked(st->w_comp, st->wi_code_base, st->wi_row_off, st->wi_minmax);
  src.k[1] = stacked(st->w_comp, st->wo_code_base, st->wo_row_off, st->wo_minmax);
  src.kinds = 2;
  src.count = st->experts;
  src.height[0] = st->d_ff;
  src.width[0] = st->d_model;
  src.height[1] = st->d_model;
  src.width[1] = st->d_ff;
  return src;
}

Source layers_source(const sub1_moe_layers *l) {
  Source src;
  src.dec = l->dec;
  src.k[0] = scattered(l->wi_w_comp, l->wi_row_off, l->wi_minmax);
  src.k[1] = scattered(l->wo_w_comp, l->wo_row_off, l->wo_minmax);
  src.kinds = 2;
  src.count = l->experts;
  src.height[0] = l->d_ff;
  src.width[0] = l->d_model;
  src.height[1] = l->d_model;
  src.width[1] = l->d_ff;
  return src;
}

Source matrix_source(const sub1_matrix_set *ms) {
  Source src;
  src.dec = ms->dec;
  src.k[0] = stacked(ms->w_comp, ms->code_base, ms->row_off, ms->ter_minmax);
  src.k[1] = KindSource{};
  src.kinds = 1;
  src.count = ms->count;
  src.height[0] = ms->height;
  src.width[0] = ms->width;
  src.height[1] = 0;
  src.width[1] = 0;
  return src;
}

// What a prepared buffer pair holds, in the terms of the kernels.
struct Prepared {
  const void *meta;
  const void *codes;
  int64_t meta_bytes, code_bytes, total_chunks;
  int kinds, count;
  int height[2], width[2];
  int max_chunks[2];
};

struct LayoutResult {
  int64_t meta_bytes, code_bytes, total_chunks;
  int max_chunks[2];
};

int prepare_layout(const Source &src, void *meta, int64_t meta_bytes, LayoutResult *out,
                   hipStream_t s, const char *who) {
  if (!meta || !out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (misaligned(meta, 256)) return fail(SUB1_ERR_ALIGN, "%s: meta must be 256-byte aligned", who);
  const MetaLayout m = meta_layout(src.count, src.kinds, src.height, src.width);
  if (meta_bytes < m.bytes)
    return fail(SUB1_ERR_SHAPE, "%s: meta needs %lld bytes", who, static_cast<long long>(m.bytes));
  int rc = check_dec(src.dec, s);
  if (rc) return rc;
  char *base = static_cast<char *>(meta);
  int32_t *status = reinterpret_cast<int32_t *>(base + m.status);
  int32_t *counts = reinterpret_cast<int32_t *>(base + m.counts);
  zero_words_kernel<<<1, 64, 0, s>>>(status, 4);
  HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(order_rows_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kOrderRowsLds)));
  int64_t slice0 = 0;
  for (int i = 0; i < src.kinds; i++) {
    const KindMeta &k = m.k[i];
    uint16_t *row_len = reinterpret_cast<uint16_t *>(base + k.row_len);
    const int64_t rows = static_cast<int64_t>(src.count) * k.height;
    count_entries_kernel<<<static_cast<unsigned>((rows + 255) / 256), 256, 0, s>>>(
        src.k[i], src.dec, row_len, status, k.height, k.width, rows);
    order_rows_kernel<<<src.count, 256, kOrderRowsLds, s>>>(
        row_len, src.k[i], reinterpret_cast<uint16_t *>(base + k.row_idx),
        reinterpret_cast<uint32_t *>(base + k.minmax),
        reinterpret_cast<uint16_t *>(base + k.slice_len), counts + slice0, status, k.height,
        k.slices, i);
    slice0 += static_cast<int64_t>(src.count) * k.slices;
  }
  scan_counts_kernel<<<1, 1024, 0, s>>>(counts, static_cast<int>(slice0));
  HIP_TRY(hipGetLastError());
  int32_t host[4] = {0, 0, 0, 0};
  int32_t total = 0;
  HIP_TRY(hipMemcpyAsync(host, status, sizeof host, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipMemcpyAsync(&total, counts + slice0, 4, hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  if (host[0])
    return fail(SUB1_ERR_SHAPE, "%s: the codes of %d rows do not cover the width", who, host[0]);
  if (total < 0) return fail(SUB1_ERR_SHAPE, "%s: stream too large", who);
  out->meta_bytes = m.bytes;
  out->total_chunks = total;
  // the entry stream, then one 128-byte checkpoint entry per group of chunks
  out->code_bytes = static_cast<int64_t>(total) * 512 +
                    (static_cast<int64_t>(total) / kGroupChunks + slice0 + 1) * 128;
  out->max_chunks[0] = host[1];
  out->max_chunks[1] = host[2];
  return SUB1_OK;
}

int prepare_codes(const Source &src, const Prepared &p, hipStream_t s, const char *who) {
  if (!p.meta || !p.codes) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (misaligned(p.meta, 256) || misaligned(p.codes, 256))
    return fail(SUB1_ERR_ALIGN, "%s: buffers must be 256-byte aligned", who);
  int rc = check_dec(src.dec, s);
  if (rc) return rc;
  const MetaLayout m = meta_layout(src.count, src.kinds, src.height, src.width);
  const char *base = static_cast<const char *>(p.meta);
  int64_t nslices = 0;
  for (int i = 0; i < src.kinds; i++) nslices += static_cast<int64_t>(src.count) * m.k[i].slices;
  if (p.total_chunks < 0 || p.meta_bytes < m.bytes ||
      p.code_bytes < p.total_chunks * 512 + (p.total_chunks / kGroupChunks + nslices + 1) * 128)
    return fail(SUB1_ERR_SHAPE, "%s: buffers smaller than the layout needs", who);
  uint2 *stream = static_cast<uint2 *>(const_cast<void *>(p.codes));
  uint16_t *ckpt = reinterpret_cast<uint16_t *>(stream + p.total_chunks * 64);
  int64_t first_slice = 0;
  for (int i = 0; i < src.kinds; i++) {
    const KindMeta &k = m.k[i];
    const int64_t kslices = static_cast<int64_t>(src.count) * k.slices;
    const int64_t lanes = kslices * 64;
    emit_entries_kernel<<<static_cast<unsigned>((lanes + 255) / 256), 256, 0, s>>>(
        src.k[i], src.dec, reinterpret_cast<const uint32_t *>(base + k.slice_base),
        reinterpret_cast<const uint16_t *>(base + k.slice_len),
        reinterpret_cast<const uint16_t *>(base + k.row_idx), stream, ckpt, k.height, k.width,
        k.slices, first_slice, lanes);
    first_slice += kslices;
  }
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

// Cut of the matrices for a batch that cannot occupy the GPU with a wavefront
// per slice.  Per projection: a workgroup takes per_wg slices (16 = no sharing)
// and waves / per_wg wavefronts share each slice, at most one per chunk group.
// The choice minimises an estimate of the kernel time in microseconds: a round
// of workgroups costs a fixed part (activations, first loads: they do not
// overlap with the previous round) plus the groups that the busiest SIMD walks
// one after the other.  Sets split and parts of every projection; returns the
// LDS bytes for partial sums, 0 if sharing nothing is estimated best (then
// nothing is changed), and the estimate in *estimate_us.
// The constants come from timing every cut of the Switch base, large and
// c-2048 layers at 1 to 64 tokens on an MI355X; the estimate ranks the cuts and
// is about 13 us below the measured time of a launch.
constexpr double kRoundFixedUs = 6.0;      // a round of workgroups before its first entry
constexpr double kGroupUs = 0.75;          // one group of 72 entries on a SIMD
constexpr double kResidentBonusUs = 8.0;   // wo workgroups already waiting when h arrives
constexpr double kLaunchUs = 13.0;         // measured launch minus estimate
size_t plan_small(PreparedArgs &a, int kinds, int tokens, int cus, int waves, size_t lds_room,
                  double *estimate_us) {
  struct Option {
    int split, parts;
    int64_t tiles;
    double round_us;
    size_t partials;
  };
  Option opt[2][5];
  int nopt[2] = {0, 0};
  for (int i = 0; i < kinds; i++) {
    const KindArgs &k = a.k[i];
    int groups_pow2 = 1;
    while (groups_pow2 < k.groups_max) groups_pow2 *= 2;
    for (int per_wg = 1; per_wg <= waves; per_wg *= 2) {
      Option o;
      o.split = waves / per_wg < groups_pow2 ? waves / per_wg : groups_pow2;
      o.partials = o.split > 1 ? static_cast<size_t>(per_wg) * k.groups_max * 256 : 0;
      if (o.partials > lds_room) continue;
      if (o.split == 1 && per_wg != waves) continue;
      o.parts = (k.slices + per_wg - 1) / per_wg;
      o.tiles = static_cast<int64_t>(tokens) * o.parts;
      const int busy = per_wg * (o.split < k.groups_max ? o.split : k.groups_max);
      const int serial = ((busy + 3) / 4) * ((k.groups_max + o.split - 1) / o.split);
      o.round_us = kRoundFixedUs + kGroupUs * serial;
      opt[i][nopt[i]++] = o;
    }
  }
  double best = 1e30;
  int pick[2] = {-1, -1};
  for (int i0 = 0; i0 < nopt[0]; i0++)
    for (int i1 = 0; i1 < (kinds == 2 ? nopt[1] : 1); i1++) {
      const Option &o0 = opt[0][i0];
      double us = std::max(1.0, static_cast<double>(o0.tiles) / cus) * o0.round_us;
      if (kinds == 2) {
        const Option &o1 = opt[1][i1];
        // wo workgroups that found a free compute unit at the start have their
        // fixed part behind them when h arrives
        const bool resident = o0.tiles + o1.tiles <= cus;
        us += std::max(1.0, static_cast<double>(o1.tiles) / cus) * o1.round_us -
              (resident ? kResidentBonusUs : 0.0);
      }
      if (us < best) {
        best = us;
        pick[0] = i0;
        pick[1] = i1;
      }
    }
  size_t partials = 0;
  for (int i = 0; i < kinds; i++)
    if (opt[i][pick[i]].partials > partials) partials = opt[i][pick[i]].partials;
  *estimate_us = best;
  if (partials == 0) return 0;
  for (int i = 0; i < kinds; i++) {
    a.k[i].split = opt[i][pick[i]].split;
    a.k[i].parts = opt[i][pick[i]].parts;
  }
  return partials;
}

// Passes a workgroup needs for a tile of `slices` slices (a pass = one slice per
// wavefront); a last pass of at most half the wavefronts is shared out between
// all of them by chunk groups and costs a fraction of one.
double tile_passes(int slices, int waves, int groups_max) {
  const int rest = slices % waves;
  double passes = slices / waves;
  if (rest > 0) {
    int split = 1;
    if (rest * 2 <= waves)
      while (split * 2 * rest <= waves && split * 2 <= groups_max) split *= 2;
    passes += split > 1 ? 1.0 / split + 0.1 : 1.0;
  }
  return passes;
}

// The time, in units of a full pass (16 wavefronts, a slice each), that a
// workgroup of `waves` wavefronts needs for `slices` slices: whole passes, then
// the rest either as a pass of its own or, if it is at most half the
// wavefronts, shared out `split` ways.  A pass with few wavefronts in it is
// faster than a full one (less contention for LDS), down to about 0.3 of it.
double part_passes(int slices, int waves, int groups_max) {
  const int rest = slices % waves;
  double passes = slices / waves;
  if (rest > 0) {
    int split = 1;
    if (rest * 2 <= waves) split = std::max(1, std::min(waves / rest, groups_max));
    passes += std::max(static_cast<double>(rest * split) / waves, 0.3) / split;
  }
  return passes;
}

// Launch of the prepared kernels.  kinds == 2: y = wo(relu(wi x)) per token,
// workspace required; kinds == 1: y += W x per token, no workspace.
// `piece`: 0 for a caller's launch; 1 and 2 for the two pieces when a launch is
// split in two (a piece is not split again).
int launch_prepared(const Prepared &p, const int32_t *token_matrix, const void *x, int64_t ldx,
                    void *y, int64_t ldy, int tokens, void *workspace, int64_t workspace_bytes,
                    hipStream_t s, const char *who, int piece = 0, bool may_allocate = true) {
  if (!p.meta || !p.codes || !x || !y) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (p.kinds == 2 && !token_matrix) return fail(SUB1_ERR_NULL, "%s: NULL token_expert", who);
  if (tokens < 0 || tokens > (1 << 20))
    return fail(SUB1_ERR_SHAPE, "%s: tokens %d outside 0..2^20", who, tokens);
  if (ldx < p.width[0] || ldy < (p.kinds == 2 ? p.height[1] : p.height[0]))
    return fail(SUB1_ERR_SHAPE, "%s: token strides smaller than the rows", who);
  if (misaligned(p.meta, 256) || misaligned(p.codes, 256) || misaligned(token_matrix, 4) ||
      misaligned(x, 2) || misaligned(y, 2))
    return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
  const int d_ff = p.kinds == 2 ? p.height[0] : 0;
  if (p.kinds == 2) {
    if (!workspace || workspace_bytes < sub1_moe_workspace_bytes(tokens, d_ff))
      return fail(SUB1_ERR_SHAPE, "%s: workspace of %lld bytes needed", who,
                  static_cast<long long>(sub1_moe_workspace_bytes(tokens, d_ff)));
    if (misaligned(workspace, 256)) return fail(SUB1_ERR_ALIGN, "%s: misaligned workspace", who);
  }
  const MetaLayout m = meta_layout(p.count, p.kinds, p.height, p.width);
  if (p.meta_bytes < m.bytes) return fail(SUB1_ERR_SHAPE, "%s: meta smaller than its layout", who);
  const char *base = static_cast<const char *>(p.meta);

  PreparedArgs a;
  a.by_ticket = 0;
  a.tagged = nullptr;
  a.lane_parts = 1;
  a.stream = static_cast<const uint2 *>(p.codes);
  a.ckpt = reinterpret_cast<const uint16_t *>(a.stream + p.total_chunks * 64);
  a.kinds = p.kinds;
  int wmax = 0;
  for (int i = 0; i < 2; i++) {
    KindArgs &ka = a.k[i];
    if (i >= p.kinds) {
      ka = a.k[0];
      ka.parts = 0;
      continue;
    }
    const KindMeta &k = m.k[i];
    ka.slice_base = reinterpret_cast<const uint32_t *>(base + k.slice_base);
    ka.slice_len = reinterpret_cast<const uint16_t *>(base + k.slice_len);
    ka.row_idx = reinterpret_cast<const uint16_t *>(base + k.row_idx);
    ka.minmax = reinterpret_cast<const uint32_t *>(base + k.minmax);
    ka.slices = k.slices;
    ka.height = k.height;
    ka.width = k.width;
    if (k.width > wmax) wmax = k.width;
  }
  // 16 wavefronts per workgroup.  A count that divides the slice counts better
  // (11 for the c-2048 shapes) leaves fewer idle wavefront slots but measured
  // 10% slower: the kernel needs the wavefronts to hide LDS latency.
  const int waves = 16;
  int device = 0, cus = 0;
  HIP_TRY(hipGetDevice(&device));
  HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  a.token_expert = token_matrix;
  a.x = static_cast<const uint16_t *>(x);
  a.y = static_cast<uint16_t *>(y);
  a.ldx = ldx;
  a.ldy = ldy;
  a.ctrl = nullptr;
  a.h = nullptr;
  a.order = nullptr;
  a.groups = nullptr;
  if (p.kinds == 2) {
    a.ctrl = static_cast<int32_t *>(workspace);
    a.h = reinterpret_cast<uint16_t *>(sub1::h_base(workspace, workspace_bytes, tokens, d_ff));
  }
  a.tokens = tokens;
  a.experts = p.count;
  a.xdwords = activation_dwords(wmax);
  a.hdwords = 0;
  a.tail_room = 0;
  a.wait_ticks = sub1::wait_limit_ticks();
  {
    const int rc = sub1::fault_words(&a.sticky, may_allocate);
    if (rc) return rc;
  }
  const size_t lds_limit = 160 * 1024 - 64;
  const size_t lds_base = static_cast<size_t>(a.xdwords) * 4;
  if (lds_base > lds_limit) return fail(SUB1_ERR_SHAPE, "%s: width %d does not fit LDS", who, wmax);
  // Tiles.  Whole matrices when the tokens alone keep every compute unit busy;
  // otherwise each matrix is cut into parts, down to one slice per wavefront
  // (the persistent kernel).  When even that leaves compute units idle (a
  // handful of tokens), the other kernel runs: a workgroup takes fewer slices
  // (8, 4, 2 or 1) and the wavefronts this frees share the slices, each
  // starting from a position checkpoint.  plan_small picks the cut by estimate.
  const int want = (cus + tokens - 1) / tokens;   // tiles per token and projection
  int64_t first_slice = 0;
  bool idle_units = false;
  for (int i = 0; i < p.kinds; i++) {
    KindArgs &k = a.k[i];
    k.first_slice = first_slice;
    first_slice += static_cast<int64_t>(p.count) * k.slices;
    k.groups_max = (p.max_chunks[i] + kGroupChunks - 1) / kGroupChunks;
    k.split = 1;
    k.tail_split = 0;
    const int max_parts = (k.slices + waves - 1) / waves;
    if (want > max_parts) idle_units = true;
    // Parts per matrix for the streaming kernel: the count that needs the fewest
    // passes of a workgroup per compute unit (a pass = one slice per wavefront;
    // a last pass of at most 8 slices is shared out between the wavefronts and
    // costs a fraction of one).
    double best = 1e30;
    for (int parts = 1; parts <= max_parts; parts++) {
      const int per_tile = (k.slices + parts - 1) / parts;
      const int64_t rounds = (static_cast<int64_t>(tokens) * parts + cus - 1) / cus;
      // a quarter of a pass per tile for staging its activations
      const double cost = rounds * (tile_passes(per_tile, waves, k.groups_max) + 0.25);
      if (cost < best - 1e-9) {
        best = cost;
        k.parts = parts;
      }
    }
  }
  // Many tokens through one matrix: four tokens per walk of the stream, once
  // such tiles (four tokens x 16 slices at least) can occupy half the compute
  // units; below that the per-token kernels, which can cut a matrix finer, are
  // faster (measured on the Switch shapes: 1.9x faster at 568 tokens, 2.3x at
  // 2048, break-even between 50 and 400 tokens depending on the shape).
  const int groups = (tokens + kGroupTokens - 1) / kGroupTokens;
  const int group_parts = (a.k[0].slices + waves - 1) / waves;
  const bool by_groups = p.kinds == 1 && !token_matrix &&
                   static_cast<int64_t>(groups) * group_parts * 2 >= cus;
  if (by_groups) {
    KindArgs &k = a.k[0];
    const int max_parts = group_parts;
    double best = 1e30;
    for (int parts = 1; parts <= max_parts; parts++) {
      const int per_tile = (k.slices + parts - 1) / parts;
      const int64_t rounds = (static_cast<int64_t>(groups) * parts + cus - 1) / cus;
      const double cost = rounds * ((per_tile + waves - 1) / waves + 0.25);
      if (cost < best - 1e-9) {
        best = cost;
        k.parts = parts;
      }
    }
    const int64_t tiles = static_cast<int64_t>(groups) * k.parts;
    const void *fn = reinterpret_cast<const void *>(matvec_group_kernel);
    HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds_base)));
    sub1::note_kernel("matvec_group_kernel");
    matvec_group_kernel<<<static_cast<unsigned>(tiles < cus ? tiles : cus), 64 * waves, lds_base,
                          s>>>(a);
    HIP_TRY(hipGetLastError());
    return SUB1_OK;
  }
  const int stream_parts[2] = {a.k[0].parts, a.k[1].parts};   // plan_small may change them
  size_t lds_partials = 0;
  double small_us = 0.0;
  if (idle_units)
    lds_partials = plan_small(a, p.kinds, tokens, cus, waves, lds_limit - lds_base, &small_us);
  const bool small = lds_partials != 0;
  int64_t tiles = 0;
  for (int i = 0; i < p.kinds; i++) tiles += static_cast<int64_t>(tokens) * a.k[i].parts;
  if (tiles > INT32_MAX - (1 << 20)) return fail(SUB1_ERR_SHAPE, "%s: too many tiles", who);
  // Whole tokens per workgroup with h in LDS (the fused kernel), or the matrices
  // cut into tiles?  By estimate, in microseconds, from measurements on the
  // Switch shapes.  One token on one compute unit takes about 8 us + entries /
  // 23400 per us; the fused kernel takes that per round of workgroups (1.94
  // times that with two workgroups of 8 wavefronts per compute unit).  The cut
  // versions pay about 8 us per launch and, per round of tiles of a projection,
  // 3 us for staging plus the tile's passes, a pass of 16 slices weighing in the
  // token's time by its share of the chunks; where wavefronts share slices
  // (plan_small) their own estimate + 13 us if that is less.
  const size_t lds_fused = (static_cast<size_t>(activation_dwords(a.k[0].width)) +
                            activation_dwords(a.k[1].width)) * 4;
  bool fused = false;
  int fused_per_cu = 1;
  int shared_parts = 0;
  if (p.kinds == 2 && lds_fused <= lds_limit) {
    const double token_us = 8.0 + static_cast<double>(p.total_chunks) * (64.0 * kFields) /
                                      p.count / 23400.0;
    auto fused_estimate = [&](int64_t n, int *per_cu) {
      const int64_t rounds16 = (n + cus - 1) / cus, rounds8 = (n + 2 * cus - 1) / (2 * cus);
      *per_cu = 1;
      if (2 * lds_fused <= lds_limit && 1.94 * rounds8 < rounds16) {
        *per_cu = 2;
        return 1.94 * rounds8 * token_us;
      }
      return rounds16 * token_us;
    };
    const double fused_us = fused_estimate(tokens, &fused_per_cu);
    double weight = 0.0;
    for (int i = 0; i < 2; i++) weight += static_cast<double>(a.k[i].slices) * p.max_chunks[i];
    double cut_us = 8.0;
    for (int i = 0; i < 2; i++) {
      const KindArgs &k = a.k[i];
      const int per_tile = (k.slices + stream_parts[i] - 1) / stream_parts[i];
      const int64_t rounds = (static_cast<int64_t>(tokens) * stream_parts[i] + cus - 1) / cus;
      const double pass_us = (token_us - 8.0) * waves * p.max_chunks[i] / weight;
      cut_us += rounds * (tile_passes(per_tile, waves, k.groups_max) * pass_us + 3.0);
    }
    cut_us *= 1.05;   // the estimate ran 5 to 8% low where tiles take several rounds
    if (small) cut_us = std::min(cut_us, small_us + kLaunchUs);
    // Up to a token per compute unit: several workgroups per token, each in
    // both projections (moe_prepared_shared_kernel), one workgroup per compute
    // unit at a time.  Up to half a token per unit that is all of them at once;
    // up to one, two rounds can still beat whole tokens on half the units (they
    // do for the c-2048 shapes at 129 to 170 tokens).  Fixed costs of 8 us plus
    // staging (by the widths), the walk of the largest share, and what more
    // workgroups cost in dispatch and in waiting for each other; measured on
    // the Switch shapes it is the fastest form from 2 tokens (1 for the smaller
    // shapes) to half the compute units: 1.1 to 1.5 times faster than cutting
    // by projection.
    const size_t lds_shared = lds_base + static_cast<size_t>(waves / 2) *
                                             std::max(a.k[0].groups_max, a.k[1].groups_max) * 256;
    auto shared_estimate = [&](int64_t n, int *best_parts) {
      double best_us = 1e30;
      *best_parts = 0;
      if (n > cus || lds_shared > lds_limit) return best_us;
      for (int parts = 2; parts <= 64 && n * parts <= 2 * cus; parts++) {
        // beyond one workgroup per compute unit the rest of the grid starts as
        // the first tokens finish: two rounds, measured 7% above twice one
        const int rounds = n * parts > cus ? 2 : 1;
        double task = (a.k[0].width + a.k[1].width) / 2700.0 + 0.03 * parts;
        for (int i = 0; i < 2; i++) {
          const KindArgs &k = a.k[i];
          const double pass_us = (token_us - 8.0) * waves * p.max_chunks[i] / weight;
          task += part_passes((k.slices + parts - 1) / parts, waves, k.groups_max) * pass_us + 0.5;
        }
        const double us = 8.0 + (rounds == 2 ? 2.24 : 1.0) * task + 0.008 * n * parts;
        if (us < best_us) {
          best_us = us;
          *best_parts = parts;
        }
      }
      return best_us;
    };
    int best_parts = 0;
    const double shared_us = shared_estimate(tokens, &best_parts);
    if (best_parts && shared_us < cut_us && shared_us < fused_us) shared_parts = best_parts;
    // More than a token per compute unit, and a last round of whole tokens that
    // would be mostly empty: whole rounds as they are, the rest as shared
    // tokens in a launch of its own (300 tokens on 256 units: 256 whole and 44
    // shared instead of cut tiles or two rounds; measured 5 to 25% faster just
    // above a whole number of rounds).  The second launch is taken as 6 us, and
    // the split must promise 7%: the estimates are no better than that.  Not
    // where tokens are grouped by expert, which wants them all in one launch.
    if (piece == 0 && tokens > cus && tokens % cus != 0 &&
        !(tokens >= 4 * static_cast<int64_t>(p.count) && tokens >= 4 * cus)) {
      const int whole = tokens / cus * cus;
      int unused = 0, rest_parts = 0;
      const double split_us = fused_estimate(whole, &unused) +
                              shared_estimate(tokens - whole, &rest_parts) + 6.0;
      if (rest_parts && split_us < 0.93 * std::min(cut_us, fused_us)) {
        const uint16_t *xs = static_cast<const uint16_t *>(x);
        uint16_t *ys = static_cast<uint16_t *>(y);
        const int rc = launch_prepared(p, token_matrix, xs, ldx, ys, ldy, whole, workspace,
                                       workspace_bytes, s, who, 1, may_allocate);
        if (rc) return rc;
        return launch_prepared(p, token_matrix + whole, xs + static_cast<int64_t>(whole) * ldx, ldx,
                               ys + static_cast<int64_t>(whole) * ldy, ldy, tokens - whole,
                               workspace, workspace_bytes, s, who, 2, may_allocate);
      }
    }
    if (!shared_parts && fused_us < cut_us) {
      fused = true;
      for (int i = 0; i < 2; i++) {
        a.k[i].parts = 1;
        a.k[i].split = 1;
      }
    }
  }
  if (shared_parts) {
    for (int i = 0; i < 2; i++) {
      a.k[i].parts = shared_parts;
      a.k[i].split = 1;
    }
    a.tail_room = (waves / 2) * std::max(a.k[0].groups_max, a.k[1].groups_max);
    a.wi_expect = a.k[0].parts + sub1::expect_extra();
    a.by_ticket = static_cast<int64_t>(tokens) * shared_parts > cus;
    const size_t lds_shared = lds_base + static_cast<size_t>(a.tail_room) * 256;
    const void *fn = reinterpret_cast<const void *>(moe_prepared_shared_kernel);
    HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds_shared)));
    // A token or two: h goes from wi to wo by tag (every workgroup of wo reads
    // all of it, eight bytes an entry: for small grids only).  One token, and
    // two where wo's rows are long (eight groups of chunks and more: the c-2048
    // shapes), give wo workgroups of its own, as many as give every wavefront at
    // most one group of chunks, so that all of wo's stream is in registers before
    // h is there (two tokens through the shorter rows of the base and large
    // shapes measured 11.4 and 12.4 us that way against 11.5 and 11.8).
    if (tokens <= sub1::kTaggedTokens && 64 * waves == kMaxThreads) {
      const KindArgs &ko = a.k[1];
      const int per_wg = std::max(1, waves / std::max(1, ko.groups_max));
      const int wo_parts = (ko.slices + per_wg - 1) / per_wg;
      // One token: two workgroups share each slice of wo by lanes, 32 rows each.
      // The walk of a slice's 9 to 14 wavefronts is bound by the one LDS they
      // gather from, and a gather of 32 lanes takes the LDS one pass instead of
      // two (c-2048: 12.3 -> 11.9 us; in four parts, and for two tokens, the
      // larger grid costs more than the walk gains: 12.6, and 12.9 -> 13.4).
      const int lane_parts = tokens == 1 ? 2 : 1;
      const bool own_wo = (tokens == 1 || ko.groups_max >= 8) &&
                          static_cast<int64_t>(tokens) * (shared_parts + wo_parts * lane_parts) <= cus;
      if (own_wo || static_cast<int64_t>(tokens) * shared_parts <= 64) {
        a.tagged = reinterpret_cast<unsigned long long *>(a.ctrl + sub1::kCtrlTagged);
        const void *tagged_fn =
            own_wo ? reinterpret_cast<const void *>(moe_prepared_tagged_split_kernel)
                   : reinterpret_cast<const void *>(moe_prepared_tagged_kernel);
        HIP_TRY(hipFuncSetAttribute(tagged_fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    static_cast<int>(lds_shared)));
        if (own_wo) {
          a.k[1].parts = wo_parts;
          // wi's workgroups wait for nobody, so the more of them the shorter their
          // walks: up to a slice each, within two thirds of the compute units
          // that wo leaves a token (one token through a c-2048 expert: 96 instead
          // of 48 workgroups 12.7 -> 12.4 us; two tokens, 63 each instead of 24:
          // 13.8 -> 12.8; with all units taken two tokens measured 13.4)
          a.lane_parts = lane_parts;
          shared_parts = std::max(shared_parts,
                                  std::min(a.k[0].slices, (cus / tokens - wo_parts * lane_parts) * 2 / 3));
          a.k[0].parts = shared_parts;
          a.wi_expect = a.k[0].parts + sub1::expect_extra();
          sub1::note_kernel("moe_prepared_tagged_split_kernel");
          moe_prepared_tagged_split_kernel<<<tokens * (shared_parts + wo_parts * lane_parts), 64 * waves,
                                             lds_shared, s>>>(a);
        } else {
          sub1::note_kernel("moe_prepared_tagged_kernel");
          moe_prepared_tagged_kernel<<<tokens * shared_parts, 64 * waves, lds_shared, s>>>(a);
        }
        HIP_TRY(hipGetLastError());
        return SUB1_OK;
      }
    }
    sub1::note_kernel("moe_prepared_shared_kernel");
    moe_prepared_shared_kernel<<<tokens * shared_parts, 64 * waves, lds_shared, s>>>(a);
    HIP_TRY(hipGetLastError());
    return SUB1_OK;
  }
  if (fused) {
    a.xdwords = activation_dwords(a.k[0].width);
    a.hdwords = activation_dwords(a.k[1].width);
    // Several tokens per expert: three or four tokens of one expert walk its
    // streams together (measured on the Switch shapes: nothing to gain below
    // four tokens per expert and four per compute unit, 1.1 to 1.3 times faster
    // at 8 to 16 per expert, 1.7 to 1.95 at 32 to 64).  The tables of the
    // grouping go where the other kernels keep h (this one keeps it in LDS).
    const int64_t table_ints = 4 * (static_cast<int64_t>(p.count) + 1);
    const int64_t order_ints = (tokens + 1) / 2 * 2;
    const int64_t group_bytes = (table_ints + order_ints) * 4 + static_cast<int64_t>(tokens) * 8;
    const bool grouped = tokens >= 4 * static_cast<int64_t>(p.count) && tokens >= 4 * cus &&
                         group_bytes <= static_cast<int64_t>(tokens) * d_ff * 2;
    // wo's last pass: with at most half the wavefronts busy, the idle ones take
    // groups of those slices (partial sums go where x was)
    KindArgs &ko = a.k[1];
    // Two workgroups of 8 wavefronts per compute unit, where two fit LDS and it
    // costs no round of workgroups more (568 tokens are three rounds of
    // workgroups of 16 but two, each twice as long, of workgroups of 8): one's
    // barriers between the phases of a token fall into the other's work
    // (measured 3% faster than one of 16 on 2048 tokens).
    const int per_cu = fused_per_cu;
    const int fw = waves / per_cu;   // wavefronts per workgroup
    const int rest = ko.slices % fw;
    if (rest > 0 && rest * 2 <= fw && ko.groups_max > 1) {
      int split = 1;
      while (split * 2 * rest <= fw && split * 2 <= ko.groups_max) split *= 2;
      // a partial sum per group of chunks and lane, four with grouped tokens
      const size_t partials = static_cast<size_t>(rest) * ko.groups_max * (grouped ? 1024 : 256);
      if (split > 1 && partials <= static_cast<size_t>(a.xdwords) * 4) ko.tail_split = split;
    }
    // a stream larger than the last-level cache (256 MB), swept by at least a
    // token per compute unit: the chunks are loaded as read-once data
    const bool once = !grouped && p.total_chunks * 512 > (256ll << 20);
    const void *fn = grouped ? reinterpret_cast<const void *>(moe_prepared_fused_kernel<true, false>)
                     : once  ? reinterpret_cast<const void *>(moe_prepared_fused_kernel<false, true>)
                             : reinterpret_cast<const void *>(moe_prepared_fused_kernel<false, false>);
    HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds_fused)));
    if (grouped) {
      int32_t *tab = reinterpret_cast<int32_t *>(a.h);
      int32_t *order = tab + table_ints;
      int2 *groups = reinterpret_cast<int2 *>(order + order_ints);
      group_tokens_kernel<<<1, 1024, 0, s>>>(token_matrix, tokens, p.count, tab, order, groups,
                                              a.ctrl);
      a.order = order;
      a.groups = groups;
    }
    const int grid = tokens < cus * per_cu ? tokens : cus * per_cu;
    sub1::note_kernel(grouped ? "moe_prepared_fused_kernel<true, false>"
                      : once  ? "moe_prepared_fused_kernel<false, true>"
                              : "moe_prepared_fused_kernel<false, false>");
    if (grouped)
      moe_prepared_fused_kernel<true, false><<<grid, 64 * fw, lds_fused, s>>>(a);
    else if (once)
      moe_prepared_fused_kernel<false, true><<<grid, 64 * fw, lds_fused, s>>>(a);
    else
      moe_prepared_fused_kernel<false, false><<<grid, 64 * fw, lds_fused, s>>>(a);
    HIP_TRY(hipGetLastError());
    return SUB1_OK;
  }
  // the persistent kernel shares out a tile's short last pass: room for the
  // partial sums of up to half the wavefronts' slices
  size_t lds_tail = 0;
  a.tail_room = 0;
  if (!small) {
    int groups_max = 0;
    for (int i = 0; i < p.kinds; i++) groups_max = std::max(groups_max, a.k[i].groups_max);
    lds_tail = static_cast<size_t>(waves / 2) * groups_max * 256;
    if (lds_base + lds_tail <= lds_limit)
      a.tail_room = (waves / 2) * groups_max;
    else
      lds_tail = 0;
  }
  const size_t lds = lds_base + lds_partials + lds_tail;
  a.wi_expect = a.k[0].parts + sub1::expect_extra();
  // Batches too small to occupy the GPU with a wavefront per slice go to the
  // latency kernel, everything else to the persistent one; either way at most
  // a workgroup per compute unit (16 wavefronts of 72 to 80 registers each).
  const void *fn = small ? reinterpret_cast<const void *>(moe_prepared_small_kernel)
                         : reinterpret_cast<const void *>(moe_prepared_kernel);
  HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds)));
  if (small) {
    const int64_t grid = tiles < cus ? tiles : cus;
    sub1::note_kernel("moe_prepared_small_kernel");
    moe_prepared_small_kernel<<<static_cast<unsigned>(grid), 64 * waves, lds, s>>>(a);
  } else {
    const int64_t grid = tiles < cus ? tiles : cus;
    sub1::note_kernel("moe_prepared_kernel");
    moe_prepared_kernel<<<static_cast<unsigned>(grid), 64 * waves, lds, s>>>(a);
  }
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

// The symbols of matrix `index` of kind `kind`, read back from the stream.
int decode_prepared(const Prepared &p, int kind, int index, void *tern_out, hipStream_t s,
                    const char *who) {
  if (!p.meta || !p.codes || !tern_out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (kind < 0 || kind >= p.kinds || index < 0 || index >= p.count)
    return fail(SUB1_ERR_SHAPE, "%s: no matrix %d of kind %d", who, index, kind);
  if (misaligned(p.meta, 256) || misaligned(p.codes, 256))
    return fail(SUB1_ERR_ALIGN, "%s: misaligned pointer", who);
  const MetaLayout m = meta_layout(p.count, p.kinds, p.height, p.width);
  if (p.meta_bytes < m.bytes) return fail(SUB1_ERR_SHAPE, "%s: meta smaller than its layout", who);
  const char *base = static_cast<const char *>(p.meta);
  const KindMeta &k = m.k[kind];
  const int64_t n = static_cast<int64_t>(k.height) * k.width;
  uint8_t *out = static_cast<uint8_t *>(tern_out);
  fill_bytes_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(out, n, 0);
  decode_entries_kernel<<<(k.slices * 64 + 255) / 256, 256, 0, s>>>(
      static_cast<const uint2 *>(p.codes), reinterpret_cast<const uint32_t *>(base + k.slice_base),
      reinterpret_cast<const uint16_t *>(base + k.slice_len),
      reinterpret_cast<const uint16_t *>(base + k.row_idx), out,
      static_cast<int64_t>(index) * k.slices, k.slices, k.width);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

int check_moe_stack(const sub1_moe_stack *st, const char *who) {
  if (!st) return fail(SUB1_ERR_NULL, "%s: NULL stack", who);
  if (st->experts < 1 || st->d_model < 1 || st->d_ff < 1)
    return fail(SUB1_ERR_SHAPE, "%s: experts %d d_model %d d_ff %d", who, st->experts,
                st->d_model, st->d_ff);
  return check_source(moe_source(st), who);
}

int check_moe_layers(const sub1_moe_layers *l, const char *who, hipStream_t s) {
  if (!l) return fail(SUB1_ERR_NULL, "%s: NULL layers", who);
  if (l->experts < 1 || l->d_model < 1 || l->d_ff < 1)
    return fail(SUB1_ERR_SHAPE, "%s: experts %d d_model %d d_ff %d", who, l->experts, l->d_model,
                l->d_ff);
  return check_source(layers_source(l), who, s);
}

void fill_moe_prepared(sub1_moe_prepared *out, void *meta, const LayoutResult &r, int experts,
                       int d_model, int d_ff) {
  out->meta = meta;
  out->codes = nullptr;
  out->meta_bytes = r.meta_bytes;
  out->code_bytes = r.code_bytes;
  out->total_chunks = r.total_chunks;
  out->experts = experts;
  out->d_model = d_model;
  out->d_ff = d_ff;
  out->max_chunks[0] = r.max_chunks[0];
  out->max_chunks[1] = r.max_chunks[1];
}

int check_matrix_set(const sub1_matrix_set *ms, const char *who) {
  if (!ms) return fail(SUB1_ERR_NULL, "%s: NULL matrix set", who);
  return check_source(matrix_source(ms), who);
}

}  // namespace

// ================================================================ C ABI =====


extern "C" int64_t sub1_moe_prepared_meta_bytes(int experts, int d_model, int d_ff) {
  if (experts < 1 || d_model < 1 || d_ff < 1) return 0;
  return moe_layout(experts, d_model, d_ff).bytes;
}

extern "C" int sub1_moe_prepare_layout(const sub1_moe_stack *st, void *meta, int64_t meta_bytes,
                                       sub1_moe_prepared *out, void *stream) {
  int rc = check_moe_stack(st, "sub1_moe_prepare_layout");
  if (rc) return rc;
  if (!out) return fail(SUB1_ERR_NULL, "sub1_moe_prepare_layout: NULL argument");
  LayoutResult r;
  rc = prepare_layout(moe_source(st), meta, meta_bytes, &r, static_cast<hipStream_t>(stream),
                      "sub1_moe_prepare_layout");
  if (rc) return rc;
  fill_moe_prepared(out, meta, r, st->experts, st->d_model, st->d_ff);
  return SUB1_OK;
}

extern "C" int sub1_moe_prepare_layout_from_layers(const sub1_moe_layers *layers, void *meta,
                                                   int64_t meta_bytes, sub1_moe_prepared *out,
                                                   void *stream) {
  const char *who = "sub1_moe_prepare_layout_from_layers";
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = check_moe_layers(layers, who, s);
  if (rc) return rc;
  if (!out) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  LayoutResult r;
  rc = prepare_layout(layers_source(layers), meta, meta_bytes, &r, s, who);
  if (rc) return rc;
  fill_moe_prepared(out, meta, r, layers->experts, layers->d_model, layers->d_ff);
  return SUB1_OK;
}

extern "C" int sub1_moe_prepared_entry_counts(const sub1_moe_prepared *p, int64_t *walked,
                                              int64_t *in_rows, void *stream) {
  const char *who = "sub1_moe_prepared_entry_counts";
  if (!p || !walked || !in_rows) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (!p->meta) return fail(SUB1_ERR_NULL, "%s: NULL meta", who);
  const MetaLayout m = moe_layout(p->experts, p->d_model, p->d_ff);
  if (p->meta_bytes < m.bytes) return fail(SUB1_ERR_SHAPE, "%s: meta smaller than its layout", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const char *base = static_cast<const char *>(p->meta);
  *walked = *in_rows = 0;
  for (int i = 0; i < 2; i++) {
    const KindMeta &k = m.k[i];
    const int64_t nslices = static_cast<int64_t>(p->experts) * k.slices;
    const int64_t nrows = static_cast<int64_t>(p->experts) * k.height;
    std::vector<uint16_t> slice_len(nslices), row_len(nrows);
    HIP_TRY(hipMemcpyAsync(slice_len.data(), base + k.slice_len, nslices * 2, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipMemcpyAsync(row_len.data(), base + k.row_len, nrows * 2, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    // the rows that pad a matrix's last slice are walked like any other lane
    for (int64_t g = 0; g < nslices; g++) *walked += 64ll * slice_len[g];
    for (int64_t g = 0; g < nrows; g++) *in_rows += row_len[g];
  }
  return SUB1_OK;
}

namespace {
Prepared from_moe(const sub1_moe_prepared *p) {
  Prepared q;
  q.meta = p->meta;
  q.codes = p->codes;
  q.meta_bytes = p->meta_bytes;
  q.code_bytes = p->code_bytes;
  q.total_chunks = p->total_chunks;
  q.kinds = 2;
  q.count = p->experts;
  q.height[0] = p->d_ff;
  q.width[0] = p->d_model;
  q.height[1] = p->d_model;
  q.width[1] = p->d_ff;
  q.max_chunks[0] = p->max_chunks[0];
  q.max_chunks[1] = p->max_chunks[1];
  return q;
}

Prepared from_matrix(const sub1_matrix_prepared *p) {
  Prepared q;
  q.meta = p->meta;
  q.codes = p->codes;
  q.meta_bytes = p->meta_bytes;
  q.code_bytes = p->code_bytes;
  q.total_chunks = p->total_chunks;
  q.kinds = 1;
  q.count = p->count;
  q.height[0] = p->height;
  q.width[0] = p->width;
  q.height[1] = 0;
  q.width[1] = 0;
  q.max_chunks[0] = p->max_chunks;
  q.max_chunks[1] = 0;
  return q;
}

bool bad_dims(int count, int h, int w) {
  return count < 1 || h < 1 || w < 1 || h > 65534 || w > SUB1_PREPARED_MAX_WIDTH;
}
}  // namespace

// ------------------------------------------------ launch without allocating --
//
// Scratch memory of sub1_moe_grouped_prepared_static: what the workspace
// argument of sub1_moe_grouped_prepared brings in (control words, then h), held
// by every GPU the library runs on until the process ends.  The name is a
// host-side stand-in, not a device address: host code uses the per-device
// address that hipGetSymbolAddress returns, never the name.
static __device__ __align__(256) unsigned char scratch[SUB1_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};   // each GPU's own copy of `scratch`

// The current device's address of the scratch array (resolved once per device,
// with that device current; no allocation).
int scratch_of_current_device(void **out) {
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return fail(SUB1_ERR_SHAPE, "device %d: the static scratch serves devices 0..%d", device,
                kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void *ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(SUB1_ERR_HIP, "hipGetSymbolAddress returned no address for the scratch");
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return SUB1_OK;
}
}  // namespace

extern "C" int sub1_init(void) {
  int32_t *sticky = nullptr;
  int rc = sub1::fault_words(&sticky, true);
  if (rc) return rc;
  void *ws = nullptr;
  return scratch_of_current_device(&ws);
}

extern "C" int sub1_moe_grouped_prepared_static(const sub1_moe_prepared *p,
                                                const int32_t *token_expert, const void *x,
                                                void *y, int tokens, void *stream) {
  const char *who = "sub1_moe_grouped_prepared_static";
  if (!p) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (tokens == 0) return SUB1_OK;
  if (bad_dims(p->experts, p->d_ff, p->d_model) || bad_dims(p->experts, p->d_model, p->d_ff))
    return fail(SUB1_ERR_SHAPE, "%s: experts %d d_model %d d_ff %d", who, p->experts, p->d_model,
                p->d_ff);
  if (tokens < 0) return fail(SUB1_ERR_SHAPE, "%s: tokens %d", who, tokens);
  // The array is split for good: control words for SUB1_STATIC_MAX_TOKENS at its
  // head, h in what follows.  Stacks of different d_ff share the array, and h of
  // one launch must never lie on words that another, larger launch counts with.
  const int64_t h_room = SUB1_STATIC_SCRATCH_BYTES - sub1::control_bytes(SUB1_STATIC_MAX_TOKENS);
  const int64_t h_bytes = static_cast<int64_t>(tokens) * p->d_ff * 2;
  if (tokens > SUB1_STATIC_MAX_TOKENS || h_bytes > h_room)
    return fail(SUB1_ERR_SHAPE,
                "%s: %d tokens of d_ff %d need %lld bytes for h, the static buffer serves up to "
                "%d tokens and %lld bytes of h; use sub1_moe_grouped_prepared with a workspace",
                who, tokens, p->d_ff, static_cast<long long>(h_bytes), SUB1_STATIC_MAX_TOKENS,
                static_cast<long long>(h_room));
  void *ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc) return rc;
  return launch_prepared(from_moe(p), token_expert, x, p->d_model, y, p->d_model, tokens, ws,
                         SUB1_STATIC_SCRATCH_BYTES, static_cast<hipStream_t>(stream), who, 0,
                         /*may_allocate=*/false);
}

extern "C" int sub1_static_scratch_pointer(void **out) {
  if (!out) return fail(SUB1_ERR_NULL, "sub1_static_scratch_pointer: NULL argument");
  return scratch_of_current_device(out);
}

extern "C" int sub1_static_scratch_reset(void *stream) {
  void *ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc) return rc;
  const int words = static_cast<int>(sub1::control_bytes(SUB1_STATIC_MAX_TOKENS) / 4);
  zero_words_kernel<<<(words + 255) / 256, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<int32_t *>(ws), words);
  HIP_TRY(hipGetLastError());
  return SUB1_OK;
}

extern "C" int sub1_moe_prepare_codes(const sub1_moe_stack *st, const sub1_moe_prepared *p,
                                      void *stream) {
  int rc = check_moe_stack(st, "sub1_moe_prepare_codes");
  if (rc) return rc;
  if (!p) return fail(SUB1_ERR_NULL, "sub1_moe_prepare_codes: NULL argument");
  if (p->experts != st->experts || p->d_model != st->d_model || p->d_ff != st->d_ff)
    return fail(SUB1_ERR_SHAPE, "sub1_moe_prepare_codes: the layout belongs to another stack");
  return prepare_codes(moe_source(st), from_moe(p), static_cast<hipStream_t>(stream),
                       "sub1_moe_prepare_codes");
}

extern "C" int sub1_moe_prepare_codes_from_layers(const sub1_moe_layers *layers,
                                                  const sub1_moe_prepared *p, void *stream) {
  const char *who = "sub1_moe_prepare_codes_from_layers";
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = check_moe_layers(layers, who, s);
  if (rc) return rc;
  if (!p) return fail(SUB1_ERR_NULL, "%s: NULL argument", who);
  if (p->experts != layers->experts || p->d_model != layers->d_model || p->d_ff != layers->d_ff)
    return fail(SUB1_ERR_SHAPE, "%s: the layout belongs to other layers", who);
  return prepare_codes(layers_source(layers), from_moe(p), s, who);
}

extern "C" int sub1_moe_grouped_prepared(const sub1_moe_prepared *p, const int32_t *token_expert,
                                         const void *x, void *y, int tokens, void *workspace,
                                         int64_t workspace_bytes, void *stream) {
  if (!p) return fail(SUB1_ERR_NULL, "sub1_moe_grouped_prepared: NULL argument");
  if (tokens == 0) return SUB1_OK;
  if (bad_dims(p->experts, p->d_ff, p->d_model) || bad_dims(p->experts, p->d_model, p->d_ff))
    return fail(SUB1_ERR_SHAPE, "sub1_moe_grouped_prepared: experts %d d_model %d d_ff %d",
                p->experts, p->d_model, p->d_ff);
  return launch_prepared(from_moe(p), token_expert, x, p->d_model, y, p->d_model, tokens,
                         workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                         "sub1_moe_grouped_prepared");
}

extern "C" int sub1_moe_prepared_decode(const sub1_moe_prepared *p, int expert, int projection,
                                        void *tern_out, void *stream) {
  if (!p) return fail(SUB1_ERR_NULL, "sub1_moe_prepared_decode: NULL argument");
  if (bad_dims(p->experts, p->d_ff, p->d_model) || bad_dims(p->experts, p->d_model, p->d_ff))
    return fail(SUB1_ERR_SHAPE, "sub1_moe_prepared_decode: experts %d d_model %d d_ff %d",
                p->experts, p->d_model, p->d_ff);
  return decode_prepared(from_moe(p), projection, expert, tern_out,
                         static_cast<hipStream_t>(stream), "sub1_moe_prepared_decode");
}

extern "C" int64_t sub1_matrix_prepared_meta_bytes(int count, int height, int width) {
  if (count < 1 || height < 1 || width < 1) return 0;
  return matrix_layout(count, height, width).bytes;
}

extern "C" int sub1_matrix_prepare_layout(const sub1_matrix_set *ms, void *meta,
                                          int64_t meta_bytes, sub1_matrix_prepared *out,
                                          void *stream) {
  int rc = check_matrix_set(ms, "sub1_matrix_prepare_layout");
  if (rc) return rc;
  if (!out) return fail(SUB1_ERR_NULL, "sub1_matrix_prepare_layout: NULL argument");
  LayoutResult r;
  rc = prepare_layout(matrix_source(ms), meta, meta_bytes, &r, static_cast<hipStream_t>(stream),
                      "sub1_matrix_prepare_layout");
  if (rc) return rc;
  out->meta = meta;
  out->codes = nullptr;
  out->meta_bytes = r.meta_bytes;
  out->code_bytes = r.code_bytes;
  out->total_chunks = r.total_chunks;
  out->count = ms->count;
  out->height = ms->height;
  out->width = ms->width;
  out->max_chunks = r.max_chunks[0];
  return SUB1_OK;
}

extern "C" int sub1_matrix_prepare_codes(const sub1_matrix_set *ms,
                                         const sub1_matrix_prepared *p, void *stream) {
  int rc = check_matrix_set(ms, "sub1_matrix_prepare_codes");
  if (rc) return rc;
  if (!p) return fail(SUB1_ERR_NULL, "sub1_matrix_prepare_codes: NULL argument");
  if (p->count != ms->count || p->height != ms->height || p->width != ms->width)
    return fail(SUB1_ERR_SHAPE, "sub1_matrix_prepare_codes: the layout belongs to other matrices");
  return prepare_codes(matrix_source(ms), from_matrix(p), static_cast<hipStream_t>(stream),
                       "sub1_matrix_prepare_codes");
}

extern "C" int sub1_matvec_prepared(const sub1_matrix_prepared *p, const int32_t *token_matrix,
                                    const void *x, int64_t ldx, void *y, int64_t ldy,
                                    int tokens, void *stream) {
  if (!p) return fail(SUB1_ERR_NULL, "sub1_matvec_prepared: NULL argument");
  if (tokens == 0) return SUB1_OK;
  if (bad_dims(p->count, p->height, p->width))
    return fail(SUB1_ERR_SHAPE, "sub1_matvec_prepared: %d matrices of %d x %d", p->count,
                p->height, p->width);
  return launch_prepared(from_matrix(p), token_matrix, x, ldx, y, ldy, tokens, nullptr, 0,
                         static_cast<hipStream_t>(stream), "sub1_matvec_prepared");
}

extern "C" int sub1_matrix_prepared_decode(const sub1_matrix_prepared *p, int matrix,
                                           void *tern_out, void *stream) {
  if (!p) return fail(SUB1_ERR_NULL, "sub1_matrix_prepared_decode: NULL argument");
  if (bad_dims(p->count, p->height, p->width))
    return fail(SUB1_ERR_SHAPE, "sub1_matrix_prepared_decode: %d matrices of %d x %d", p->count,
                p->height, p->width);
  return decode_prepared(from_matrix(p), 0, matrix, tern_out, static_cast<hipStream_t>(stream),
                         "sub1_matrix_prepared_decode");
}
