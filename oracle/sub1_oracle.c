/*
 * CPU oracle for the QMoE sub-1-bit codec and decode+matvec path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates the reference algorithm on the
 * CPU so that the HIP kernels can be checked against it.  Nothing in the
 * shipped library links or calls it; only the tests, the smoke check and the
 * benchmark's cpu_baseline leg do, as the checker or as the timed CPU figure.
 *
 * Every function names the reference lines it follows (paths are relative to
 * the reference checkout):
 *
 *   sub1o_build_tables   sub1.py:29-102   (dictionary, dec table, encode trie)
 *   sub1o_encode         sub1_cuda_kernel.cu:211-250, test.py:86-100
 *   sub1o_decode         sub1_cuda_kernel.cu:186-192, test.py:103-115
 *   sub1o_dequant        test.py:110, sub1_cuda_kernel.cu:156-157,170-171
 *   sub1o_matvec_lanes   sub1_cuda_kernel.cu:143-201 (lane order, tree, y +=)
 *   sub1o_matvec_seq     same sums, taken per symbol, in groups of 32 codes
 *   sub1o_matvec_wave    same sums, codeword i of a row in lane i mod 64, the 64
 *                        lanes summed by a butterfly (the order of the
 *                        wavefront-per-row kernel behind sub1_matvec)
 *   sub1o_gap_entries    a row's non-zero weights as the 7-bit gap entries of
 *                        the library's prepared stream (no reference lines:
 *                        the format is the library's own; pinned by decoding
 *                        the entries back to the row)
 *   sub1o_matvec_gap     same sums, one fused multiply-add per entry, in
 *                        groups of 72 entries
 *   sub1o_matvec_f64     textbook GEMV in double on the decoded matrix
 *   sub1o_expert_ffn     sub1.py:132-143 twice with ReLU between (the
 *                        DenseActDense call made at sub1.py:317)
 *
 * How each one is pinned is written next to its test in tests/.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define SUB1O_COUNT 65536      /* sub1.py:30 */
#define SUB1O_MAXPAIRS 14      /* sub1.py:54 */
#define SUB1O_ROOT 65536       /* sub1.py:89, sub1_cuda_kernel.cu:209 */

/* ---------------------------------------------------------------- bf16 --- */

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, the rounding of __float2bfloat16 and torch's cast */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* NaN */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

uint16_t sub1o_f32_to_bf16(float f) { return f32_to_bf16(f); }
float sub1o_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* ----------------------------------------------------- dictionary heap --- */

/* One heap item = (negated probability, pair string).  Ordering is that of the
 * Python tuple (float, list) used at sub1.py:49-57: by the float, then by the
 * list lexicographically with a proper prefix sorting first. */
typedef struct {
  double key;
  uint8_t len;
  uint8_t seq[SUB1O_MAXPAIRS];
} item_t;

static int item_less(const item_t *a, const item_t *b) {
  if (a->key < b->key) return 1;
  if (a->key > b->key) return 0;
  int n = a->len < b->len ? a->len : b->len;
  for (int i = 0; i < n; i++) {
    if (a->seq[i] != b->seq[i]) return a->seq[i] < b->seq[i];
  }
  return a->len < b->len;
}

typedef struct {
  item_t *v;
  size_t n, cap;
} heap_t;

static int heap_push(heap_t *h, const item_t *it) {
  if (h->n == h->cap) {
    size_t nc = h->cap ? 2 * h->cap : 1024;
    item_t *nv = (item_t *)realloc(h->v, nc * sizeof(item_t));
    if (!nv) return -1;
    h->v = nv;
    h->cap = nc;
  }
  size_t i = h->n++;
  while (i > 0) {
    size_t p = (i - 1) / 2;
    if (!item_less(it, &h->v[p])) break;
    h->v[i] = h->v[p];
    i = p;
  }
  h->v[i] = *it;
  return 0;
}

static item_t heap_pop(heap_t *h) {
  item_t top = h->v[0];
  item_t last = h->v[--h->n];
  size_t i = 0;
  for (;;) {
    size_t c = 2 * i + 1;
    if (c >= h->n) break;
    if (c + 1 < h->n && item_less(&h->v[c + 1], &h->v[c])) c++;
    if (!item_less(&h->v[c], &last)) break;
    h->v[i] = h->v[c];
    i = c;
  }
  if (h->n) h->v[i] = last;
  return top;
}

/* The 9 pair probabilities of sub1.py:33-44: index r = 3a+b, value
 * (1.0*p[a])*p[b] in IEEE double, p = [.885, (1-.885)/2, (1-.885)/2].
 * volatile stops the compiler from folding with a different association. */
static void pair_probs(double out[9]) {
  volatile double zeros = .885;
  volatile double one = 1.;
  double p[3];
  p[0] = zeros;
  p[1] = (one - zeros) / 2;
  p[2] = (one - zeros) / 2;
  for (int a = 0; a < 3; a++)
    for (int b = 0; b < 3; b++) {
      volatile double first = one * p[a];
      out[3 * a + b] = first * p[b];
    }
}

/* Dictionary entries in index order, each a string of pair symbols 0..8.
 * Best-first expansion, sub1.py:49-57. */
static int build_entries(item_t *res) {
  double probs[9];
  pair_probs(probs);
  heap_t h = {0, 0, 0};
  item_t root;
  memset(&root, 0, sizeof root);
  root.key = -1.;
  if (heap_push(&h, &root)) return -1;
  int count = 0;
  while (count < SUB1O_COUNT) {
    if (h.n == 0) { free(h.v); return -2; }
    item_t top = heap_pop(&h);
    if (top.key != -1.) res[count++] = top;
    if (top.len == SUB1O_MAXPAIRS) continue;
    for (int i = 0; i < 9; i++) {
      item_t ch = top;
      volatile double k = top.key * probs[i];
      ch.key = k;
      ch.seq[ch.len++] = (uint8_t)i;
      if (heap_push(&h, &ch)) { free(h.v); return -1; }
    }
  }
  free(h.v);
  return 0;
}

/* dec[2i], dec[2i+1]: pairs 0-6 / 7-13 of entry i, pair j at bits 4+4j..7+4j
 * (low 2 bits r%3 = even-position weight, high 2 bits r/3 = odd-position
 * weight), bits 0-3 of both words = pair count.  sub1.py:60-72.
 * trie[9*node+sym] = child entry or -1, root at row 65536.  sub1.py:74-97. */
int sub1o_build_tables(int32_t *dec, int32_t *trie) {
  item_t *res = (item_t *)malloc(SUB1O_COUNT * sizeof(item_t));
  if (!res) return -1;
  int rc = build_entries(res);
  if (rc) { free(res); return rc; }

  if (dec) {
    for (int i = 0; i < SUB1O_COUNT; i++) {
      uint32_t w[2] = {0, 0};
      for (int j = 0; j < res[i].len; j++) {
        uint32_t r = res[i].seq[j];
        int half = j / 7, slot = j % 7;
        w[half] |= (r % 3) << (4 * slot + 0);
        w[half] |= (r / 3) << (4 * slot + 2);
      }
      dec[2 * i + 0] = (int32_t)((w[0] << 4) | res[i].len);
      dec[2 * i + 1] = (int32_t)((w[1] << 4) | res[i].len);
    }
  }

  if (trie) {
    for (long i = 0; i < (long)(SUB1O_COUNT + 1) * 9; i++) trie[i] = -1;
    /* An entry's parent (the string minus its last pair) has a strictly
     * smaller key, so it sits at a smaller index; walk from the root. */
    for (int i = 0; i < SUB1O_COUNT; i++) {
      int node = SUB1O_ROOT;
      for (int j = 0; j + 1 < res[i].len; j++) {
        node = trie[9 * node + res[i].seq[j]];
        if (node < 0) { free(res); return -3; } /* not prefix closed */
      }
      trie[9 * node + res[i].seq[res[i].len - 1]] = i;
    }
  }
  free(res);
  return 0;
}

/* Entry strings themselves, for tests: out[i*15] = length, then the pairs. */
int sub1o_dictionary_entries(uint8_t *out, double *keys) {
  item_t *res = (item_t *)malloc(SUB1O_COUNT * sizeof(item_t));
  if (!res) return -1;
  int rc = build_entries(res);
  if (!rc) {
    for (int i = 0; i < SUB1O_COUNT; i++) {
      out[15 * i] = res[i].len;
      memset(out + 15 * i + 1, 0, 14);
      memcpy(out + 15 * i + 1, res[i].seq, res[i].len);
      if (keys) keys[i] = res[i].key;
    }
  }
  free(res);
  return rc;
}

/* -------------------------------------------------------------- encode --- */

/* Greedy longest-match parse of each row, sub1_cuda_kernel.cu:217-238: pair
 * symbol = 3*w[i+1] + w[i] (the odd tail keeps only w[i]); when the current
 * node has no child for the symbol the node is emitted and the walk restarts
 * at the root; the node reached at the row end is emitted too.  row_off is
 * cumulative in codewords (sub1_cuda_kernel.cu:112), codes never span rows,
 * and the stream is the rows' codes back to back (sub1_cuda_kernel.cu:247-249).
 * Returns the codeword count, or -1 if it exceeds cap (row_off is still
 * filled so the caller can size the buffer). */
int64_t sub1o_encode(const int32_t *trie, const int32_t *w_tern, int height,
                     int width, uint16_t *codes, int64_t cap, int32_t *row_off) {
  int64_t n = 0;
  int overflow = 0;
  row_off[0] = 0;
  for (int r = 0; r < height; r++) {
    const int32_t *w = w_tern + (int64_t)r * width;
    int node = SUB1O_ROOT;
    for (int i = 0; i < width; i += 2) {
      int num = 0;
      for (int j = 1; j >= 0; j--)
        if (i + j < width) num = 3 * num + w[i + j];
      if (trie[9 * node + num] == -1) {
        if (n < cap) codes[n] = (uint16_t)node; else overflow = 1;
        n++;
        node = SUB1O_ROOT;
      }
      node = trie[9 * node + num];
    }
    if (n < cap) codes[n] = (uint16_t)node; else overflow = 1;
    n++;
    row_off[r + 1] = (int32_t)n;
  }
  return overflow ? -1 : n;
}

/* -------------------------------------------------------------- decode --- */

/* Ternary digit d (0..27) of entry e, the extraction at
 * sub1_cuda_kernel.cu:153-154,188-189. */
static inline int entry_digit(const int32_t *dec, int e, int d) {
  uint32_t w = (uint32_t)dec[2 * e + d / 14];
  return (int)((w >> (4 + 2 * (d % 14))) & 3u);
}

/* Symbols 0/1/2 of every weight.  Column position advances by two per pair
 * (sub1_cuda_kernel.cu:192); digits that fall beyond the row width are
 * dropped (test.py:111-113).  Returns 0, or 1+row of the first row whose
 * codes do not cover exactly ceil(width/2) pairs. */
int sub1o_decode(const int32_t *dec, const uint16_t *codes, const int32_t *row_off,
                 int height, int width, uint8_t *tern) {
  for (int r = 0; r < height; r++) {
    uint8_t *t = tern + (int64_t)r * width;
    int idx = 0;
    for (int c = row_off[r]; c < row_off[r + 1]; c++) {
      int e = codes[c];
      int npairs = dec[2 * e] & 0xf;
      for (int d = 0; d < 2 * npairs; d++)
        if (idx + d < width) t[idx + d] = (uint8_t)entry_digit(dec, e, d);
      idx += 2 * npairs;
    }
    if (idx != ((width + 1) & ~1)) return 1 + r;
  }
  return 0;
}

/* Symbol -> bf16 weight: 0 -> 0, 1 -> ter_minmax[2r], 2 -> ter_minmax[2r+1]. */
void sub1o_dequant(const uint8_t *tern, const uint16_t *ter_minmax, int height,
                   int width, uint16_t *w_bf16) {
  for (int r = 0; r < height; r++)
    for (int k = 0; k < width; k++) {
      int s = tern[(int64_t)r * width + k];
      w_bf16[(int64_t)r * width + k] = s == 0 ? 0 : ter_minmax[2 * r + (s - 1)];
    }
}

/* -------------------------------------------------------------- matvec --- */

/* The reference kernel's arithmetic, sub1_cuda_kernel.cu:174-200: lane l of 28
 * accumulates in fp32, with a fused multiply-add, the weight at in-codeword
 * offset l of every codeword of the row times x at that column (columns past
 * the width read the zero pad); the 32 lanes (28..31 hold zero) are summed by
 * the 16/8/4/2/1 shuffle-down tree; the row result is rounded to bf16 and
 * added onto y in bf16. */
void sub1o_matvec_lanes(const int32_t *dec, const uint16_t *codes,
                        const int32_t *row_off, const uint16_t *ter_minmax,
                        const uint16_t *x, uint16_t *y, int height, int width) {
  float *xs = (float *)calloc((size_t)width + 28, sizeof(float));
  for (int k = 0; k < width; k++) xs[k] = bf16_to_f32(x[k]);
  for (int r = 0; r < height; r++) {
    float deq[3];
    deq[0] = 0.f;
    deq[1] = bf16_to_f32(ter_minmax[2 * r]);
    deq[2] = bf16_to_f32(ter_minmax[2 * r + 1]);
    float lane[32];
    for (int l = 0; l < 32; l++) lane[l] = 0.f;
    int idx = 0;
    for (int c = row_off[r]; c < row_off[r + 1]; c++) {
      int e = codes[c];
      for (int l = 0; l < 28; l++) {
        /* columns >= width + 28 cannot be reached: idx <= width + 1 - 2 */
        lane[l] = fmaf(deq[entry_digit(dec, e, l)], xs[idx + l], lane[l]);
      }
      idx += 2 * (dec[2 * e] & 0xf);
    }
    for (int s = 16; s > 0; s /= 2)
      for (int l = 0; l + s < 32; l++) lane[l] += lane[l + s];
    float acc = bf16_to_f32(y[r]) + bf16_to_f32(f32_to_bf16(lane[0]));
    y[r] = f32_to_bf16(acc);
  }
  free(xs);
}

/* Same product in the order the HIP kernels add: s1 = sum of x over the weights
 * with symbol 1, s2 likewise for symbol 2, both in fp32.  A row's codes are
 * taken in groups of SUB1O_GROUP consecutive codes; within a group the
 * activations are added left to right onto a partial sum that starts at zero,
 * and the partial sums are added, first group first, onto the row's sum.  Then
 * res = fma(min, s1, max*s2), bf16, +=.  A second fp32 ordering of the same
 * sum as sub1o_matvec_lanes. */
#define SUB1O_GROUP 32

void sub1o_matvec_seq(const int32_t *dec, const uint16_t *codes,
                      const int32_t *row_off, const uint16_t *ter_minmax,
                      const uint16_t *x, uint16_t *y, int height, int width) {
  for (int r = 0; r < height; r++) {
    float s[3] = {0.f, 0.f, 0.f};
    int idx = 0;
    for (int c0 = row_off[r]; c0 < row_off[r + 1]; c0 += SUB1O_GROUP) {
      float p[3] = {0.f, 0.f, 0.f};
      int c1 = c0 + SUB1O_GROUP < row_off[r + 1] ? c0 + SUB1O_GROUP : row_off[r + 1];
      for (int c = c0; c < c1; c++) {
        int e = codes[c];
        int n = 2 * (dec[2 * e] & 0xf);
        for (int d = 0; d < n && idx + d < width; d++) {
          int t = entry_digit(dec, e, d);
          if (t) p[t] += bf16_to_f32(x[idx + d]);
        }
        idx += n;
      }
      s[1] += p[1];
      s[2] += p[2];
    }
    float res = fmaf(bf16_to_f32(ter_minmax[2 * r]), s[1],
                     bf16_to_f32(ter_minmax[2 * r + 1]) * s[2]);
    float acc = bf16_to_f32(y[r]) + bf16_to_f32(f32_to_bf16(res));
    y[r] = f32_to_bf16(acc);
  }
}

/* Same product in the order of the library's wavefront-per-row kernel: codeword
 * i of a row belongs to lane i mod 64; a lane adds, for its codewords in turn
 * and their non-zero digits left to right, x * (row min | row max) with one
 * fused multiply-add onto its own fp32 sum; the 64 lane sums are then combined
 * by a butterfly, lane l taking l + (l ^ m) for m = 1, 2, 4, 8, 16, 32 (both
 * partners compute the same sum: fp32 addition commutes); bf16; +=.  A third
 * fp32 ordering of the sum of sub1o_matvec_lanes. */
void sub1o_matvec_wave(const int32_t *dec, const uint16_t *codes,
                       const int32_t *row_off, const uint16_t *ter_minmax,
                       const uint16_t *x, uint16_t *y, int height, int width) {
  for (int r = 0; r < height; r++) {
    float deq[3] = {0.f, bf16_to_f32(ter_minmax[2 * r]), bf16_to_f32(ter_minmax[2 * r + 1])};
    float lane[64], next[64];
    for (int l = 0; l < 64; l++) lane[l] = 0.f;
    int idx = 0;
    for (int c = row_off[r]; c < row_off[r + 1]; c++) {
      int e = codes[c];
      int l = (c - row_off[r]) & 63;
      int n = 2 * (dec[2 * e] & 0xf);
      for (int d = 0; d < n && idx + d < width; d++) {
        int t = entry_digit(dec, e, d);
        if (t) lane[l] = fmaf(bf16_to_f32(x[idx + d]), deq[t], lane[l]);
      }
      idx += n;
    }
    for (int m = 1; m < 64; m *= 2) {
      for (int l = 0; l < 64; l++) next[l] = lane[l] + lane[l ^ m];
      memcpy(lane, next, sizeof lane);
    }
    float acc = bf16_to_f32(y[r]) + bf16_to_f32(f32_to_bf16(lane[0]));
    y[r] = f32_to_bf16(acc);
  }
}

/* The prepared stream's view of a row.  Activations are laid out by physical
 * column: real column c is physical column q = c + c/16 + 1, every 17th
 * physical column (0, 17, 34, ...) is a zero column.  A position p = 2q + s - 1
 * names the column and the symbol (1 = row min, 2 = row max) of a weight; the
 * positions 34k and 34k+1 are zeros.  The row is the sequence of steps (0..127)
 * that visits its non-zero weights in column order, starting from 0: a step to
 * a non-zero more than 127 away first goes to the farthest zero column within
 * reach (the largest multiple of 34 not beyond p+127), repeatedly; after the
 * last non-zero one step goes to the next multiple of 34.  Writes the steps to
 * out (if not NULL; at most cap) and returns their number, or -1 if the codes
 * do not cover ceil(width/2) pairs. */
#define SUB1O_GAP_MAX 127
#define SUB1O_GAP_ZERO 17

static int gap_position(int col, int sym) { return 2 * (col + col / 16 + 1) + sym - 1; }

int sub1o_gap_entries(const int32_t *dec, const uint16_t *codes, int ncodes,
                      int width, uint8_t *out, int cap) {
  const int period = 2 * SUB1O_GAP_ZERO;
  int n = 0, j = 0, idx = 0;
  for (int c = 0; c < ncodes; c++) {
    int e = codes[c];
    int npairs = dec[2 * e] & 0xf;
    for (int d = 0; d < 2 * npairs && idx + d < width; d++) {
      int t = entry_digit(dec, e, d);
      if (!t) continue;
      int target = gap_position(idx + d, t);
      while (target - j > SUB1O_GAP_MAX) {
        int z = (j + SUB1O_GAP_MAX) / period * period;
        if (out && n < cap) out[n] = (uint8_t)(z - j);
        n++;
        j = z;
      }
      if (out && n < cap) out[n] = (uint8_t)(target - j);
      n++;
      j = target;
    }
    idx += 2 * npairs;
  }
  if (idx != ((width + 1) & ~1)) return -1;
  if ((j / 2) % SUB1O_GAP_ZERO) {
    int z = (j + period - 1) / period * period;
    if (out && n < cap) out[n] = (uint8_t)(z - j);
    n++;
  }
  return n;
}

/* The product in the order the prepared-stream kernels add: the row's entries
 * in groups of SUB1O_GAP_GROUP; within a group each entry that stands on an
 * activation adds x * w (w = row min or max) with one fused multiply-add onto a
 * partial sum that starts at zero (entries on a zero column add nothing); the
 * partial sums are added, first group first, onto the row's sum; bf16; +=. */
#define SUB1O_GAP_GROUP 72

int sub1o_matvec_gap(const int32_t *dec, const uint16_t *codes,
                     const int32_t *row_off, const uint16_t *ter_minmax,
                     const uint16_t *x, uint16_t *y, int height, int width) {
  int cap = width + width / 40 + 8;
  uint8_t *steps = (uint8_t *)malloc((size_t)cap);
  for (int r = 0; r < height; r++) {
    int n = sub1o_gap_entries(dec, codes + row_off[r], row_off[r + 1] - row_off[r],
                              width, steps, cap);
    if (n < 0 || n > cap) {
      free(steps);
      return 1 + r;
    }
    float w[2] = {bf16_to_f32(ter_minmax[2 * r]), bf16_to_f32(ter_minmax[2 * r + 1])};
    float sum = 0.f;
    int j = 0;
    for (int i0 = 0; i0 < n; i0 += SUB1O_GAP_GROUP) {
      float p = 0.f;
      int i1 = i0 + SUB1O_GAP_GROUP < n ? i0 + SUB1O_GAP_GROUP : n;
      for (int i = i0; i < i1; i++) {
        j += steps[i];
        int q = j / 2;
        if (q % SUB1O_GAP_ZERO) p = fmaf(bf16_to_f32(x[q - 1 - q / SUB1O_GAP_ZERO]), w[j & 1], p);
      }
      sum += p;
    }
    float acc = bf16_to_f32(y[r]) + bf16_to_f32(f32_to_bf16(sum));
    y[r] = f32_to_bf16(acc);
  }
  free(steps);
  return 0;
}

/* Dense double-precision product of the decoded matrix with x, and the sum of
 * |w*x| per row that bounds any fp32 summation order's error. */
void sub1o_matvec_f64(const uint8_t *tern, const uint16_t *ter_minmax,
                      const uint16_t *x, double *y, double *yabs, int height,
                      int width) {
  for (int r = 0; r < height; r++) {
    double deq[3] = {0., (double)bf16_to_f32(ter_minmax[2 * r]),
                     (double)bf16_to_f32(ter_minmax[2 * r + 1])};
    double acc = 0., aacc = 0.;
    for (int k = 0; k < width; k++) {
      double p = deq[tern[(int64_t)r * width + k]] * (double)bf16_to_f32(x[k]);
      acc += p;
      aacc += fabs(p);
    }
    y[r] = acc;
    if (yabs) yabs[r] = aacc;
  }
}

/* One expert FFN on one token as the model runs it (sub1.py:317 calls
 * wo(relu(wi(x))), each projection through sub1.py:132-143: zeroed bf16
 * output, one matvec).  h is bf16 between the stages.  order: 0 = lane order,
 * 1 = per-symbol stream order, 2 = prepared-stream order, 3 = wavefront-per-row
 * order.  h_out may be NULL. */
void sub1o_expert_ffn(const int32_t *dec,
                      const uint16_t *wi_codes, const int32_t *wi_row_off,
                      const uint16_t *wi_minmax,
                      const uint16_t *wo_codes, const int32_t *wo_row_off,
                      const uint16_t *wo_minmax,
                      const uint16_t *x, uint16_t *y, uint16_t *h_out,
                      int d_model, int d_ff, int order) {
  uint16_t *h = (uint16_t *)calloc((size_t)d_ff, sizeof(uint16_t));
  if (order == 0)
    sub1o_matvec_lanes(dec, wi_codes, wi_row_off, wi_minmax, x, h, d_ff, d_model);
  else if (order == 1)
    sub1o_matvec_seq(dec, wi_codes, wi_row_off, wi_minmax, x, h, d_ff, d_model);
  else if (order == 3)
    sub1o_matvec_wave(dec, wi_codes, wi_row_off, wi_minmax, x, h, d_ff, d_model);
  else
    sub1o_matvec_gap(dec, wi_codes, wi_row_off, wi_minmax, x, h, d_ff, d_model);
  for (int i = 0; i < d_ff; i++)
    if (h[i] & 0x8000u) h[i] = 0; /* relu; -0 -> +0 as max(x,0) gives */
  if (h_out) memcpy(h_out, h, (size_t)d_ff * sizeof(uint16_t));
  memset(y, 0, (size_t)d_model * sizeof(uint16_t));
  if (order == 0)
    sub1o_matvec_lanes(dec, wo_codes, wo_row_off, wo_minmax, h, y, d_model, d_ff);
  else if (order == 1)
    sub1o_matvec_seq(dec, wo_codes, wo_row_off, wo_minmax, h, y, d_model, d_ff);
  else if (order == 3)
    sub1o_matvec_wave(dec, wo_codes, wo_row_off, wo_minmax, h, y, d_model, d_ff);
  else
    sub1o_matvec_gap(dec, wo_codes, wo_row_off, wo_minmax, h, y, d_model, d_ff);
  free(h);
}
