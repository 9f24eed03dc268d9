/*
 * libsub1_hip - C ABI of the gfx950 (MI355X) implementation of QMoE's
 * compressed-expert operator: dictionary decode fused with matrix-vector
 * product over ternary expert weights coded as 16-bit dictionary indices.
 *
 * The entry points are what a binding for the reference's `sub1_cuda`
 * extension (reference sub1_cuda.cpp:35-59) would call: plain pointers and
 * sizes, no torch types.  All device pointers must belong to the device that
 * is current when the function is called; `stream` is a hipStream_t passed as
 * void* (NULL = the null stream).  Functions return SUB1_OK or a negative
 * status; sub1_last_error() gives the message for the calling thread.  No
 * function synchronises the device unless stated.
 *
 * Data layout (reference sub1.py:114-130, identical here):
 *   dec         int32 [131072]   decode table, entry e = words 2e, 2e+1
 *   trie        int32 [65537*9]  encode trie, root at row 65536
 *   w_comp      int16 [C]        codeword stream, rows back to back
 *   row_off     int32 [H+1]      cumulative codeword count, row_off[0] = 0
 *   ter_minmax  bf16  [2H]       (min, max) of row r at 2r, 2r+1
 *   x           bf16  [W]        activations
 *   y           bf16  [H]        output, ACCUMULATED INTO (y += W x)
 */
#ifndef SUB1_HIP_H_
#define SUB1_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SUB1_OK 0
#define SUB1_ERR_NULL (-1)       /* a required pointer is NULL */
#define SUB1_ERR_SHAPE (-2)      /* height/width/count out of the supported range */
#define SUB1_ERR_ALIGN (-3)      /* a pointer is not aligned for its element type */
#define SUB1_ERR_HIP (-4)        /* a HIP runtime call failed */
#define SUB1_ERR_INTERNAL (-5)

#define SUB1_DICT_ENTRIES 65536              /* reference sub1.py:30 */
#define SUB1_DEC_WORDS (2 * SUB1_DICT_ENTRIES)
#define SUB1_TRIE_ROWS (SUB1_DICT_ENTRIES + 1)
#define SUB1_TRIE_WORDS (9 * SUB1_TRIE_ROWS)
#define SUB1_MAX_WIDTH 12288                 /* sub1_moe_grouped: x is staged in LDS */

/* Message of the last failure on this thread ("" if none). */
const char *sub1_last_error(void);

/* ABI version, bumped on any signature change. */
int sub1_abi_version(void);

/*
 * Name of the kernel that the calling thread's last product or expert-layer
 * entry point launched ("" before the first): the library picks among several
 * by batch size, and a benchmark reports which one it timed.  A launch that
 * was split in two reports the second.
 */
const char *sub1_last_kernel(void);

/*
 * Build the fixed dictionary on the HOST: dec_host[131072], trie_host[65537*9].
 * Either may be NULL.  Replaces the Python `setup()` of reference
 * sub1.py:29-102 (same table bytes).  Deterministic, no GPU needed.
 */
int sub1_build_tables(int32_t *dec_host, int32_t *trie_host);

/*
 * y[r] += bf16( sum_k deq(w[r,k]) * x[k] ),  fp32 accumulation, for any
 * height >= 1 and width >= 1.  Replaces `sub1matvec` (reference
 * sub1_cuda.cpp:35-45, sub1_cuda_kernel.cu:70-88,129-202), which handled six
 * hard-coded shapes and silently did nothing for others.  A wavefront per row;
 * the dictionary entries are read straight from `dec`: nothing is derived,
 * cached or allocated, so the call may be captured in a stream from the first.
 */
int sub1_matvec(const int32_t *dec, const int16_t *w_comp, const int32_t *row_off,
                const void *ter_minmax, const void *x, void *y, int height,
                int width, void *stream);

/*
 * T products with one matrix: y[t, :] += W x[t, :], x row stride `ldx`, y row
 * stride `ldy` (elements).  One launch; what the token loop of reference
 * sub1.py:139-142 does with T launches.
 */
int sub1_matvec_tokens(const int32_t *dec, const int16_t *w_comp,
                       const int32_t *row_off, const void *ter_minmax,
                       const void *x, void *y, int height, int width,
                       int tokens, int64_t ldx, int64_t ldy, void *stream);

/*
 * Encoder, phase 1.  Replaces `Sub1PreparePack` plus the cumulative sum of
 * reference sub1_cuda_kernel.cu:103-112,211-239: greedy longest-match parse
 * of every row of w_tern (int32 [H, W], symbols 0/1/2).  w_tern is
 * OVERWRITTEN with the row's codes (row r's codes at w_tern[r*W ...]) and
 * row_off [H+1] receives the cumulative counts.  The caller then reads
 * row_off[H] (a device-to-host copy, as the reference does at
 * sub1_cuda_kernel.cu:115) to size w_comp.
 */
int sub1_pack_count(const int32_t *trie, int32_t *w_tern, int32_t *row_off,
                    int height, int width, void *stream);

/*
 * Encoder, phase 2.  Replaces `Sub1Pack` (reference
 * sub1_cuda_kernel.cu:241-250): compacts the codes left in w_tern by
 * sub1_pack_count into w_comp[row_off[r] + i].
 */
int sub1_pack_emit(const int32_t *w_tern, const int32_t *row_off, int16_t *w_comp,
                   int height, int width, void *stream);

/*
 * Decoder without the product, for checking: out_tern (uint8 [H, W], symbols)
 * and/or out_w (bf16 [H, W], dequantised weights) may each be NULL.  What the
 * Python `decompress` of reference test.py:103-115 computes.
 * bad_rows (int32 [1], device, may be NULL) is incremented for every row whose
 * codes do not cover exactly the row width.
 */
int sub1_decode(const int32_t *dec, const int16_t *w_comp, const int32_t *row_off,
                const void *ter_minmax, uint8_t *out_tern, void *out_w,
                int32_t *bad_rows, int height, int width, void *stream);

/*
 * One MoE layer's expert FFNs in ONE persistent launch: for every token t
 * with expert e = token_expert[t] >= 0,
 *     y[t] = wo_e( relu( wi_e( x[t] ) ) )      (h is rounded to bf16 between)
 * and y[t] = x[t] for tokens with token_expert[t] < 0 (tokens the router
 * dropped keep their input, reference sub1.py:312).  Replaces the per-expert
 * Python loop of reference sub1.py:315-317 and the two launches per token
 * inside it.  Unlike sub1_matvec, y is OVERWRITTEN.
 *
 * The stack is the experts' Sub1Linear buffers back to back:
 *   w_comp            int16, all streams in one buffer
 *   wi_code_base[e]   int64 [E]  first codeword of expert e's wi stream
 *   wo_code_base[e]   int64 [E]  likewise for wo
 *   wi_row_off        int32 [E, d_ff+1]     each row starts at 0
 *   wo_row_off        int32 [E, d_model+1]
 *   wi_minmax         bf16  [E, 2*d_ff]
 *   wo_minmax         bf16  [E, 2*d_model]
 * workspace: at least sub1_moe_workspace_bytes(tokens, d_ff) bytes of device
 * memory, 256-byte aligned, ZEROED ONCE by the caller before its first use.
 * Its head holds the control words (a fixed part of 192 KB, then 64 bytes per
 * token); h, which may hold anything, is kept in the LAST tokens * d_ff * 2
 * bytes of the workspace_bytes given.  Every launch leaves the control words it
 * counts with at zero again, so a launch is one kernel and the same workspace
 * serves any number of launches of any batch size that fits it, in any order:
 * give every launch the size of the whole buffer as workspace_bytes, not the
 * size that launch needs, so that a small launch's h stays clear of the words
 * a larger one counts with.  Launches that share a workspace must not overlap
 * in time.  Words 1 and 2 (int32) count, over all launches, the waits that gave
 * up and the tokens whose expert id was >= experts (those tokens are passed
 * through like dropped ones).  After a wait fault (sub1_fault_flags) the words
 * may be left at other values than zero (a workgroup that reports after the
 * waiters of its token have given up), and no later launch would notice: once
 * the faulting work has ended, ZERO THE WORKSPACE AGAIN before its next launch.
 * sub1_fault_epoch() counts the wait faults that sub1_clear_faults() has
 * cleared; an owner of workspaces keeps the count it saw when it zeroed each
 * and zeroes again when the count has moved on.
 */
typedef struct sub1_moe_stack {
  const int32_t *dec;
  const int16_t *w_comp;
  const int64_t *wi_code_base;
  const int64_t *wo_code_base;
  const int32_t *wi_row_off;
  const int32_t *wo_row_off;
  const void *wi_minmax;
  const void *wo_minmax;
  int32_t experts;
  int32_t d_model;
  int32_t d_ff;
} sub1_moe_stack;

int64_t sub1_moe_workspace_bytes(int tokens, int d_ff);

int sub1_moe_grouped(const sub1_moe_stack *stack, const int32_t *token_expert,
                     const void *x, void *y, int tokens, void *workspace,
                     int64_t workspace_bytes, void *stream);

/*
 * token_expert from a top-1 router's mask, in one launch: replaces
 * `expert_index = torch.argmax(router_mask, dim=-1)` (reference sub1.py:311)
 * and the test for tokens without an expert (sub1.py:315-318 runs no expert on
 * a token whose mask row is all zero; such a token keeps its input).
 *   mask          [tokens, experts], contiguous, integers of element_bytes
 *                 (8: int64, 4: int32, 1: uint8 / bool)
 *   route[t]      index of the row's first largest element, or -1 where the row
 *                 is all zero: the token_expert of the grouped launches
 *   expert_index  NULL, or int64 [tokens]: the argmax itself (0 for an all-zero
 *                 row), which the reference returns beside the hidden states
 */
int sub1_route_from_mask(const void *mask, int element_bytes, int tokens, int experts,
                         int32_t *route, int64_t *expert_index, void *stream);

/*
 * Prepared stack: the fast form of sub1_moe_grouped (no counterpart in the
 * reference).  Preparing decodes the stack once and stores every row's
 * non-zero weights as a gap-coded stream the GPU walks at full width:
 *
 *   - the kernels keep the activations in LDS by physical column: real column
 *     c is physical column q = c + c/16 + 1, every 17th physical column (0, 17,
 *     34, ...) holds zeros; a physical column is two dwords, (x[c], 0) read for
 *     a row-min weight and (0, x[c]) read for a row-max weight.  A position
 *     p = 2q + symbol - 1 therefore names a weight's column and symbol;
 *   - a row is a sequence of 7-bit entries, each the step from the row's
 *     position (0 at the start) to the next: to the next non-zero weight's
 *     position, or, where that is more than 127 away, to the farthest zero
 *     column within reach (a multiple of 34); after its last non-zero a row
 *     steps to the next multiple of 34 and pads with steps of 0;
 *   - nine entries make a chunk (8 bytes, entry q in bits 7q..7q+6, bit 63
 *     zero); rows are ordered by chunk count and cut into 64-row slices, each
 *     as long as its longest row and at least one chunk; chunk c of lane l of
 *     a slice sits at byte (slice_base * 64 + c * 64 + l) * 8 of `codes`.
 *
 * With 10% non-zero weights this takes 0.72 bit per weight (the dictionary
 * codes: 0.69), and a weight costs the kernel one LDS read and one
 * multiply-add.  Only for the fixed dictionary (dec is compared with it, once)
 * and 1 <= d_model, d_ff <= SUB1_PREPARED_MAX_WIDTH.
 *
 *   meta_bytes = sub1_moe_prepared_meta_bytes(experts, d_model, d_ff);
 *   sub1_moe_prepared p;
 *   sub1_moe_prepare_layout(stack, meta, meta_bytes, &p, stream);   // synchronises; sets p.code_bytes
 *   p.codes = <device buffer of p.code_bytes bytes>;
 *   sub1_moe_prepare_codes(stack, &p, stream);
 *   sub1_moe_grouped_prepared(&p, token_expert, x, y, tokens, workspace, bytes, stream);
 *
 * meta and codes are device buffers the caller owns, 256-byte aligned; the
 * original stack is not referenced after sub1_moe_prepare_codes has run.
 * sub1_moe_grouped_prepared has the semantics of sub1_moe_grouped and the same
 * workspace.  A row's result is the fp32 sum of x[c] * w[r, c] over its
 * non-zero weights, taken in groups of 72 entries (8 chunks): a partial sum
 * per group from zero, the partial sums added first group first; the same bits
 * for every batch size.  With few tokens several wavefronts share a row slice
 * (the buffer carries position checkpoints for that); the results do not
 * change.  A batch with several tokens per expert (at least four per expert
 * and per compute unit on average) is grouped by expert on the GPU, and three
 * or four tokens of an expert walk its streams together; the tables of that
 * grouping live in the workspace; every token's result stays the same to the
 * bit for finite activations (tokens that share a walk share dwords of the
 * activation array: an infinity or NaN of one spoils its partner's sums).
 *
 * sub1_moe_prepared_decode writes the symbols (0, 1 = row min, 2 = row max) of
 * one matrix, read back from the stream, to tern_out (uint8 [rows, width] on
 * the device; projection 0 = wi, 1 = wo): the check that preparing kept every
 * weight.
 */
#define SUB1_PREPARED_MAX_WIDTH 12288

typedef struct sub1_moe_prepared {
  const void *meta;
  const void *codes;
  int64_t meta_bytes;
  int64_t code_bytes;
  int64_t total_chunks;    /* 512-byte chunk rows of the entry stream; checkpoints follow */
  int32_t experts;
  int32_t d_model;
  int32_t d_ff;
  int32_t max_chunks[2];   /* longest 64-row slice of wi, wo in chunks */
} sub1_moe_prepared;

int64_t sub1_moe_prepared_meta_bytes(int experts, int d_model, int d_ff);

int sub1_moe_prepare_layout(const sub1_moe_stack *stack, void *meta, int64_t meta_bytes,
                            sub1_moe_prepared *prepared, void *stream);

int sub1_moe_prepare_codes(const sub1_moe_stack *stack, const sub1_moe_prepared *prepared,
                           void *stream);

/*
 * The same preparation straight from the layers' own buffers, wherever they
 * lie: per projection and buffer a DEVICE array [experts] of device pointers to
 * what expert e's Sub1Linear holds (reference sub1.py:116-130: w_comp int16,
 * row_off int32 [rows + 1] starting at 0, ter_minmax bf16 [2 * rows]; 2-, 4-
 * and 4-byte aligned).  Nothing is stacked first: a layer is loaded into its
 * Sub1Linear buffers as the reference does (sub1.py:284-292) and prepared from
 * there, and the only memory a launch needs afterwards is the prepared pair.
 * Both calls copy the six tables to the host to look at them (they synchronise
 * the stream).  Same results as preparing the stacked copy of these buffers.
 */
typedef struct sub1_moe_layers {
  const int32_t *dec;
  const void *const *wi_w_comp;
  const void *const *wo_w_comp;
  const void *const *wi_row_off;
  const void *const *wo_row_off;
  const void *const *wi_minmax;
  const void *const *wo_minmax;
  int32_t experts;
  int32_t d_model;
  int32_t d_ff;
} sub1_moe_layers;

int sub1_moe_prepare_layout_from_layers(const sub1_moe_layers *layers, void *meta,
                                        int64_t meta_bytes, sub1_moe_prepared *prepared,
                                        void *stream);

int sub1_moe_prepare_codes_from_layers(const sub1_moe_layers *layers,
                                       const sub1_moe_prepared *prepared, void *stream);

/*
 * What the stream spends on padding: *walked = entries a sweep of all experts
 * walks (64 lanes x the length of every slice), *in_rows = entries of the rows
 * themselves (their non-zero weights and the steps over zeros that long gaps
 * need).  Reads two small tables back from meta; synchronises the stream.
 */
int sub1_moe_prepared_entry_counts(const sub1_moe_prepared *prepared, int64_t *walked,
                                   int64_t *in_rows, void *stream);

int sub1_moe_grouped_prepared(const sub1_moe_prepared *prepared, const int32_t *token_expert,
                              const void *x, void *y, int tokens, void *workspace,
                              int64_t workspace_bytes, void *stream);

int sub1_moe_prepared_decode(const sub1_moe_prepared *prepared, int expert, int projection,
                             void *tern_out, void *stream);

/*
 * sub1_moe_grouped_prepared without the workspace argument, for callers that
 * cannot allocate device memory: code under a HIP graph capture, tight serving
 * loops, harnesses that forbid it.  No counterpart in the reference (whose
 * kernels need no scratch memory).  The control words and h live in a static
 * device array of SUB1_STATIC_SCRATCH_BYTES that every GPU the library runs on
 * holds until the process ends; the call allocates nothing, on the device or
 * pinned (so sub1_init() must have run once in the process).  The array is
 * split once and for all: control words for SUB1_STATIC_MAX_TOKENS tokens at
 * its head, h in the rest, so that stacks of different d_ff can take turns on
 * it; a batch of more tokens, or whose h (tokens * d_ff * 2 bytes) is larger
 * than that rest (799 KB: 66 tokens of a Switch-c-2048 layer), is refused.
 * Same kernels and same results as sub1_moe_grouped_prepared.  All calls on
 * one GPU share the one array: two that overlap there (different streams,
 * different threads) race; calls on one stream run in order and are safe.
 * After a wait fault (sub1_fault_flags) the control words may be left at other
 * values than zero: sub1_static_scratch_reset(stream) zeroes them again with one
 * small kernel on `stream` (no allocation, no memset node), once the work that
 * faulted has ended.
 */
#define SUB1_STATIC_SCRATCH_BYTES (1 << 20)
#define SUB1_STATIC_MAX_TOKENS 512

int sub1_moe_grouped_prepared_static(const sub1_moe_prepared *prepared,
                                     const int32_t *token_expert, const void *x, void *y,
                                     int tokens, void *stream);
int sub1_static_scratch_reset(void *stream);
/* The current device's address of that array (its words 1 and 2 count waits
 * that gave up and tokens with an expert id >= experts, as in a workspace). */
int sub1_static_scratch_pointer(void **address);

/*
 * The same preparation for plain products: `count` matrices of one shape
 * (count = 1: one Sub1Linear), then
 *     y[t, :] += W_m x[t, :],   m = token_matrix[t]  (NULL: matrix 0 for all),
 * the semantics of sub1_matvec_tokens, in one launch without a workspace.
 * Without token_matrix and with enough tokens to occupy the GPU that way, the
 * stream is walked once per four tokens (same results to the bit).
 * Tokens whose matrix index is negative or >= count are left alone.
 *
 *   meta_bytes = sub1_matrix_prepared_meta_bytes(count, height, width);
 *   sub1_matrix_prepared p;
 *   sub1_matrix_prepare_layout(&set, meta, meta_bytes, &p, stream);   // synchronises
 *   p.codes = <device buffer of p.code_bytes bytes>;
 *   sub1_matrix_prepare_codes(&set, &p, stream);
 *   sub1_matvec_prepared(&p, NULL, x, ldx, y, ldy, tokens, stream);
 */
typedef struct sub1_matrix_set {
  const int32_t *dec;
  const int16_t *w_comp;       /* all streams in one buffer */
  const int64_t *code_base;    /* int64 [count] first codeword of each matrix; NULL if count == 1 */
  const int32_t *row_off;      /* int32 [count, height+1], each row starts at 0 */
  const void *ter_minmax;      /* bf16  [count, 2*height] */
  int32_t count;
  int32_t height;
  int32_t width;
} sub1_matrix_set;

typedef struct sub1_matrix_prepared {
  const void *meta;
  const void *codes;
  int64_t meta_bytes;
  int64_t code_bytes;
  int64_t total_chunks;
  int32_t count;
  int32_t height;
  int32_t width;
  int32_t max_chunks;
} sub1_matrix_prepared;

int64_t sub1_matrix_prepared_meta_bytes(int count, int height, int width);

int sub1_matrix_prepare_layout(const sub1_matrix_set *set, void *meta, int64_t meta_bytes,
                               sub1_matrix_prepared *prepared, void *stream);

int sub1_matrix_prepare_codes(const sub1_matrix_set *set, const sub1_matrix_prepared *prepared,
                              void *stream);

int sub1_matvec_prepared(const sub1_matrix_prepared *prepared, const int32_t *token_matrix,
                         const void *x, int64_t ldx, void *y, int64_t ldy, int tokens,
                         void *stream);

int sub1_matrix_prepared_decode(const sub1_matrix_prepared *prepared, int matrix,
                                void *tern_out, void *stream);

/*
 * Many tokens through one matrix on the matrix cores (no counterpart in the
 * reference, whose Sub1Linear.forward launches one product per token,
 * sub1.py:137-142): y[t, :] += W_m x[t, :] for all tokens in one launch, the
 * weights turned back into bf16 values in registers and multiplied by MFMA
 * (v_mfma_f32_32x32x16_bf16), 64 rows x 64 tokens per workgroup.  For that the
 * matrices are copied once into a tile form of 2 bits per weight whatever the
 * density (0 = row min, 1 = row max, 2 = zero): units of 32 rows x 128 columns
 * of 1 KB, each laid out as the 64 lanes' shares of the MFMA B operand, so that
 * a wavefront fetches a unit with one 16-byte load per lane and builds the
 * operands with a byte permute of the row's (min, max) word, without a table;
 * rows are padded to 64, columns to 128 (c-2048 wi: 3.4 MB against 1.1 MB of
 * codes).  Worth it from 64 tokens on; below that sub1_matvec_tokens or
 * sub1_matvec_prepared walk the non-zeros per token.  Products are exact and
 * summed in fp32 in the matrix cores' order: results agree with the other
 * kernels to rounding (1e-2 bar), not to the bit.  A zero weight is multiplied
 * like any other (as the reference kernel does, sub1_cuda_kernel.cu:190): an
 * infinite or NaN activation makes every row of its token NaN, where the
 * walking kernels only touch the rows that have a weight in that column.
 *
 *   meta_bytes = sub1_tiles_meta_bytes(count, height, width);
 *   sub1_tiles t;
 *   sub1_tiles_layout(&set, meta, meta_bytes, &t, stream);      // synchronises; sets t.entry_bytes
 *   t.entries = <device buffer of t.entry_bytes bytes>;
 *   sub1_tiles_entries(&set, &t, stream);
 *   sub1_matvec_tiles(&t, matrix, x, ldx, y, ldy, tokens, stream);
 *
 * meta and entries are device buffers the caller owns, 256-byte aligned; the
 * source matrices are not referenced after sub1_tiles_entries has run.  Any
 * dictionary with symbols 0..2; any height and width; up to 65535 * 64 tokens
 * a launch.  x rows are read 16 bytes at a time when x is 16-byte aligned and
 * ldx a multiple of 8 (else element by element, slower).  The windows of 128
 * columns of a matrix are summed in 1, 2 or 4 parts, a number that depends on
 * the matrix's shape alone: a token's result does not depend on the launch it
 * is part of, although long launches take another kernel (workgroups of four
 * wavefronts that share their activations; it also wants y 4-byte aligned, ldy
 * and the height even).  sub1_tiles_decode writes one matrix's symbols, read back
 * from the tile form, to tern_out (uint8 [height, width]): the check that the
 * copy kept every weight.
 */
typedef struct sub1_tiles {
  const void *meta;
  const void *entries;
  int64_t meta_bytes;
  int64_t entry_bytes;
  int64_t total_chunks;    /* 512-byte chunk rows of all segments */
  int32_t count;
  int32_t height;
  int32_t width;
} sub1_tiles;

int64_t sub1_tiles_meta_bytes(int count, int height, int width);

int sub1_tiles_layout(const sub1_matrix_set *set, void *meta, int64_t meta_bytes, sub1_tiles *tiles,
                      void *stream);

int sub1_tiles_entries(const sub1_matrix_set *set, const sub1_tiles *tiles, void *stream);

int sub1_matvec_tiles(const sub1_tiles *tiles, int matrix, const void *x, int64_t ldx, void *y,
                      int64_t ldy, int tokens, void *stream);

/*
 * For tests (no counterpart in the reference): later sub1_matvec_tiles launches
 * take the kernel named here instead of the one estimated faster, where the
 * arguments allow it.  0: by estimate; 1: a wavefront with tiles of its own;
 * 2: workgroups that share their activations, blocks of 64 tokens; 3: the
 * same, blocks of 128 tokens.  The results must not depend on it.
 */
int sub1_test_tiles_kernel(int which);

int sub1_tiles_decode(const sub1_tiles *tiles, int matrix, void *tern_out, void *stream);

/*
 * Average duration in microseconds of the most recent launches, measured with
 * HIP events on the launch stream: call sub1_timing_begin(stream) before and
 * sub1_timing_end(stream, &us) after a run of launches (end synchronises).
 * For benchmarks; not thread safe.
 */
int sub1_timing_begin(void *stream);
int sub1_timing_end(void *stream, double *elapsed_us);

/*
 * Faults that a launch cannot return (no counterpart in the reference, whose
 * kernels do not wait for each other).  The grouped launches let workgroups
 * wait for each other's part of h; every such wait is bounded in TIME (default
 * 250 ms on the device's constant-rate clock, far above any wait of a healthy
 * launch, which lasts microseconds).  A wait that reaches the bound gives up:
 * the kernel carries on and exits normally, its output is wrong, and it sets a
 * sticky flag in pinned host memory that no launch clears.  A second flag is
 * set when a launch finds that `dec` no longer holds what the table cached for
 * its address was derived from (see sub1_unregister_dec).
 *
 *   sub1_init()               allocates the flag words (pinned host memory) and
 *                             prepares the current device; the other entry
 *                             points do this themselves on first use, so it is
 *                             only needed before a stream capture or
 *                             sub1_moe_grouped_prepared_static.  Safe to call
 *                             again; call it once with each device current
 *                             that will use the static scratch.
 *   sub1_fault_flags(f)       f[0] = a wait gave up, f[1] = dec changed; read
 *                             from host memory, no synchronisation: a flag is
 *                             seen once the launch that set it has got that far.
 *   sub1_fault_words_host()   the two flags as int32 words in host memory (NULL
 *                             before sub1_init or a first launch): a caller
 *                             that polls between launches reads them directly.
 *   sub1_clear_faults()       resets both; a wait fault among them moves
 *                             sub1_fault_epoch() on by one.
 *   sub1_fault_epoch()        wait faults cleared so far: every workspace that
 *                             was in use before the count moved must be zeroed
 *                             again before its next launch (and the static
 *                             scratch by sub1_static_scratch_reset).
 *   sub1_set_wait_limit_us(n) the bound, 1 .. 60 000 000 us, for later launches.
 *   sub1_test_overstate_wait(k)  for tests of the above: later launches expect k
 *                             more workgroups in every wait than will ever
 *                             report, so each wait runs into the bound.
 */
int sub1_init(void);
int sub1_fault_flags(int32_t *flags);
const int32_t *sub1_fault_words_host(void);
int sub1_clear_faults(void);
int64_t sub1_fault_epoch(void);
int sub1_set_wait_limit_us(int64_t microseconds);
int sub1_test_overstate_wait(int extra);

/*
 * sub1_moe_grouped keeps the compact table it derives from `dec` by the
 * ADDRESS of dec (per device), and the prepare calls remember that they have
 * compared a dec at that address with the fixed dictionary.  Call this before freeing a dec
 * buffer whose address may be handed out again for other contents; NULL drops
 * every cached table.  Synchronises the device.  (A launch that finds other
 * contents at a cached address sets the flag above and the next call derives
 * the tables afresh.)
 */
int sub1_unregister_dec(const int32_t *dec);

#ifdef __cplusplus
}
#endif
#endif /* SUB1_HIP_H_ */
