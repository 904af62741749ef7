/*
 * georefine_amd -- C ABI of the MI355X (gfx950) decode path for GeoRefine's
 * lossless BF16 context codec.
 *
 * Two shared libraries implement this header:
 *
 *   libgeorefine_codec.so   host C++ (no GPU needed): the functions the reference
 *                           binds with ctypes, same names and argument meaning.
 *   libgeorefine_hip.so     device entry points.  The reference launches Triton
 *                           kernels from Python for these steps, so each entry
 *                           point cites the Python/Triton interface it replaces.
 *
 * Conventions: every function returns 0 on success and a small positive
 * category code otherwise; nothing throws across the boundary.  Host functions
 * own nothing but the encoder outputs, which are released with bcx_free /
 * p_free.  Device functions take raw device pointers and a hipStream_t passed
 * as void*, allocate nothing, never synchronise, and report data errors by
 * OR-ing bits into a caller-provided device int32 (GRF_ERR_*), never by
 * trapping.  All paths below are relative to the reference tree,
 * GCR = context-runtime/georefine_context_runtime.
 */
#ifndef GEOREFINE_AMD_H
#define GEOREFINE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ host codec */

/* GCR/bitexact_context_ans.cpp:235  count, normalise and rANS-encode one symbol stream.
 * kind 0: 10-bit main symbols, context (row class, column class); kind 1: 6-bit
 * residuals, context = main symbol.  freq: caller buffer [nctx*vocab]. */
int bcx_encode(const uint16_t *w, uint64_t n, uint32_t rows, uint32_t cols, const uint8_t *rc,
               const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind, uint32_t *freq, uint8_t **stream,
               size_t *stream_n);
/* GCR/bitexact_context_ans.cpp:267  tables only */
int bcx_frequencies(const uint16_t *w, uint64_t n, uint32_t rows, uint32_t cols, const uint8_t *rc,
                    const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind, uint32_t *freq);
/* GCR/bitexact_context_ans.cpp:291 and :309  (1 bad arguments, 2 invalid stream/tables, 3 internal) */
int bcx_decode(const uint8_t *stream, size_t stream_n, uint64_t n, uint32_t rows, uint32_t cols,
               const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
               const uint16_t *resctx, const uint32_t *freq, uint16_t *out);
int bcx_decode_compact(const uint8_t *stream, size_t stream_n, uint64_t n, uint32_t rows, uint32_t cols,
                       const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                       const uint16_t *resctx, const uint32_t *freq, uint16_t *out);
/* GCR/bitexact_context_ans.cpp:327 */
void bcx_free(void *p);
/* GCR/bitexact_context_ans.cpp:328 and :346  6-bit residuals, MSB first, zero padding */
int bcx_pack6(const uint16_t *w, uint64_t n, uint8_t **out, size_t *bytes);
int bcx_unpack6(const uint8_t *in, size_t bytes, uint64_t n, uint16_t *out);
/* GCR/bitexact_context_gpu_index.cpp:21  frame-index builder: (state, byte offset) before
 * every stride-th symbol; outputs written only on success; codes 1..6 */
int bcx_checkpoint(const uint8_t *stream, size_t stream_bytes, uint64_t n, uint32_t rows, uint32_t cols,
                   const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                   const uint16_t *resctx, const uint32_t *freq, uint32_t stride, uint32_t *states,
                   uint32_t *offsets, uint16_t *out);
/* Symbol pair -> BF16 word, the inverse of the split at GCR/bitexact_context_ans.cpp:9-12
 * (the reference does this step in numpy, GCR/bitexact_context_codec.py:426). 2 = symbol out of range. */
int grf_bctx_join(const uint16_t *main_sym, const uint16_t *res_sym, uint64_t n, uint16_t *out);
/* GCR/bitexact_predictive_ans.cpp:10-12  generic context coder of the predictive frames */
int p_encode(const uint16_t *v, const uint16_t *cx, uint64_t n, uint32_t nc, uint32_t vocab, uint32_t **freq,
             uint8_t **stream, size_t *stream_n);
int p_decode(const uint8_t *st, size_t bytes, uint64_t n, const uint16_t *cx, uint32_t nc, uint32_t vocab,
             const uint32_t *freq, uint16_t *out);
void p_free(void *p);
/* GCR/bitexact_predictive_gpu_index.cpp:9 and :38 */
int ppcx_checkpoint(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx, uint32_t nctx,
                    uint32_t vocab, const uint32_t *freq, uint32_t stride, uint32_t *states, uint32_t *offsets,
                    uint16_t *symbols);
int ppcx_checkpoint_binary(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx, uint32_t nctx,
                           uint32_t vocab, const uint32_t *freq, uint32_t stride, uint32_t *states,
                           uint32_t *offsets, uint16_t *symbols);

/* ------------------------------------------------------------------ device side */

/* bits OR-ed into the caller's device error word */
#define GRF_ERR_SYMBOL 1      /* slot maps to no symbol / zero frequency / dead context */
#define GRF_ERR_OVERRUN 2     /* decoder wanted bytes past the end of a stream */
#define GRF_ERR_UNDERFLOW 4   /* state still below 2^23 after two refill bytes */
#define GRF_ERR_CHECKPOINT 8  /* segment did not end on the next checkpoint */

/* return codes of the launch functions */
#define GRF_OK 0
#define GRF_BAD_ARGUMENT 1
#define GRF_UNSUPPORTED 2
#define GRF_LAUNCH_FAILED 3

/* One entropy-coded symbol stream resident in device memory, with its
 * checkpoint index and the lookup tables derived from its frequency rows.
 *   cum     u32 [nctx][vocab+1]  inclusive prefix sums (cum[c][0] = 0)
 *   bucket  u32 [nctx][256]      lo | hi<<16: first and last symbol whose slot
 *                                range meets slots [b<<8, (b<<8)+255]
 *   states / offsets  u32 [ceil(n/stride)]  decoder state and byte position
 *                                before symbol k*stride */
typedef struct grf_stream {
  const uint8_t *bytes;
  uint32_t n_bytes;
  uint32_t vocab;
  uint32_t nctx;
  const uint32_t *cum;
  const uint32_t *bucket;
  const uint32_t *states;
  const uint32_t *offsets;
} grf_stream;

/* A BCTX frame as the decode kernels see it (the buffers CudaContextTensor keeps,
 * GCR/bitexact_context_gpu.py:96-125). mode 0: residual.bytes is the packed 6-bit
 * stream and the other residual fields are unused; mode 128: residual is a full stream.
 * raw6_segment (mode 0): 0 when the 6-bit fields are in the frame's own order (element e at
 * bit 6 e); S > 0 when the 12-byte groups of 16 fields are kept in the order the fused
 * kernels read them for segments of S symbols: raw6_block_rows and raw6_row_pos are then
 * grf_bctx_fused.raw_interleaved and grf_bctx_fused.row_pos of the same tensor. */
typedef struct grf_bctx_frame {
  grf_stream main;
  grf_stream residual;
  const uint8_t *row_class;
  const uint8_t *col_class;
  const uint32_t *raw6_row_pos;
  uint32_t rows, cols;
  uint32_t nc;
  uint32_t mode;
  uint32_t stride;
  uint32_t raw6_segment;
  uint32_t raw6_block_rows;
} grf_bctx_frame;

/* Replaces the Triton launch of decode_words (GCR/bitexact_context_gpu.py:149-150,
 * kernel GCR/bitexact_context_gpu_kernels.py:114-169).  Decodes `count` checkpointed
 * segments; segment j of the launch is block_ids[j] (device int64) or j itself when
 * block_ids is NULL.  out holds count*stride words: out[j*stride + t]. */
int grf_bctx_decode(const grf_bctx_frame *frame, const int64_t *block_ids, uint32_t count, uint16_t *out,
                    int32_t *error, void *hip_stream);

/* A PPCX frame (the buffers CudaPredictiveTensor keeps, GCR/bitexact_predictive_gpu.py:116-132).
 * mode 0: residual.bytes is the packed 5-bit stream; mode 1: residual is a full stream. */
typedef struct grf_ppcx_frame {
  grf_stream main;
  grf_stream residual;
  const uint8_t *labels;
  const uint8_t *flips;
  const uint16_t *thresholds; /* 15 monotone ordinal keys */
  uint32_t rows, cols;
  uint32_t mode;
  uint32_t stride;
  /* mode 0 only: the order of the packed 5-bit fields.  raw5_segment == 0: the frame's own
   * order.  Otherwise the blocked order grf_ppcx_fused describes (records of 32 fields, segments
   * of raw5_segment symbols, blocks of raw5_block_rows rows at the positions raw5_row_pos gives,
   * NULL = the row itself), so that one resident array serves this kernel and the tile walker. */
  const uint32_t *raw5_row_pos;
  uint32_t raw5_segment, raw5_block_rows;
} grf_ppcx_frame;

/* Replaces the Triton launch of the predictive decode_words
 * (GCR/bitexact_predictive_gpu.py:172, kernel GCR/bitexact_predictive_gpu_kernels.py:24-58).
 * reference: device BF16 words [rows*cols]; out: ceil(n/stride)*stride words. */
int grf_ppcx_decode(const grf_ppcx_frame *frame, const uint16_t *reference, uint16_t *out, int32_t *error,
                    void *hip_stream);

/* Replaces the CUDA branch of predict() (GCR/bitexact_predictive_mix.py:91-102):
 * out = high16( fl32(fl32(up*c0) + fl32(gate*c1)) + c2 ) with separate IEEE operations.
 * coeff: BF16 [rows][3].  Sets GRF_ERR_SYMBOL in *error when any input, coefficient or
 * result is not finite. */
int grf_mix_predict(const uint16_t *up, const uint16_t *gate, const uint16_t *coeff, uint16_t *out,
                    uint32_t rows, uint32_t cols, int32_t *error, void *hip_stream);

/* A BCTX frame prepared for the fused kernels: main rANS stream as in the frame,
 * residuals in the packed 6-bit form, segments of a length that divides the row
 * length, and per-row-class lookup tables laid out for LDS:
 *   seg_state / seg_offset  the checkpoint index: rANS state and stream offset at the start
 *                           of every segment.  With raw_interleaved == 0: u32
 *                           [rows*segs_per_row + 1] in the frame's order; the extra last
 *                           entry is (2^23, main_n_bytes).  With raw_interleaved == B: in
 *                           the blocked order of the residuals (below)
 *   lut         u8  [nr][nc << lognb]        lognb = 16 - shift; sparse index of a
 *                                            symbol with slots in the bucket (best: the
 *                                            one owning most of them)
 *   tab         u64 [nr][nc][tabn+1]         entry(cc, sparse): low32 = start |
 *                                            (freq & 0xFFFF)<<16 (0 stands for 65536),
 *                                            high32 = symbol<<5; unused entries: 0
 *   col_class   u8  [cols]
 * raw_interleaved: 0 = raw6 in the frame's order (the 12-byte group g of row r at
 * (r * cols / 16 + g) * 12); B = 1, 2, 4, 8 or 16 = in blocks of B rows, and inside a block
 * by position in the segment first, then by segment, then by row: with q the row's position
 * (row_pos[r], or r itself when row_pos is null) and G = seg_len / 16, group t of segment s
 * lies at (((q / B * G + t) * segs_per_row + s) * B + q % B) * 12.  The lanes of a wave unit
 * of the GEMV (B = 64 / lanes_per_row rows, at the same position of neighbouring segments)
 * then read one run of 768 bytes per visit, and every 128-byte line is used in a single visit.
 * The index arrays follow the same order: every row holds segs_per_row + 1 entries (the last
 * one the end of its last segment: the start of the next row's first in the frame's order, or
 * (2^23, main_n_bytes)), and entry s of the row at position q lies at
 * ((q / B) * (segs_per_row + 1) + s) * B + q % B, so that the B rows of a unit find their
 * checkpoints side by side; the arrays hold (rows held) * (segs_per_row + 1) entries, and
 * entries of positions no row has are never read.
 * row_pos: u32 [rows], a one-to-one map of the rows to positions below
 * ceil(max position / B) * B (the array holds that many rows; positions no row has are never
 * read).  The host side orders the rows by row class, as the tilings do, and starts every
 * class on a multiple of 16, so that the rows of a unit are the rows of a block.
 * whole_range: nonzero if some context is a single symbol of frequency 65536 (entry field 0,
 * the state does not change there); 0 promises there is none, and the scan for lanes whose
 * lookup byte names a neighbour of their symbol then leaves that case out.
 * main_bytes must be readable for 16 bytes past main_n_bytes (the kernels copy it in
 * 16-byte units).  raw6 is 4-byte aligned; with seg_len 64 and 16-byte alignment the slab
 * kernels read a segment's 48 residual bytes once, as it starts, instead of 12 at a time. */
typedef struct grf_bctx_fused {
  const uint8_t *main_bytes;
  const uint8_t *raw6;
  const uint32_t *seg_state;
  const uint32_t *seg_offset;
  const uint8_t *lut;
  const uint64_t *tab;
  const uint8_t *col_class;
  const uint32_t *row_pos;
  uint32_t main_n_bytes;
  uint32_t rows, cols;
  uint32_t nr, nc;
  uint32_t seg_len, segs_per_row;
  uint32_t shift, lognb, tabn;
  uint32_t raw_interleaved;
  uint32_t whole_range;
} grf_bctx_fused;

/* How a launch cuts the frame into workgroups.  A tile is up to rows_per_tile rows of
 * one row class; threads is a multiple of 64, at most 1024.
 *   tile_rows   u32 [n_tiles*rows_per_tile]  row of each slot, 0xFFFFFFFF = empty
 *   tile_class  u8  [n_tiles]                row class shared by the tile's rows
 *   piece_cap   LDS bytes reserved per row piece of one slab (multiple of 16): at least the
 *               longest span from the 16-byte aligned start of a piece's first segment to
 *               the end of its last one, plus 8 (the refill reads an aligned 8-byte window)
 *   scheme      GRF_TILE_SLABS: lane (r, p) of the workgroup walks segment b*lanes_per_row + p
 *               of the tile's row r in slab b, the whole workgroup slab by slab
 *               (threads >= rows_per_tile*lanes_per_row).
 *               GRF_TILE_WAVES, GEMV: a wave is a unit of 64/lanes_per_row rows by
 *               lanes_per_row segments (lanes_per_row a power of two, 4..64); the waves of
 *               the workgroup take the tile's units (row group g, slab b) in turn and share
 *               nothing but the lookup tables, so there is no barrier between the table copy
 *               and the final row sums.
 *               GRF_TILE_WAVES, GEMM: a wave keeps 16 rows of the tile and four of a slab's
 *               lanes_per_row segments for the whole launch and stages its own stream pieces
 *               (see grf_bctx_gemm for threads and piece_cap).
 *               Wave tilings take matrices with fewer than 2^24 rows and 2^24 columns.
 *   k_parts     0 or 1: every tile walks all slabs.  k > 1 (grf_bctx_gemm / grf_ppcx_gemm only):
 *               the launch is cut along K: tile_rows / tile_class describe n_tiles / k row
 *               tiles, which must hold every row of the matrix once; launch tile t is row tile
 *               t mod (n_tiles / k), part t / (n_tiles / k), and walks the slabs [part * s,
 *               (part + 1) * s), s = ceil(n_slabs / k).  The parts' sums are added in part order
 *               by a second kernel, in the workspace (grf_gemm_workspace_bytes_split).
 * n_slabs = ceil(segs_per_row / lanes_per_row) in both schemes. */
#define GRF_TILE_SLABS 0
#define GRF_TILE_WAVES 1
typedef struct grf_fused_tiling {
  const uint32_t *tile_rows;
  const uint8_t *tile_class;
  uint32_t threads;
  uint32_t lanes_per_row, rows_per_tile, n_slabs, n_tiles;
  uint32_t piece_cap;
  uint32_t scheme;
  uint32_t k_parts;
} grf_fused_tiling;

/* Fused decode-GEMV, the slot the reference leaves for "a backend with a fused GEMM"
 * behind the CudaContextTensor contract (GCR/bitexact_context_serving.py:3-5; it replaces
 * decode() + F.linear of BctxLinear.forward, :365-376).  y[m][n] = bf16(sum_k x[m][k] *
 * W[n][k] + bias[n]) for 1 <= m_rows <= 8, fp32 accumulation in an order that does not
 * depend on m_rows (the M-invariance contract of GS/miv_gemv.py:10-29).
 * x: BF16 [m_rows][ldx], y: BF16 [m_rows][ldy], bias: BF16 [rows] or NULL.  With a
 * GRF_TILE_WAVES tiling x must be 16-byte aligned with ldx a multiple of 8 (the kernel reads
 * it in 16-byte vectors, two rows per launch: more rows run as further launches with the same
 * arithmetic per row); with a GRF_TILE_SLABS tiling 4-byte aligned with an even ldx. */
int grf_bctx_gemv(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream);

/* Host-side check of a caller-built frame and tiling before their first launch; no reference
 * counterpart (the reference builds its descriptors in Python and launches Triton).  The entry
 * points check the scalars of the two structures on every call; what the kernels take on
 * trust from the arrays behind them is checked here, on HOST copies of those arrays (the
 * structures' own pointers are device addresses and are not read; they may be null):
 *   seg_offset  in the order frame->raw_interleaved declares (the frame's: rows*segs_per_row
 *               + 1 entries; blocked: the rows held times segs_per_row + 1, row_pos required):
 *               never decreasing along a row, no entry below 4, the highest == main_n_bytes
 *               (a kernel copies [offset[s] & ~15, offset[s + lanes]) to LDS)
 *   tile_rows / tile_class  as in grf_fused_tiling (for k_parts > 1: the n_tiles / k_parts row
 *               tiles): slots name rows of the matrix, every row exactly once (use 3: any rows,
 *               any number of times), classes below nr
 *   row_class   u8 [rows] or NULL: when given, every row must be of its tile's class
 *   row_pos     u32 [rows] or NULL: when given, one-to-one
 * and every stream piece the launch stages (lanes_per_row segments of a row for use 0, 1 and
 * 3, four segments for use 2) must fit piece_cap, and the launch's LDS demand 160 KiB.
 * use: 0 = grf_bctx_fused_decode, 1 = grf_bctx_gemv(_group), 2 = grf_bctx_gemm(_group,
 * _noalloc), 3 = grf_bctx_fused_gather.  Returns GRF_OK or GRF_BAD_ARGUMENT / GRF_UNSUPPORTED
 * with the reason in grf_last_error().  Runs without a GPU. */
int grf_bctx_fused_validate_host(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, int use,
                                 const uint32_t *seg_offset, const uint32_t *tile_rows, const uint8_t *tile_class,
                                 const uint8_t *row_class, const uint32_t *row_pos);

/* Same walker with a store sink: out[rows*cols] BF16 words (decode() for fused frames). */
int grf_bctx_fused_decode(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint16_t *out,
                          int32_t *error, void *hip_stream);

/* Rows of a coded matrix, decoded by the same walker into a compact output (the embedding
 * lookup of CudaContextTensor.gather_rows, GCR/bitexact_context_gpu.py:159-168, without
 * decoding checkpoint blocks one lane each).  The tiling names the rows: slot s = tile *
 * rows_per_tile + r holds row tile_rows[s] (0xFFFFFFFF = empty; a row may appear in any
 * number of slots) and is written to out[s][cols]; the rows of a tile must share the row
 * class tile_class[tile].  One row per tile with lanes_per_row = segs_per_row needs no
 * grouping at all.  Rows outside the matrix are the caller's to reject. */
int grf_bctx_fused_gather(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint16_t *out,
                          int32_t *error, void *hip_stream);

/* Fused decode-GEMM on the matrix cores for any number of activation rows; same operand
 * meaning as grf_bctx_gemv.  Batch-invariant in the sense of GS/bi_csrc/bi_gemm.cuh:1-17:
 * with one tiling, row m of y is a function of row m of x and of W only.  x must be
 * 8-byte aligned with ldx a multiple of 4.  More than 128 rows run as several launches.
 *
 * A tiling for this function has scheme = GRF_TILE_WAVES, threads = 64 *
 * ceil(rows_per_tile / 16) * ceil(lanes_per_row / 4), and a piece_cap that holds the longest
 * stream piece of four consecutive segments of a row (from its 16-byte aligned start, + 8):
 * a wave walks four lane-segments of 16 rows and feeds the words it decodes to the matrix
 * cores from its registers.  workspace: device memory, 16-byte
 * aligned, at least grf_gemm_workspace_bytes(cols, m_rows) bytes (grf_gemm_workspace_bytes_split
 * for a tiling with k_parts > 1); each launch first writes
 * its activation rows there in operand order (a copy of x: cols * 32 + 256 bytes per 16 rows),
 * so calls that share a workspace must be ordered on one stream. */
int grf_bctx_gemm(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, void *workspace,
                  size_t workspace_bytes, int32_t *error, void *hip_stream);
size_t grf_gemm_workspace_bytes(uint32_t cols, uint32_t m_rows);
/* The workspace of a launch with a tiling cut into k_parts along K: the packed activations,
 * then (from the next multiple of 256 bytes) the parts' fp32 sums [k_parts][min(m_rows, 128)][rows].
 * Equal to grf_gemm_workspace_bytes for k_parts <= 1.  With x == NULL the caller has packed
 * the rows into the front of a workspace of this size. */
size_t grf_gemm_workspace_bytes_split(uint32_t cols, uint32_t rows, uint32_t k_parts, uint32_t m_rows);

/* grf_bctx_gemm without the workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid it).  No
 * counterpart in the reference.  The packed activations go to an 8 MiB array that is part of
 * the library's device image (every GPU the library runs on holds its copy until the process
 * ends); the call allocates and frees nothing.  It fails with GRF_UNSUPPORTED when
 * grf_gemm_workspace_bytes_split(cols, rows, k_parts, min(m_rows, 128)) exceeds
 * grf_gemm_noalloc_limit_bytes() (a tiling that is not cut along K, 128 rows: matrices up to
 * 32 752 columns; 64 rows: twice that).  x must not be NULL.  All
 * calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are ordered.  Results are those of grf_bctx_gemm, bit for bit. */
int grf_bctx_gemm_noalloc(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                          uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                          void *hip_stream);
size_t grf_gemm_noalloc_limit_bytes(void);

/* For several matrices that take the same activations (q/k/v, gate/up): writes 1..128 rows
 * of x into workspace in operand order once; grf_bctx_gemm / grf_ppcx_gemm called with
 * x == NULL, the same m_rows, a frame of this width and that workspace then multiply
 * without packing again.  No reference counterpart. */
int grf_pack_activations(const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint32_t cols, void *workspace,
                         size_t workspace_bytes, void *hip_stream);
uint32_t grf_bctx_gemm_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling);

/* Up to four coded matrices of one width that take the same activations (q/k/v, gate/up) in
 * one launch: y[i] = x W_i^T (+ bias[i]).  The grid is the members' tiles one after the
 * other, so small members fill the machine beside large ones; every member keeps its own
 * tiling, and a member's rows see exactly the arithmetic of grf_bctx_gemv / grf_bctx_gemm
 * with that tiling.  The tilings must share one thread count.  bias may be NULL, and so
 * may any bias[i]; the other arguments are those of the single-matrix entry points (for
 * the GEMM: x == NULL for rows packed by grf_pack_activations).  No reference counterpart. */
int grf_bctx_gemv_group(uint32_t n, const grf_bctx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint16_t *const *y, const uint32_t *ldy,
                        const uint16_t *const *bias, int32_t *error, void *hip_stream);
int grf_bctx_gemm_group(uint32_t n, const grf_bctx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint16_t *const *y, const uint32_t *ldy,
                        const uint16_t *const *bias, void *workspace, size_t workspace_bytes, int32_t *error,
                        void *hip_stream);

/* LDS bytes a launch needs for the given m_rows (0 for the store sink). */
uint32_t grf_bctx_fused_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint32_t m_rows);

/* PPCX frame prepared for the tile walker (modes 0 and 1 with the residuals resident as the
 * frame's packed 5-bit form; GCR/bitexact_predictive_codec.py:145-166, 179-186).  The row
 * label plays the part of the row class, the reference-word bin that of the column class:
 *   main_bytes  the frame's main rANS stream, readable for 16 bytes past main_n_bytes
 *   raw5        packed 5-bit residuals, MSB first, readable for 16 bytes past the end
 *   seg_state / seg_offset  as in grf_bctx_fused, contexts label[row]*16 + bin
 *   lut  u8 [n_labels][16 << lognb], tab u64 [n_labels][16][tabn+1]   as in grf_bctx_fused:
 *        low32 = start | (freq & 0xFFFF)<<16, high32 = the symbol's bits in the BF16 word
 *        (sign, exponent, mantissa bits 6..5) in place of symbol<<5
 * seg_len must be a multiple of 32.  Tilings are built over row labels.
 * raw_interleaved: 0 = raw5, and the bins plane given with every call, in the frame's order
 * (element i of the matrix: field i of raw5; bits 4*(i%8) of bins[i/8]).  B = 1, 2, 4, 8 or 16 =
 * both in records of 32 consecutive symbols of a row (20 bytes of raw5, 16 of bins), in blocks
 * of B rows: with q the row's position (row_pos[r], or r when row_pos is null) and U =
 * seg_len / 32, record t of segment s lies at index ((q / B * U + t) * segs_per_row + s) * B +
 * q % B -- the order grf_bctx_fused gives its 12-byte groups, for the same reason: the lanes of
 * a wave unit then read one run of bytes per visit.  grf_ppcx_bins_ordered writes a plane in
 * that order.  seg_state / seg_offset are then in the blocked order as well, exactly as
 * grf_bctx_fused describes it (segs_per_row + 1 entries per row). */
typedef struct grf_ppcx_fused {
  const uint8_t *main_bytes;
  const uint8_t *raw5;
  const uint32_t *seg_state;
  const uint32_t *seg_offset;
  const uint8_t *lut;
  const uint64_t *tab;
  const uint32_t *row_pos;
  uint32_t main_n_bytes;
  uint32_t rows, cols;
  uint32_t n_labels;
  uint32_t seg_len, segs_per_row;
  uint32_t shift, lognb, tabn;
  uint32_t whole_range; /* as in grf_bctx_fused */
  uint32_t raw_interleaved;
} grf_ppcx_fused;

/* The bin of every reference word (GCR/bitexact_predictive_codec.py:106-110, device form
 * GCR/bitexact_predictive_gpu_kernels.py:36-42: sign alignment by the row's flip, ordinal
 * key, number of thresholds <= key), packed 4 bits per element: element i in bits
 * 4*(i%8) of bins[i/8].  reference: BF16 [rows][cols] dense, 16-byte aligned, cols % 16 == 0;
 * flips u8 [rows]; thresholds u16 [15]; bins u32 [rows*cols/8]. */
int grf_ppcx_bins(const uint16_t *reference, const uint8_t *flips, const uint16_t *thresholds, uint32_t rows,
                  uint32_t cols, uint32_t *bins, void *hip_stream);
/* The same plane in the blocked order of a grf_ppcx_fused with raw_interleaved = block_rows
 * (seg_len, row_pos as there; cols % 32 == 0, seg_len % 32 == 0): bins u32 [rows_held * cols / 8]
 * with rows_held the rows the order holds (a multiple of block_rows above the largest
 * position); dwords of positions no row has are not written.  block_rows == 0 is
 * grf_ppcx_bins. */
int grf_ppcx_bins_ordered(const uint16_t *reference, const uint8_t *flips, const uint16_t *thresholds, uint32_t rows,
                          uint32_t cols, uint32_t seg_len, uint32_t block_rows, const uint32_t *row_pos,
                          uint32_t *bins, void *hip_stream);

/* Decode a prepared PPCX frame to dense BF16 words given the bins of its reference (replaces
 * the Triton launch of CudaPredictiveTensor.decode, GCR/bitexact_predictive_gpu.py:160-174,
 * for frames that meet the walker's limits).  A reference that is not the one the frame was
 * coded against makes segments miss their checkpoints: GRF_ERR_CHECKPOINT in *error. */
int grf_ppcx_fused_decode(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins,
                          uint16_t *out, int32_t *error, void *hip_stream);

/* Fused products on a prepared PPCX frame given the bins of its reference: the sinks and the
 * reduction orders of grf_bctx_gemv (1 <= m_rows <= 8, tilings as for that function) and
 * grf_bctx_gemm (any m_rows, one tiling for every row count).  They replace decode() +
 * F.linear of PredictiveContextTensor weights (GCR/bitexact_predictive_serving.py:490-523)
 * for frames stored untransposed. */
int grf_ppcx_gemv(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins, const uint16_t *x,
                  uint32_t ldx, uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream);
int grf_ppcx_gemm(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins, const uint16_t *x,
                  uint32_t ldx, uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, void *workspace,
                  size_t workspace_bytes, int32_t *error, void *hip_stream);

/* Up to four prepared PPCX frames of one width that take the same activations in one launch,
 * as grf_bctx_gemv_group / grf_bctx_gemm_group do for BCTX frames (same grid of the members'
 * tiles, same restrictions on the tilings, a member's rows bit-equal to grf_ppcx_gemv /
 * grf_ppcx_gemm with that tiling); bins[i] is the bins plane of member i's reference.  The
 * reference multiplies every such weight on its own (GCR/bitexact_predictive_serving.py:490-523). */
int grf_ppcx_gemv_group(uint32_t n, const grf_ppcx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint32_t *const *bins, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                        uint16_t *const *y, const uint32_t *ldy, const uint16_t *const *bias, int32_t *error,
                        void *hip_stream);
int grf_ppcx_gemm_group(uint32_t n, const grf_ppcx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint32_t *const *bins, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                        uint16_t *const *y, const uint32_t *ldy, const uint16_t *const *bias, void *workspace,
                        size_t workspace_bytes, int32_t *error, void *hip_stream);

/* A one-lane kernel that writes slot[0] = the device's constant-rate counter
 * (grf_wall_clock_khz), slot[1] = its shader-clock counter and slot[2] = the identifier of the
 * compute unit it ran on, all read when the kernel runs, i.e. in stream order after the work
 * launched before it.  Two of them around launches give their duration on the device where
 * events cannot be recorded (inside a captured HIP graph); two that ran on the same compute
 * unit (shader-clock counters of different parts of the chip do not share a zero) also give
 * the shader clock the work between them ran at.  slot: device memory, three 64-bit words.
 * No reference counterpart; it allocates nothing and can be captured. */
int grf_timestamp(uint64_t *slot, void *hip_stream);
/* Rate of the constant counter of the current device in kHz (0 if the runtime does not say). */
int grf_wall_clock_khz(void);

const char *grf_last_error(void);
int grf_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif
