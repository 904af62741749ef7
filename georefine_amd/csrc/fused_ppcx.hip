// Fused decode of PPCX frames: the tile walker of the context codec with the predictive
// symbol model.
//
// A PPCX main symbol is coded in the context (row label, bin of the reference word at the
// same position) -- GCR/bitexact_predictive_codec.py:179-186, device form
// GCR/bitexact_predictive_gpu_kernels.py:24-58.  The row label takes the part of the row
// class (a tile holds rows of one label, so 16 bin contexts are live and their tables fit in
// LDS); the bin takes the part of the column class, but differs per element.  It is computed
// from the dense reference words by a separate elementwise kernel into a transient plane of
// 4-bit bins, which the walker then reads like column classes: 8 bytes per 16 symbols.
// Doing the threshold search inside the walk would add ~12 instructions to a 25-instruction
// step; the plane costs one pass over the reference at memory speed.
//
// Residuals are the packed 5-bit fields of the frame (GCR/bitexact_predictive_codec.py:145-166,
// MSB first): 10 bytes per 16 symbols, so every second group starts half a dword in.
//
// The walker plugs into the generic sinks of fused_kernels.h: store (decode), GEMV, GEMM.
#include "fused_kernels.h"

namespace {

// ---- bins plane ----

// A workgroup first tabulates the bin of all 65 536 sign-aligned words in LDS (64 KiB, one
// byte each; 64 entries per thread), then streams its share of the matrix through the
// table: per element one xor with the row's flip, one LDS byte read and one shift-or.
// 16 elements per thread and pass: 32 bytes of reference words in, two dwords of eight
// 4-bit bins out (element i of the matrix in bits 4*(i%8) of dword i/8).
constexpr uint32_t kBinsThreads = 1024;

// Where the two dwords of the group of 16 elements that starts at element `at` go: the frame's
// order, or (block != 0) the blocked order of records of 32 elements (four dwords each).
struct BinsOrder {
  uint32_t cols, seg_len, segs_per_row, block;
  const uint32_t *row_pos;
  __device__ __forceinline__ uint64_t dword_of(uint64_t at) const {
    if (!block) return at / 8;
    const uint32_t row = (uint32_t)(at / cols), col = (uint32_t)(at % cols);
    const uint32_t q = row_pos ? row_pos[row] : row, within = q % block;
    const uint64_t record = (uint64_t)(q - within) * (cols / 32) +
                            ((uint64_t)((col % seg_len) / 32) * segs_per_row + col / seg_len) * block + within;
    return record * 4 + (col % 32) / 8;
  }
};

__global__ __launch_bounds__(kBinsThreads) void ppcx_bins_kernel(const uint16_t *reference, const uint8_t *flips,
                                                                  const uint16_t *thresholds, uint32_t cols,
                                                                  uint64_t n, uint32_t *bins, BinsOrder order) {
  extern __shared__ __align__(16) uint8_t table[];  // bin of the sign-aligned word
  __shared__ uint16_t th[16];
  if (threadIdx.x < 15) th[threadIdx.x] = thresholds[threadIdx.x];
  __syncthreads();
  for (uint32_t a = threadIdx.x * 4; a < 65536; a += kBinsThreads * 4) {
    uint32_t four = 0;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) four |= grf::threshold_bin(th, grf::ordinal_key(a + i, 0)) << (8 * i);
    *reinterpret_cast<uint32_t *>(table + a) = four;
  }
  __syncthreads();
  // two chunks of 16 elements per thread and pass, their loads issued together
  const uint64_t stride = (uint64_t)gridDim.x * kBinsThreads * 16;
  for (uint64_t first = ((uint64_t)blockIdx.x * kBinsThreads + threadIdx.x) * 16; first < n; first += 2 * stride) {
    const uint64_t at[2] = {first, first + stride};
    uint4 raw[2][2];
    uint32_t flip[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (at[c] >= n) continue;
      const uint4 *src = reinterpret_cast<const uint4 *>(reference + at[c]);  // cols % 16 == 0: one row
      raw[c][0] = src[0];
      raw[c][1] = src[1];
      flip[c] = flips[at[c] / cols] ? 0x80008000u : 0u;
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (at[c] >= n) continue;
      const uint32_t w[8] = {raw[c][0].x ^ flip[c], raw[c][0].y ^ flip[c], raw[c][0].z ^ flip[c], raw[c][0].w ^ flip[c],
                             raw[c][1].x ^ flip[c], raw[c][1].y ^ flip[c], raw[c][1].z ^ flip[c], raw[c][1].w ^ flip[c]};
      uint32_t packed[2] = {0, 0};
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t a = (i % 2) ? (w[i / 2] >> 16) : (w[i / 2] & 0xFFFFu);
        packed[i / 8] |= (uint32_t)table[a] << (4 * (i % 8));
      }
      *reinterpret_cast<uint2 *>(bins + order.dword_of(at[c])) = make_uint2(packed[0], packed[1]);
    }
  }
}

// ---- walker ----

// Sixteen packed 5-bit residuals: 80 bits that start `lead` bits (0 or 16) into three
// big-endian dwords.
struct Raw5x16 {
  uint32_t w0, w1, w2;  // the 80 bits left-aligned in w0:w1:w2
  __device__ __forceinline__ void set(uint32_t a, uint32_t b, uint32_t c, uint32_t lead) {
    a = __builtin_bswap32(a);
    b = __builtin_bswap32(b);
    c = __builtin_bswap32(c);
    // shift the 96-bit string left by lead (alignbit shifts a 64-bit pair right by 32 - lead)
    w0 = lead ? __builtin_amdgcn_alignbit(a, b, 32 - lead) : a;
    w1 = lead ? __builtin_amdgcn_alignbit(b, c, 32 - lead) : b;
    w2 = lead ? c << lead : c;
  }
  template <int K>
  __device__ __forceinline__ uint32_t field() const {
    constexpr int bit = K * 5, word = bit / 32, off = bit % 32;
    const uint32_t a = word == 0 ? w0 : (word == 1 ? w1 : w2);
    if constexpr (off + 5 <= 32) {
      return __builtin_amdgcn_ubfe(a, 32 - 5 - off, 5);
    } else {
      const uint32_t b = word == 0 ? w1 : w2;
      return __builtin_amdgcn_ubfe(__builtin_amdgcn_alignbit(a, b, 64 - 5 - off), 0, 5);
    }
  }
};

struct PpcxWalk {
  grf::Cursor c;
  uint32_t gofs, eofs;        // byte offsets of this segment's and the next segment's checkpoints
  uint32_t end_state, end_jb;  // what the walk must end on: the next checkpoint's state, and its offset as an LDS cursor
  const uint8_t *rawp;    // the residual array (uniform)
  const uint2 *binp;      // the bins plane (uniform)
  uint32_t n0, n1, n2;
  uint2 nb;
  Raw5x16 rr;      // the group being decoded
  uint32_t bw[2];

  // The residuals and bins of the group of 16 symbols g of the segment: in the frame's order a
  // segment's bytes are one run (10 and 8 bytes a group); in the blocked order a record of two
  // groups (20 and 16 bytes) is followed by the same record of the block's next row.  Either
  // way the second group of a record starts two bytes into its third dword.
  uint32_t raw_off, bin_off;        // byte offsets of the segment's first record in the two arrays
  uint32_t raw_stride, bin_stride;  // bytes from a record to the segment's next record
  __device__ __forceinline__ const uint32_t *group_dwords(uint32_t g) const {
    return reinterpret_cast<const uint32_t *>(rawp + (raw_off + (g >> 1) * raw_stride + (g & 1u) * 8u));
  }
  __device__ __forceinline__ uint2 group_bins(uint32_t g) const {
    return *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint8_t *>(binp) +
                                            (bin_off + (g >> 1) * bin_stride + (g & 1u) * 8u));
  }
  // global reads of the segment, issued before the wait for the slab's stream bytes
  __device__ __forceinline__ void prefetch(const grf_bctx_fused &f, uint32_t seg_, uint32_t elem0, uint32_t,
                                           uint32_t seg_in_row, uint32_t rpos) {
    const uint32_t slot = seg_, next = slot + grf::fused_seg_step(f);  // (seg_: the entry, fused_seg_slot)
    gofs = grf::fused_index_entry(f.seg_offset, slot);
    eofs = grf::fused_index_entry(f.seg_offset, next);
    c.state = grf::fused_index_entry(f.seg_state, slot);
    end_state = grf::fused_index_entry(f.seg_state, next);
    rawp = f.raw6;
    binp = reinterpret_cast<const uint2 *>(f.col_class);
    if (f.raw_interleaved) {
      const uint32_t B = f.raw_interleaved, within = rpos & (B - 1);
      const uint32_t record = (rpos - within) * (f.cols / 32) + seg_in_row * B + within;  // (once per segment)
      raw_off = record * 20;
      bin_off = record * 16;
      raw_stride = f.segs_per_row * B * 20;
      bin_stride = f.segs_per_row * B * 16;
    } else {
      raw_off = elem0 / 8 * 5;
      bin_off = elem0 / 2;
      raw_stride = 20;
      bin_stride = 16;
    }
    const uint32_t *d = group_dwords(0);
    n0 = d[0];
    n1 = d[1];
    n2 = d[2];
    nb = group_bins(0);
  }
  __device__ __forceinline__ void start(uint32_t piece_off, uint32_t a0) {
    c.jb = (piece_off + (gofs - a0)) << 3;
    end_jb = c.jb + ((eofs - gofs) << 3);
  }

  __device__ __forceinline__ void begin16(uint32_t t, uint32_t S) {
    rr.set(n0, n1, n2, (t & 16u) ? 16u : 0u);
    bw[0] = nb.x;
    bw[1] = nb.y;
    // the last group loads itself again rather than branch around the loads
    const uint32_t next = min(t / 16 + 1, S / 16 - 1);
    const uint32_t *d = group_dwords(next);
    n0 = d[0];
    n1 = d[1];
    n2 = d[2];
    nb = group_bins(next);
  }
  template <int H, int SCAN = grf::kScanAny>
  __device__ __forceinline__ void half(const grf::FusedParams &q, uint32_t (&pair)[4]) {
    uint32_t bits[8];
#define GRF_STEP2(i)                                                                                  \
  {                                                                                                   \
    const uint32_t bin0 = __builtin_amdgcn_ubfe(bw[H], 4 * (i), 4);                                   \
    const uint32_t bin1 = __builtin_amdgcn_ubfe(bw[H], 4 * (i) + 4, 4);                               \
    uint32_t h0, h1;                                                                                  \
    grf::fused_symbol_pair_in<SCAN>(c, __umul24(bin0, q.block_pitch), __umul24(bin1, q.block_pitch), q, h0, h1); \
    bits[i] = h0 | rr.field<8 * H + (i)>();                                                           \
    bits[(i) + 1] = h1 | rr.field<8 * H + (i) + 1>();                                                 \
  }
    GRF_STEP2(0) GRF_STEP2(2) GRF_STEP2(4) GRF_STEP2(6)
#undef GRF_STEP2
#pragma unroll
    for (int k = 0; k < 4; ++k) pair[k] = __builtin_amdgcn_perm(bits[2 * k + 1], bits[2 * k], 0x05040100u);
  }
  __device__ __forceinline__ void decode16(uint32_t t, uint32_t S, const grf::FusedParams &q, uint32_t (&pair)[8]) {
    begin16(t, S);
    half<0>(q, reinterpret_cast<uint32_t (&)[4]>(pair[0]));
    half<1>(q, reinterpret_cast<uint32_t (&)[4]>(pair[4]));
  }

  __device__ __forceinline__ bool ended_on_checkpoint(const grf_bctx_fused &f) const {
    (void)f;
    return c.state == end_state && c.jb == end_jb;
  }
};

// The PPCX frame in the walker's frame structure: raw6 = packed 5-bit residuals,
// col_class = the bins plane, nr = labels, nc = 16 bins.
int walker_frame(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins, const char *who,
                 grf_bctx_fused &f, grf::TilingUse use = grf::kSlabTiling) {
  if (!frame || !tiling || !bins) return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": null argument");
  f = grf_bctx_fused{};
  f.main_bytes = frame->main_bytes;
  f.raw6 = frame->raw5;
  f.seg_state = frame->seg_state;
  f.seg_offset = frame->seg_offset;
  f.lut = frame->lut;
  f.tab = frame->tab;
  f.col_class = reinterpret_cast<const uint8_t *>(bins);
  f.main_n_bytes = frame->main_n_bytes;
  f.rows = frame->rows;
  f.cols = frame->cols;
  f.nr = frame->n_labels;
  f.nc = 16;
  f.seg_len = frame->seg_len;
  f.segs_per_row = frame->segs_per_row;
  f.shift = frame->shift;
  f.lognb = frame->lognb;
  f.tabn = frame->tabn;
  f.whole_range = frame->whole_range;
  f.raw_interleaved = frame->raw_interleaved;
  f.row_pos = frame->row_pos;
  if (int rc = grf::check_fused_frame(f, *tiling, who, use)) return rc;
  if (f.seg_len % 32)  // a segment's residual bytes must start on a dword
    return grf::set_error(GRF_UNSUPPORTED, std::string(who) + ": segment length must be a multiple of 32");
  return GRF_OK;
}

}  // namespace

extern "C" {

int grf_ppcx_bins_ordered(const uint16_t *reference, const uint8_t *flips, const uint16_t *thresholds, uint32_t rows,
                          uint32_t cols, uint32_t seg_len, uint32_t block_rows, const uint32_t *row_pos,
                          uint32_t *bins, void *hip_stream) {
  if (!reference || !flips || !thresholds || !bins)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_bins: null argument");
  if (!rows || !cols || cols % 16 || ((uintptr_t)reference & 15) || ((uintptr_t)bins & 7))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          "grf_ppcx_bins: row length must be a multiple of 16, reference 16-byte and bins 8-byte aligned");
  if (block_rows && (block_rows > 16 || (block_rows & (block_rows - 1)) || !seg_len || seg_len % 32 || cols % seg_len))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          "grf_ppcx_bins_ordered: blocks of 1, 2, 4, 8 or 16 rows, segments a multiple of 32 that divides the row");
  const uint64_t n = (uint64_t)rows * cols;
  if (n > 0xFFFFFFFFull) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_bins: matrix too large");
  const uint64_t chunks = (n / 16 + kBinsThreads - 1) / kBinsThreads;
  const uint32_t blocks = (uint32_t)(chunks < 512 ? chunks : 512);  // two workgroups per CU amortise the table
  const BinsOrder order{cols, seg_len, seg_len ? cols / seg_len : 0, block_rows, row_pos};
  hipLaunchKernelGGL(ppcx_bins_kernel, dim3(blocks), dim3(kBinsThreads), 65536, (hipStream_t)hip_stream, reference,
                     flips, thresholds, cols, n, bins, order);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("bins kernel: ") + hipGetErrorString(e));
  return GRF_OK;
}

int grf_ppcx_bins(const uint16_t *reference, const uint8_t *flips, const uint16_t *thresholds, uint32_t rows,
                  uint32_t cols, uint32_t *bins, void *hip_stream) {
  return grf_ppcx_bins_ordered(reference, flips, thresholds, rows, cols, 0, 0, nullptr, bins, hip_stream);
}

int grf_ppcx_fused_decode(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins,
                          uint16_t *out, int32_t *error, void *hip_stream) {
  if (!out || !error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_fused_decode: null argument");
  grf_bctx_fused f;
  if (int rc = walker_frame(frame, tiling, bins, "grf_ppcx_fused_decode", f)) return rc;
  return grf::launch_walk<PpcxWalk, 1, grf::kStore>(f, *tiling, nullptr, 0, nullptr, 0, nullptr, out, error,
                                             (hipStream_t)hip_stream);
}

int grf_ppcx_gemv(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins, const uint16_t *x,
                  uint32_t ldx, uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream) {
  if (!x || !y || !error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_gemv: null argument");
  grf_bctx_fused f;
  if (int rc = walker_frame(frame, tiling, bins, "grf_ppcx_gemv", f, grf::kGemvTiling)) return rc;
  return grf::launch_gemv<PpcxWalk>("grf_ppcx_gemv", f, *tiling, x, ldx, m_rows, y, ldy, bias, error,
                                    (hipStream_t)hip_stream);
}

int grf_ppcx_gemm(const grf_ppcx_fused *frame, const grf_fused_tiling *tiling, const uint32_t *bins, const uint16_t *x,
                  uint32_t ldx, uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, void *workspace,
                  size_t workspace_bytes, int32_t *error, void *hip_stream) {
  if (!y || !error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_gemm: null argument");  // x may be null: packed rows
  grf_bctx_fused f;
  if (int rc = walker_frame(frame, tiling, bins, "grf_ppcx_gemm", f, grf::kGemmTiling)) return rc;
  return grf::launch_gemm<PpcxWalk>("grf_ppcx_gemm", f, *tiling, x, ldx, m_rows, y, ldy, bias, workspace,
                                    workspace_bytes, error, (hipStream_t)hip_stream);
}


}  // extern "C"

namespace {

// The members of a grouped PPCX launch in the walker's frame structure.
struct PpcxMembers {
  grf_bctx_fused frames[grf::kMaxGroup];
  const grf_bctx_fused *pointers[grf::kMaxGroup];
  int fill(const char *who, uint32_t n, const grf_ppcx_fused *const *members, const grf_fused_tiling *const *tilings,
           const uint32_t *const *bins, grf::TilingUse use) {
    if (n < 1 || n > grf::kMaxGroup) return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": a group has 1..4 members");
    if (!members || !tilings || !bins) return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": null argument");
    for (uint32_t i = 0; i < n; ++i) {
      if (int rc = walker_frame(members[i], tilings[i], bins[i], who, frames[i], use)) return rc;
      pointers[i] = &frames[i];
    }
    return GRF_OK;
  }
};

}  // namespace

extern "C" {

int grf_ppcx_gemv_group(uint32_t n, const grf_ppcx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint32_t *const *bins, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                        uint16_t *const *y, const uint32_t *ldy, const uint16_t *const *bias, int32_t *error,
                        void *hip_stream) {
  if (!error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_gemv_group: null argument");
  PpcxMembers members;
  if (int rc = members.fill("grf_ppcx_gemv_group", n, frames, tilings, bins, grf::kGemvTiling)) return rc;
  const grf::GroupSpec spec{n, members.pointers, tilings, y, ldy, bias};
  return grf::launch_gemv_group<PpcxWalk>("grf_ppcx_gemv_group", spec, x, ldx, m_rows, error, (hipStream_t)hip_stream);
}

int grf_ppcx_gemm_group(uint32_t n, const grf_ppcx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint32_t *const *bins, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                        uint16_t *const *y, const uint32_t *ldy, const uint16_t *const *bias, void *workspace,
                        size_t workspace_bytes, int32_t *error, void *hip_stream) {
  if (!error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_ppcx_gemm_group: null argument");
  PpcxMembers members;
  if (int rc = members.fill("grf_ppcx_gemm_group", n, frames, tilings, bins, grf::kGemmTiling)) return rc;
  const grf::GroupSpec spec{n, members.pointers, tilings, y, ldy, bias};
  return grf::launch_gemm_group<PpcxWalk>("grf_ppcx_gemm_group", spec, x, ldx, m_rows, workspace, workspace_bytes,
                                          error, (hipStream_t)hip_stream);
}

}  // extern "C"
