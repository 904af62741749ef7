// Fused decode-GEMV (VALU dot products, 1 <= M <= 8) and the store-sink twin that
// backs decode() for fused frames.  See fused_device.h for the decomposition.
//
// Reduction order of one output element, fixed for every M and for every tiling:
// the S products of a segment are folded into one fp32 accumulator two columns at a
// time in increasing k (v_dot2c_f32_bf16: acc += w[k]*x[k] + w[k+1]*x[k+1]); the K/S
// segment partials of a row are then added in segment order 0..K/S-1 by one thread
// (slab after slab into a running sum); bias is added in fp32 and the sum is rounded
// to BF16 once.
#include <hip/hip_runtime.h>

#include <string>

#include "fused_device.h"

namespace grf {
int set_error(int code, const std::string &what);  // decode_general.hip
}

namespace {

using grf::FusedLdsLayout;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2_bf16(uint32_t w_pair, uint32_t x_pair, float acc) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w_pair), __builtin_bit_cast(bf16x2_t, x_pair),
                                         acc, false);
#else
  return acc + (float)(w_pair ^ x_pair);  // host pass only parses this
#endif
}

__device__ __forceinline__ uint16_t round_bf16(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

template <int M, bool STORE>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_walk_kernel(grf_bctx_fused f, grf_fused_tiling g,
                                                                            const uint16_t *x, uint32_t ldx,
                                                                            uint16_t *y, uint32_t ldy,
                                                                            const uint16_t *bias, uint16_t *out,
                                                                            int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const FusedLdsLayout L(f, g, STORE ? 0 : M);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x, tile = blockIdx.x;
  const uint32_t P = g.lanes_per_row, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = g.tile_class[tile];

  grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f)};

  const uint32_t r = tid / P, p = tid % P;
  const uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;
  uint16_t *xs = reinterpret_cast<uint16_t *>(lds + L.xs);
  const uint32_t xpitch = S + grf::kXPad;
  const uint32_t width = P * S;
  float *part = reinterpret_cast<float *>(lds + L.part);      // [R][P][M] partials of one slab
  float *rowsum = reinterpret_cast<float *>(lds + L.rowsum);  // [R][M] running sums
  uint32_t bad = 0;

  grf::PieceSpan span{0, 0};
  if (row != grf::kNoRow) span.fetch(f, row * f.segs_per_row, min(P, f.segs_per_row));
  for (uint32_t b = 0; b < g.n_slabs; ++b) {
    if (b) __syncthreads();  // everyone is done with the previous slab's LDS data
    const uint32_t col_base = b * width;
    if (!STORE) {  // x slab as BF16 pairs, one padded run per lane-segment
      const uint32_t pairs = width / 2;
      for (uint32_t i = tid; i < M * pairs; i += nthreads) {
        const uint32_t m = i / pairs, c = (i % pairs) * 2, col = col_base + c;
        uint32_t v = 0;
        if (col < K) v = *reinterpret_cast<const uint32_t *>(x + (size_t)m * ldx + col);
        *reinterpret_cast<uint32_t *>(xs + (m * P + c / S) * xpitch + c % S) = v;
      }
    }
    const uint32_t first_seg = b * P;
    const uint32_t nseg = min(P, f.segs_per_row - first_seg);
    const uint32_t piece_off = L.stream + r * g.piece_cap;
    const bool walks = row != grf::kNoRow && p < nseg;
    const uint32_t seg_base = row != grf::kNoRow ? row * f.segs_per_row + first_seg : 0;
    const uint32_t col0 = (first_seg + p) * S;
    const uint64_t elem0 = (uint64_t)row * K + col0;
    grf::SegmentWalk w;
    uint32_t a0 = 0;
    if (walks) w.prefetch(f, seg_base + p, elem0, col0);
    if (row != grf::kNoRow) {
      a0 = grf::fused_stage_piece(lds, piece_off, f, span, p, P);
      if (b + 1 < g.n_slabs)  // the next slab's byte range, while this one is walked
        span.fetch(f, seg_base + P, min(P, f.segs_per_row - first_seg - P));
    }
    __syncthreads();
    if (walks) {
      w.start(piece_off, a0);
      const uint16_t *xr = xs + p * xpitch;
      float acc[M];
#pragma unroll
      for (int m = 0; m < M; ++m) acc[m] = 0.f;
      for (uint32_t t = 0; t < S; t += 16) {
        uint32_t pair[8];
        w.decode16(t, S, q, pair);
        if (STORE) {
          uint4 *dst = reinterpret_cast<uint4 *>(out + elem0 + t);
          dst[0] = make_uint4(pair[0], pair[1], pair[2], pair[3]);
          dst[1] = make_uint4(pair[4], pair[5], pair[6], pair[7]);
        } else {
#pragma unroll
          for (int m = 0; m < M; ++m) {
            const uint4 *xm = reinterpret_cast<const uint4 *>(xr + m * P * xpitch + t);
            const uint4 xa = xm[0], xb = xm[1];
            const uint32_t xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[m] = dot2_bf16(pair[k], xv[k], acc[m]);
          }
        }
      }
      if (!STORE) {
#pragma unroll
        for (int m = 0; m < M; ++m) part[(r * P + p) * M + m] = acc[m];
      }
      if (!w.ended_on_checkpoint(f)) bad |= GRF_ERR_CHECKPOINT;
    }
    if (!STORE) {  // fold this slab's partials into the running row sums, in segment order
      __syncthreads();
      for (uint32_t i = tid; i < R * M; i += nthreads) {
        const uint32_t rr = i / M, m = i % M;
        const float *pr = part + (rr * P) * M + m;
        float sum = b ? rowsum[i] : pr[0];
        for (uint32_t j = b ? 0 : 1; j < nseg; ++j) sum += pr[j * M];
        rowsum[i] = sum;
      }
    }
  }

  if (!STORE) {
    // every running sum was last written by the thread that reads it here
    for (uint32_t i = tid; i < R * M; i += nthreads) {
      const uint32_t rr = i / M, m = i % M;
      const uint32_t orow = g.tile_rows[tile * R + rr];
      if (orow == grf::kNoRow) continue;
      float sum = rowsum[i];
      if (bias) sum += __uint_as_float((uint32_t)bias[orow] << 16);
      y[(size_t)m * ldy + orow] = round_bf16(sum);
    }
  }
  if (bad) atomicOr(error, (int)bad);
}

}  // namespace

namespace grf {
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who) {
  auto bad = [&](const char *why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (!f.main_bytes || !f.raw6 || !f.seg_state || !f.seg_offset || !g.tile_rows || !g.tile_class || !f.lut ||
      !f.tab || !f.col_class)
    return bad("null pointer in frame");
  if (!f.rows || !f.cols || !g.n_tiles || !g.n_slabs) return bad("empty geometry");
  if (f.seg_len == 0 || f.seg_len % 16 || (uint64_t)f.seg_len * f.segs_per_row != f.cols)
    return bad("segment length must be a multiple of 16 that divides the row length");
  if (!g.threads || g.threads % 64 || g.threads > (uint32_t)grf::kFusedMaxThreads) return bad("thread count");
  if (!g.lanes_per_row || !g.rows_per_tile || g.lanes_per_row * g.rows_per_tile > g.threads)
    return bad("tile does not fit one workgroup");
  if (g.n_slabs != (f.segs_per_row + g.lanes_per_row - 1) / g.lanes_per_row) return bad("slab count mismatch");
  if (f.nc == 0 || f.nc > 16 || (f.nc & (f.nc - 1))) return bad("column class count");
  if (f.shift > 12 || f.lognb != 16 - f.shift) return bad("bucket shift");
  if (f.tabn == 0 || f.tabn > 255) return bad("sparse table size");
  if (g.piece_cap % 16 || g.piece_cap < 16) return bad("piece capacity");
  if ((uint64_t)f.rows * f.cols > 0xFFFFFFFFull) return bad("matrix too large");
  return GRF_OK;
}
}  // namespace grf

namespace {
using grf::check_fused_frame;

template <int M, bool STORE>
int launch(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint16_t *y,
           uint32_t ldy, const uint16_t *bias, uint16_t *out, int32_t *error, hipStream_t s) {
  const FusedLdsLayout L(f, g, STORE ? 0 : M);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  auto kernel = fused_walk_kernel<M, STORE>;
  if (L.total > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total);
    if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("LDS attribute: ") + hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(g.threads), L.total, s, f, g, x, ldx, y, ldy, bias, out, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused kernel: ") + hipGetErrorString(e));
  return GRF_OK;
}

}  // namespace

extern "C" {

uint32_t grf_bctx_fused_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint32_t m_rows) {
  if (!frame || !tiling) return 0;
  return FusedLdsLayout(*frame, *tiling, m_rows).total;
}

int grf_bctx_gemv(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream) {
  if (!frame || !tiling || !x || !y || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv: null argument");
  if (int rc = check_fused_frame(*frame, *tiling, "grf_bctx_gemv")) return rc;
  if (m_rows < 1 || m_rows > 8) return grf::set_error(GRF_UNSUPPORTED, "grf_bctx_gemv: 1 <= m_rows <= 8");
  if (ldx < frame->cols || ldy < frame->rows || (ldx & 1) || ((uintptr_t)x & 3))
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv: x must be 4-byte aligned with an even leading dimension");
  hipStream_t s = (hipStream_t)hip_stream;
  const grf_bctx_fused &f = *frame;
  const grf_fused_tiling &g = *tiling;
  switch (m_rows) {
    case 1: return launch<1, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 2: return launch<2, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 3: return launch<3, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 4: return launch<4, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 5: return launch<5, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 6: return launch<6, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 7: return launch<7, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    default: return launch<8, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
  }
}

int grf_bctx_fused_decode(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint16_t *out,
                          int32_t *error, void *hip_stream) {
  if (!frame || !tiling || !out || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_decode: null argument");
  if (int rc = check_fused_frame(*frame, *tiling, "grf_bctx_fused_decode")) return rc;
  return launch<1, true>(*frame, *tiling, nullptr, 0, nullptr, 0, nullptr, out, error, (hipStream_t)hip_stream);
}

}  // extern "C"
