// Fused decode-GEMV (VALU FMA chains, 1 <= M <= 8) and the store-sink twin that
// backs decode() for fused frames.  See fused_device.h for the decomposition.
//
// Reduction order of one output element, fixed for every M: each lane folds the
// S products of its segment into one fp32 accumulator in increasing k with fmaf,
// continues with its segment of the next slab, and at the end the P lane
// partials of a row are added in lane order 0..P-1 by one thread; bias is added
// in fp32 and the sum is rounded to BF16 once.
#include <hip/hip_runtime.h>

#include <string>

#include "fused_device.h"

namespace grf {
int set_error(int code, const std::string &what);  // decode_general.hip
}

namespace {

using grf::FusedLdsLayout;
using grf::kFusedThreads;

__device__ __forceinline__ uint16_t round_bf16(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

template <int M, bool STORE>
__global__ __launch_bounds__(kFusedThreads) void fused_walk_kernel(grf_bctx_fused f, const uint16_t *x,
                                                                    uint32_t ldx, uint16_t *y, uint32_t ldy,
                                                                    const uint16_t *bias, uint16_t *out,
                                                                    int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const FusedLdsLayout L(f, STORE ? 0 : M);
  const uint32_t tid = threadIdx.x, tile = blockIdx.x;
  const uint32_t P = f.lanes_per_row, R = f.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = f.tile_class[tile];

  {  // this row class's lookup tables -> LDS
    const uint32_t lut_bytes = f.nc << f.lognb;
    const uint4 *src = reinterpret_cast<const uint4 *>(f.lut + (size_t)cls * lut_bytes);
    uint4 *dst = reinterpret_cast<uint4 *>(lds + L.lut);
    for (uint32_t i = tid; i < lut_bytes / 16; i += kFusedThreads) dst[i] = src[i];
    const uint32_t entries = (f.tabn + 1) * f.nc;
    const uint2 *ts = reinterpret_cast<const uint2 *>(f.tab) + (size_t)cls * entries;
    uint2 *td = reinterpret_cast<uint2 *>(lds + L.tab);
    for (uint32_t i = tid; i < entries; i += kFusedThreads) td[i] = ts[i];
  }

  const uint32_t r = tid / P, p = tid % P;
  const uint32_t row = r < R ? f.tile_rows[tile * R + r] : grf::kNoRow;
  float *xs = reinterpret_cast<float *>(lds + L.xs);
  uint8_t *ccs = lds + L.cc8;
  const uint32_t xpitch = S + 4;
  const uint32_t width = P * S;
  float acc[M];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m] = 0.f;
  uint32_t bad = 0;

  for (uint32_t b = 0; b < f.n_slabs; ++b) {
    __syncthreads();  // everyone is done with the previous slab's LDS data
    const uint32_t col_base = b * width;
    if (!STORE) {
      for (uint32_t i = tid; i < M * width; i += kFusedThreads) {
        const uint32_t m = i / width, c = i % width, col = col_base + c;
        const uint32_t bits = col < K ? (uint32_t)x[(size_t)m * ldx + col] << 16 : 0u;
        xs[(m * P + c / S) * xpitch + c % S] = __uint_as_float(bits);
      }
    }
    for (uint32_t i = tid; i < width; i += kFusedThreads) {
      const uint32_t col = col_base + i;
      ccs[i] = col < K ? f.col_class[col] : 0;
    }
    const uint32_t first_seg = b * P;
    const uint32_t nseg = min(P, f.segs_per_row - first_seg);
    uint32_t a0 = 0, seg_base = 0;
    uint8_t *piece = lds + L.stream + r * f.piece_cap;
    if (row != grf::kNoRow) {
      seg_base = row * f.segs_per_row + first_seg;
      const uint32_t g0 = f.seg_offset[seg_base], g1 = f.seg_offset[seg_base + nseg];
      a0 = g0 & ~15u;
      for (uint32_t o = a0 + p * 16; o < g1; o += P * 16)
        *reinterpret_cast<uint4 *>(piece + (o - a0)) = *reinterpret_cast<const uint4 *>(f.main_bytes + o);
    }
    __syncthreads();
    if (row != grf::kNoRow && p < nseg) {
      const uint32_t seg = seg_base + p;
      uint32_t state = f.seg_state[seg];
      const uint32_t g = f.seg_offset[seg];
      const uint32_t ip0 = L.stream + r * f.piece_cap + (g - a0);
      uint32_t ip = ip0;
      const uint32_t col0 = (first_seg + p) * S;
      const uint64_t elem0 = (uint64_t)row * K + col0;
      const uint8_t *rawp = f.raw6 + elem0 / 4 * 3;
      const float *xr = xs + p * xpitch;
      const uint8_t *cr = ccs + p * S;
      for (uint32_t t = 0; t < S; t += 16) {
        grf::Raw6x16 rr;
        rr.load(rawp + t / 16 * 12);
        const uint4 c4 = *reinterpret_cast<const uint4 *>(cr + t);
        const uint32_t cw[4] = {c4.x, c4.y, c4.z, c4.w};
        uint32_t bits[16];
#define GRF_STEP(k)                                                                                        \
  {                                                                                                        \
    const uint32_t cc = (cw[(k) / 4] >> (8 * ((k) % 4))) & 0xFFu;                                          \
    const uint32_t hi = grf::fused_symbol(state, ip, lds, L.lut, L.tab, cc, f.shift, f.lognb, f.lognc);    \
    bits[k] = grf::fused_value_bits(hi, rr.field<k>());                                                    \
  }
        GRF_STEP(0) GRF_STEP(1) GRF_STEP(2) GRF_STEP(3) GRF_STEP(4) GRF_STEP(5) GRF_STEP(6) GRF_STEP(7)
        GRF_STEP(8) GRF_STEP(9) GRF_STEP(10) GRF_STEP(11) GRF_STEP(12) GRF_STEP(13) GRF_STEP(14) GRF_STEP(15)
#undef GRF_STEP
        if (STORE) {
          uint32_t packed[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) packed[k] = (bits[2 * k] >> 16) | (bits[2 * k + 1] & 0xFFFF0000u);
          uint4 *dst = reinterpret_cast<uint4 *>(out + elem0 + t);
          dst[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
          dst[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
        } else {
#pragma unroll
          for (int m = 0; m < M; ++m) {
            const float *xm = xr + m * P * xpitch + t;
#pragma unroll
            for (int k = 0; k < 16; ++k) acc[m] = fmaf(__uint_as_float(bits[k]), xm[k], acc[m]);
          }
        }
      }
      // the segment must end exactly on the next checkpoint
      if (state != f.seg_state[seg + 1] || g + (ip - ip0) != f.seg_offset[seg + 1]) bad |= GRF_ERR_CHECKPOINT;
    }
  }

  if (!STORE) {
    float *part = reinterpret_cast<float *>(lds + L.part);
    if (r < R) {
#pragma unroll
      for (int m = 0; m < M; ++m) part[(r * P + p) * M + m] = acc[m];
    }
    __syncthreads();
    for (uint32_t i = tid; i < R * M; i += kFusedThreads) {
      const uint32_t rr = i / M, m = i % M;
      const uint32_t orow = f.tile_rows[tile * R + rr];
      if (orow == grf::kNoRow) continue;
      float sum = part[(rr * P) * M + m];
      for (uint32_t q = 1; q < P; ++q) sum += part[(rr * P + q) * M + m];
      if (bias) sum += __uint_as_float((uint32_t)bias[orow] << 16);
      y[(size_t)m * ldy + orow] = round_bf16(sum);
    }
  }
  if (bad) atomicOr(error, (int)bad);
}

int check_frame(const grf_bctx_fused &f, const char *who) {
  auto bad = [&](const char *why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (!f.main_bytes || !f.raw6 || !f.seg_state || !f.seg_offset || !f.tile_rows || !f.tile_class || !f.lut ||
      !f.tab || !f.col_class)
    return bad("null pointer in frame");
  if (!f.rows || !f.cols || !f.n_tiles || !f.n_slabs) return bad("empty geometry");
  if (f.seg_len == 0 || f.seg_len % 16 || (uint64_t)f.seg_len * f.segs_per_row != f.cols)
    return bad("segment length must be a multiple of 16 that divides the row length");
  if (!f.lanes_per_row || !f.rows_per_tile || f.lanes_per_row * f.rows_per_tile > (uint32_t)kFusedThreads)
    return bad("tile does not fit one workgroup");
  if (f.n_slabs != (f.segs_per_row + f.lanes_per_row - 1) / f.lanes_per_row) return bad("slab count mismatch");
  if (f.nc == 0 || f.nc > 16 || (1u << f.lognc) != f.nc) return bad("column class count");
  if (f.shift > 12 || f.lognb != 16 - f.shift) return bad("bucket shift");
  if (f.tabn == 0 || f.tabn > 255) return bad("sparse table size");
  if (f.piece_cap % 16 || f.piece_cap < 32) return bad("piece capacity");
  if ((uint64_t)f.rows * f.cols > 0xFFFFFFFFull) return bad("matrix too large");
  return GRF_OK;
}

template <int M, bool STORE>
int launch(const grf_bctx_fused &f, const uint16_t *x, uint32_t ldx, uint16_t *y, uint32_t ldy,
           const uint16_t *bias, uint16_t *out, int32_t *error, hipStream_t s) {
  const FusedLdsLayout L(f, STORE ? 0 : M);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  auto kernel = fused_walk_kernel<M, STORE>;
  if (L.total > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total);
    if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("LDS attribute: ") + hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kernel, dim3(f.n_tiles), dim3(kFusedThreads), L.total, s, f, x, ldx, y, ldy, bias, out, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused kernel: ") + hipGetErrorString(e));
  return GRF_OK;
}

}  // namespace

extern "C" {

uint32_t grf_bctx_fused_lds_bytes(const grf_bctx_fused *frame, uint32_t m_rows) {
  if (!frame) return 0;
  return FusedLdsLayout(*frame, m_rows).total;
}

int grf_bctx_gemv(const grf_bctx_fused *frame, const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint16_t *y,
                  uint32_t ldy, const uint16_t *bias, int32_t *error, void *hip_stream) {
  if (!frame || !x || !y || !error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv: null argument");
  if (int rc = check_frame(*frame, "grf_bctx_gemv")) return rc;
  if (m_rows < 1 || m_rows > 8) return grf::set_error(GRF_UNSUPPORTED, "grf_bctx_gemv: 1 <= m_rows <= 8");
  if (ldx < frame->cols || ldy < frame->rows) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv: leading dimension");
  hipStream_t s = (hipStream_t)hip_stream;
  const grf_bctx_fused &f = *frame;
  switch (m_rows) {
    case 1: return launch<1, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 2: return launch<2, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 3: return launch<3, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 4: return launch<4, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 5: return launch<5, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 6: return launch<6, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    case 7: return launch<7, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
    default: return launch<8, false>(f, x, ldx, y, ldy, bias, nullptr, error, s);
  }
}

int grf_bctx_fused_decode(const grf_bctx_fused *frame, uint16_t *out, int32_t *error, void *hip_stream) {
  if (!frame || !out || !error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_decode: null argument");
  if (int rc = check_frame(*frame, "grf_bctx_fused_decode")) return rc;
  return launch<1, true>(*frame, nullptr, 0, nullptr, 0, nullptr, out, error, (hipStream_t)hip_stream);
}

}  // extern "C"
