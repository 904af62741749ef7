// Fused decode-GEMM on the matrix cores: the tile walker's words go to an LDS tile
// 16 columns at a time and are contracted with v_mfma_f32_16x16x16_bf16.
//
// Batch invariance (the contract of GS/bi_csrc/bi_gemm.cuh:1-17): output element
// (m, n) is one accumulator fed by a fixed sequence of MFMA operations -- slabs in
// increasing order, inside a slab the 16-column groups in increasing order, inside a
// group the P lane-segments p = 0..P-1 -- whose A operand row is x[m] and whose B
// operand column is W[n].  Neither the number of activation rows, nor the tile a row
// sits in, nor what the other rows hold enters that sequence: every M runs the same
// kernel (M < 16 is padded with zero rows), and more than 128 rows are cut into
// launches of 128, which only repeats the same per-row arithmetic.
#include <hip/hip_runtime.h>

#include <string>

#include "fused_device.h"

namespace grf {
int set_error(int code, const std::string &what);  // decode_general.hip
}

namespace {

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr uint32_t kGroup = 16;      // columns decoded between two contractions
constexpr uint32_t kMaxAcc = 4;      // 16x16 output blocks a wave may own
constexpr uint32_t kMaxRowsPerLaunch = 128;

// LDS regions of the GEMM kernel.  Word and activation tiles hold, per (row, p), one
// 32-byte run of 16 BF16 values; a row's runs are padded by 8 bytes so that the 16 rows
// an MFMA operand touches fall into different banks.
struct GemmLdsLayout {
  uint32_t blocks, block_pitch, stream, wt, wt_pitch, xt, xt_pitch, total;
  __host__ __device__ GemmLdsLayout(const grf_bctx_fused &f, const grf_fused_tiling &g, uint32_t m16) {
    uint32_t at = 0;
    blocks = at;
    block_pitch = grf::fused_table_bytes(f) + (1u << f.lognb);
    at = grf::align_up(at + f.nc * block_pitch, 16);
    stream = at;
    at = grf::align_up(at + g.rows_per_tile * g.piece_cap, 16);
    wt_pitch = g.lanes_per_row * 32 + 8;
    xt_pitch = wt_pitch;
    wt = at;
    at = grf::align_up(at + grf::align_up(g.rows_per_tile, 16) * wt_pitch, 16);
    xt = at;
    at = grf::align_up(at + m16 * xt_pitch, 16);
    total = at;
  }
};

__device__ __forceinline__ uint16_t round_bf16(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// MT: 16-row activation tiles per launch (m_rows <= 16*MT)
template <int MT>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_gemm_kernel(grf_bctx_fused f, grf_fused_tiling g,
                                                                            const uint16_t *x, uint32_t ldx,
                                                                            uint32_t m_rows, uint16_t *y,
                                                                            uint32_t ldy, const uint16_t *bias,
                                                                            int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const GemmLdsLayout L(f, g, MT * 16);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x, tile = blockIdx.x;
  const uint32_t P = g.lanes_per_row, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = g.tile_class[tile];
  grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f)};

  const uint32_t r = tid / P, p = tid % P;
  const uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;

  // contraction roles: wave -> one 16-column block of the tile (nt) and every MW-th row tile
  const uint32_t wave = tid / 64, lane = tid % 64, nwaves = nthreads / 64;
  const uint32_t NT = (R + 15) / 16;
  const uint32_t MW = nwaves / NT;  // waves per column block (host guarantees >= 1)
  const uint32_t nt = wave % NT, mslot = wave / NT;
  const bool contracts = mslot < MW;
  const uint32_t li = lane % 16, kq = lane / 16;
  float4v acc[kMaxAcc];
#pragma unroll
  for (uint32_t j = 0; j < kMaxAcc; ++j) acc[j] = (float4v){0.f, 0.f, 0.f, 0.f};
  uint32_t bad = 0;

  grf::PieceSpan span{0, 0};
  if (row != grf::kNoRow) span.fetch(f, row * f.segs_per_row, min(P, f.segs_per_row));
  for (uint32_t b = 0; b < g.n_slabs; ++b) {
    __syncthreads();  // previous slab's stream bytes and tiles are no longer read
    const uint32_t first_seg = b * P;
    const uint32_t nseg = min(P, f.segs_per_row - first_seg);
    const uint32_t piece_off = L.stream + r * g.piece_cap;
    const bool active = row != grf::kNoRow && p < nseg;
    const uint32_t seg_base = row != grf::kNoRow ? row * f.segs_per_row + first_seg : 0;
    const uint32_t col0 = (first_seg + p) * S;
    grf::SegmentWalk w;
    uint32_t a0 = 0;
    if (active) w.prefetch(f, seg_base + p, (uint64_t)row * K + col0, col0);
    if (row != grf::kNoRow) {
      a0 = grf::fused_stage_piece(lds, piece_off, f, span, p, P);
      if (b + 1 < g.n_slabs)  // the next slab's byte range, while this one is walked
        span.fetch(f, seg_base + P, min(P, f.segs_per_row - first_seg - P));
    }
    __syncthreads();
    if (active) w.start(piece_off, a0);
    for (uint32_t t = 0; t < S; t += kGroup) {
      if (active) {  // 16 words of this lane's segment -> word tile
        uint32_t pair[8];
        w.decode16(t, S, q, pair);
        uint2 *dst = reinterpret_cast<uint2 *>(lds + L.wt + r * L.wt_pitch + p * 32);
        dst[0] = make_uint2(pair[0], pair[1]);
        dst[1] = make_uint2(pair[2], pair[3]);
        dst[2] = make_uint2(pair[4], pair[5]);
        dst[3] = make_uint2(pair[6], pair[7]);
      }
      // the same 16 columns of every lane-segment of the activations -> activation tile
      for (uint32_t c = tid; c < MT * 16 * P * 4; c += nthreads) {
        const uint32_t part = c % 4, pp = (c / 4) % P, m = c / (4 * P);
        const uint32_t col = (first_seg + pp) * S + t + part * 4;
        uint2 v = make_uint2(0u, 0u);
        if (m < m_rows && pp < nseg) v = *reinterpret_cast<const uint2 *>(x + (size_t)m * ldx + col);
        *reinterpret_cast<uint2 *>(lds + L.xt + m * L.xt_pitch + pp * 32 + part * 8) = v;
      }
      __syncthreads();
      if (contracts) {
        const uint8_t *brow = lds + L.wt + (nt * 16 + li) * L.wt_pitch + kq * 8;
#pragma unroll
        for (uint32_t j = 0; j < kMaxAcc; ++j) {
          const uint32_t mt = mslot + j * MW;
          if (mt < MT) {
            const uint8_t *arow = lds + L.xt + (mt * 16 + li) * L.xt_pitch + kq * 8;
            for (uint32_t pp = 0; pp < nseg; ++pp) {
              const short4v a = *reinterpret_cast<const short4v *>(arow + pp * 32);
              const short4v bb = *reinterpret_cast<const short4v *>(brow + pp * 32);
#if defined(__HIP_DEVICE_COMPILE__)
              acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, bb, acc[j], 0, 0, 0);
#else
              (void)a;
              (void)bb;
#endif
            }
          }
        }
      }
      __syncthreads();  // tiles are overwritten by the next group
    }
    if (active && !w.ended_on_checkpoint(f)) bad |= GRF_ERR_CHECKPOINT;
  }

  if (contracts) {
    const uint32_t n_local = nt * 16 + li;
    const uint32_t orow = n_local < R ? g.tile_rows[tile * R + n_local] : grf::kNoRow;
    if (orow != grf::kNoRow) {
      const float bv = bias ? __uint_as_float((uint32_t)bias[orow] << 16) : 0.f;
#pragma unroll
      for (uint32_t j = 0; j < kMaxAcc; ++j) {
        const uint32_t mt = mslot + j * MW;
        if (mt < MT) {
#pragma unroll
          for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t m = mt * 16 + kq * 4 + i;
            if (m < m_rows) y[(size_t)m * ldy + orow] = round_bf16(acc[j][i] + bv);
          }
        }
      }
    }
  }
  if (bad) atomicOr(error, (int)bad);
}

template <int MT>
int launch(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
           uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  const GemmLdsLayout L(f, g, MT * 16);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "grf_bctx_gemm: LDS demand exceeds 160 KiB");
  const uint32_t nwaves = g.threads / 64, NT = (g.rows_per_tile + 15) / 16;
  if (NT > nwaves) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm: more column blocks than waves");
  const uint32_t MW = nwaves / NT;
  if ((MT + MW - 1) / MW > kMaxAcc)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm: tiling leaves more than 4 row tiles per wave");
  auto kernel = fused_gemm_kernel<MT>;
  if (L.total > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total);
    if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("LDS attribute: ") + hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(g.threads), L.total, s, f, g, x, ldx, m_rows, y, ldy, bias, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("grf_bctx_gemm: ") + hipGetErrorString(e));
  return GRF_OK;
}

}  // namespace

namespace grf {
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who);  // fused_gemv.hip
}

extern "C" {

uint32_t grf_bctx_gemm_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint32_t m_rows) {
  if (!frame || !tiling) return 0;
  const uint32_t m = m_rows > kMaxRowsPerLaunch ? kMaxRowsPerLaunch : m_rows;
  const uint32_t mt = m <= 16 ? 1 : m <= 32 ? 2 : m <= 64 ? 4 : 8;
  return GemmLdsLayout(*frame, *tiling, mt * 16).total;
}

int grf_bctx_gemm(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream) {
  if (!frame || !tiling || !x || !y || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm: null argument");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_gemm")) return rc;
  if (!m_rows) return GRF_OK;
  if (ldx < frame->cols || ldy < frame->rows || (ldx & 3) || ((uintptr_t)x & 7))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          "grf_bctx_gemm: x must be 8-byte aligned with a leading dimension that is a multiple of 4");
  hipStream_t s = (hipStream_t)hip_stream;
  for (uint32_t m0 = 0; m0 < m_rows; m0 += kMaxRowsPerLaunch) {
    const uint32_t m = m_rows - m0 < kMaxRowsPerLaunch ? m_rows - m0 : kMaxRowsPerLaunch;
    const uint16_t *xs = x + (size_t)m0 * ldx;
    uint16_t *ys = y + (size_t)m0 * ldy;
    int rc;
    if (m <= 16) rc = launch<1>(*frame, *tiling, xs, ldx, m, ys, ldy, bias, error, s);
    else if (m <= 32) rc = launch<2>(*frame, *tiling, xs, ldx, m, ys, ldy, bias, error, s);
    else if (m <= 64) rc = launch<4>(*frame, *tiling, xs, ldx, m, ys, ldy, bias, error, s);
    else rc = launch<8>(*frame, *tiling, xs, ldx, m, ys, ldy, bias, error, s);
    if (rc) return rc;
  }
  return GRF_OK;
}

}  // extern "C"
