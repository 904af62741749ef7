// Kernels and launchers of the fused sinks, generic over the segment walker: the same
// bodies serve the context codec (grf::SegmentWalk) and the predictive codec (its walker
// in fused_ppcx.hip).  A walker provides prefetch(frame, segment, first element, first
// column), start(piece offset, staged-from offset), decode16(t, S, params, pair[8]) and
// ended_on_checkpoint(frame).
//
// GEMV: reduction order of one output element, fixed for every M and for every tiling:
// the S products of a segment are folded into one fp32 accumulator two columns at a
// time in increasing k (v_dot2c_f32_bf16: acc += w[k]*x[k] + w[k+1]*x[k+1]); the K/S
// segment partials of a row are then added in segment order 0..K/S-1 by one thread
// (slab after slab into a running sum); bias is added in fp32 and the sum is rounded
// to BF16 once.
//
// GEMM, batch invariance (the contract of GS/bi_csrc/bi_gemm.cuh:1-17): output element
// (m, n) is one accumulator fed by a fixed sequence of MFMA operations -- slabs in
// increasing order, inside a slab the 16-column groups in increasing order, inside a
// group the P lane-segments p = 0..P-1 -- whose A operand row is x[m] and whose B
// operand column is W[n].  Neither the number of activation rows, nor the tile a row
// sits in, nor what the other rows hold enters that sequence: every M runs the same
// kernel (M < 16 is padded with zero rows), and more than 128 rows are cut into
// launches of 128, which only repeats the same per-row arithmetic.
#pragma once
#include <hip/hip_runtime.h>

#include <string>

#include "fused_device.h"

namespace grf {
int set_error(int code, const std::string &what);                                          // decode_general.hip
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who);  // fused_gemv.hip

// ---------------------------------------------------------------- GEMV and store sinks

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

template <class Walk, int M, bool STORE>
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
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f)};

  const uint32_t r = tid / P, p = tid % P;
  const uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;
  uint16_t *xs = reinterpret_cast<uint16_t *>(lds + L.xs);
  const uint32_t xpitch = S + grf::kXPad;
  const uint32_t width = P * S;
  float *part = reinterpret_cast<float *>(lds + L.part);      // [R][P][M] partials of one slab
  float *rowsum = reinterpret_cast<float *>(lds + L.rowsum);  // [R][M] running sums
  uint32_t bad = 0;

  // the first slab's byte range is two dependent global reads away (row, then offsets):
  // start them before the tables are copied so that the latencies overlap
  grf::PieceSpan span{0, 0};
  if (row != grf::kNoRow) span.fetch(f, row * f.segs_per_row, min(P, f.segs_per_row));
  grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);
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
    Walk w;
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

template <class Walk, int M, bool STORE>
int launch_walk(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                uint16_t *y,
                uint32_t ldy, const uint16_t *bias, uint16_t *out, int32_t *error, hipStream_t s) {
  const FusedLdsLayout L(f, g, STORE ? 0 : M);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  auto kernel = fused_walk_kernel<Walk, M, STORE>;
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

// y = x W^T (+ bias) for 1..8 activation rows; `who` names the entry point in messages
template <class Walk>
int launch_gemv(const char *who, const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  if (m_rows < 1 || m_rows > 8) return grf::set_error(GRF_UNSUPPORTED, std::string(who) + ": 1 <= m_rows <= 8");
  if (ldx < f.cols || ldy < f.rows || (ldx & 1) || ((uintptr_t)x & 3))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          std::string(who) + ": x must be 4-byte aligned with an even leading dimension");
  switch (m_rows) {
    case 1: return launch_walk<Walk, 1, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 2: return launch_walk<Walk, 2, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 3: return launch_walk<Walk, 3, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 4: return launch_walk<Walk, 4, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 5: return launch_walk<Walk, 5, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 6: return launch_walk<Walk, 6, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 7: return launch_walk<Walk, 7, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    default: return launch_walk<Walk, 8, false>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
  }
}

// ---------------------------------------------------------------- GEMM sink

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr uint32_t kGroup = 16;      // columns decoded between two contractions
constexpr uint32_t kMaxAcc = 4;      // 16x16 output blocks a wave may own
constexpr uint32_t kMaxRowsPerLaunch = 128;
constexpr uint32_t kChunkTiles = 4;  // 16-row activation tiles staged in LDS at a time (64 rows)

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

// MT: 16-row activation tiles per launch (m_rows <= 16*MT)
template <class Walk, int MT>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_gemm_kernel(grf_bctx_fused f, grf_fused_tiling g,
                                                                            const uint16_t *x, uint32_t ldx,
                                                                            uint32_t m_rows, uint16_t *y,
                                                                            uint32_t ldy, const uint16_t *bias,
                                                                            int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  constexpr uint32_t CT = MT < kChunkTiles ? MT : kChunkTiles;  // activation tiles per chunk
  const GemmLdsLayout L(f, g, CT * 16);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x, tile = blockIdx.x;
  const uint32_t P = g.lanes_per_row, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = g.tile_class[tile];
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f)};

  const uint32_t r = tid / P, p = tid % P;
  const uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;
  grf::PieceSpan span{0, 0};  // started before the table copy so that the latencies overlap
  if (row != grf::kNoRow) span.fetch(f, row * f.segs_per_row, min(P, f.segs_per_row));
  grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);

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

  for (uint32_t b = 0; b < g.n_slabs; ++b) {
    __syncthreads();  // previous slab's stream bytes and tiles are no longer read
    const uint32_t first_seg = b * P;
    const uint32_t nseg = min(P, f.segs_per_row - first_seg);
    const uint32_t piece_off = L.stream + r * g.piece_cap;
    const bool active = row != grf::kNoRow && p < nseg;
    const uint32_t seg_base = row != grf::kNoRow ? row * f.segs_per_row + first_seg : 0;
    const uint32_t col0 = (first_seg + p) * S;
    Walk w;
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
      // The same 16 columns of every lane-segment of the activations -> activation tile, 64
      // rows at a time: the tile's size bounds the lanes per row a tiling can have, and an
      // output element's sequence of operations does not depend on the chunking.
      for (uint32_t mc = 0; mc < MT; mc += CT) {
        if (mc) __syncthreads();  // the previous chunk has been consumed
        for (uint32_t c = tid; c < CT * 16 * P * 4; c += nthreads) {
          const uint32_t part = c % 4, pp = (c / 4) % P, ml = c / (4 * P), m = mc * 16 + ml;
          const uint32_t col = (first_seg + pp) * S + t + part * 4;
          uint2 v = make_uint2(0u, 0u);
          if (m < m_rows && pp < nseg) v = *reinterpret_cast<const uint2 *>(x + (size_t)m * ldx + col);
          *reinterpret_cast<uint2 *>(lds + L.xt + ml * L.xt_pitch + pp * 32 + part * 8) = v;
        }
        __syncthreads();
        if (contracts) {
          const uint8_t *brow = lds + L.wt + (nt * 16 + li) * L.wt_pitch + kq * 8;
#pragma unroll
          for (uint32_t j = 0; j < kMaxAcc; ++j) {
            const uint32_t mt = mslot + j * MW;
            if (mt >= mc && mt < mc + CT && mt < MT) {
              const uint8_t *arow = lds + L.xt + ((mt - mc) * 16 + li) * L.xt_pitch + kq * 8;
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

template <class Walk, int MT>
int launch_gemm_rows(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
           uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  const GemmLdsLayout L(f, g, (MT < kChunkTiles ? MT : kChunkTiles) * 16);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused GEMM: LDS demand exceeds 160 KiB");
  const uint32_t nwaves = g.threads / 64, NT = (g.rows_per_tile + 15) / 16;
  if (NT > nwaves) return grf::set_error(GRF_BAD_ARGUMENT, "fused GEMM: more column blocks than waves");
  const uint32_t MW = nwaves / NT;
  if ((MT + MW - 1) / MW > kMaxAcc)
    return grf::set_error(GRF_BAD_ARGUMENT, "fused GEMM: tiling leaves more than 4 row tiles per wave");
  auto kernel = fused_gemm_kernel<Walk, MT>;
  if (L.total > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total);
    if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("LDS attribute: ") + hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(g.threads), L.total, s, f, g, x, ldx, m_rows, y, ldy, bias, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused GEMM: ") + hipGetErrorString(e));
  return GRF_OK;
}

// y = x W^T (+ bias) for any number of activation rows, 128 per launch
template <class Walk>
int launch_gemm(const char *who, const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  if (!m_rows) return GRF_OK;
  if (ldx < f.cols || ldy < f.rows || (ldx & 3) || ((uintptr_t)x & 7))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) +
                                                ": x must be 8-byte aligned with a leading dimension that is a multiple of 4");
  for (uint32_t m0 = 0; m0 < m_rows; m0 += kMaxRowsPerLaunch) {
    const uint32_t m = m_rows - m0 < kMaxRowsPerLaunch ? m_rows - m0 : kMaxRowsPerLaunch;
    const uint16_t *xs = x + (size_t)m0 * ldx;
    uint16_t *ys = y + (size_t)m0 * ldy;
    int rc;
    if (m <= 16) rc = launch_gemm_rows<Walk, 1>(f, g, xs, ldx, m, ys, ldy, bias, error, s);
    else if (m <= 32) rc = launch_gemm_rows<Walk, 2>(f, g, xs, ldx, m, ys, ldy, bias, error, s);
    else if (m <= 64) rc = launch_gemm_rows<Walk, 4>(f, g, xs, ldx, m, ys, ldy, bias, error, s);
    else rc = launch_gemm_rows<Walk, 8>(f, g, xs, ldx, m, ys, ldy, bias, error, s);
    if (rc) return rc;
  }
  return GRF_OK;
}

inline uint32_t gemm_lds_bytes(const grf_bctx_fused &f, const grf_fused_tiling &g, uint32_t m_rows) {
  const uint32_t m = m_rows > kMaxRowsPerLaunch ? kMaxRowsPerLaunch : m_rows;
  const uint32_t mt = m <= 16 ? 1 : m <= 32 ? 2 : 4;  // activations are staged 64 rows at a time
  return GemmLdsLayout(f, g, mt * 16).total;
}

}  // namespace grf
