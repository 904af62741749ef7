// Kernels and launchers of the fused sinks, generic over the segment walker: the same
// bodies serve the context codec (grf::SegmentWalk) and the predictive codec (its walker
// in fused_ppcx.hip).  A walker provides prefetch(frame, segment, first element, first
// column, segment's number in its row, the row's position in the residual order),
// start(piece offset, staged-from offset),
// begin16(t, S) + half<0|1, scan kind>(params, pair[4]) for the two halves of a group of
// 16 symbols (decode16 = all three) and ended_on_checkpoint(frame).
//
// GEMV: reduction order of one output element, fixed for every M: the S products of a
// segment are folded into one fp32 accumulator two columns at a time in increasing k
// (v_dot2c_f32_bf16: acc += w[k]*x[k] + w[k+1]*x[k+1]).  Wave tilings (the GEMV the host
// side uses) then add a row's segment partials as one pairwise tree per aligned block of 64
// segments and the blocks in increasing order, whatever the tiling (fused_wave_body).  Slab
// tilings (kept for experiments) add the K/S segment partials of a row in segment order
// 0..K/S-1 by one thread, slab after slab into a running sum: a different order, so their
// outputs agree with the wave tilings' to rounding, not bit for bit.  Bias is added in fp32
// and the sum is rounded to BF16 once.
//
// GEMM, batch invariance (the contract of GS/bi_csrc/bi_gemm.cuh:1-17): output element
// (m, n) is the sum, in quad order, of one fp32 accumulator per quad of lane-segments;
// each accumulator is fed by a fixed sequence of MFMA operations -- slabs in increasing
// order, inside a slab the 8-column half groups in increasing order, one operation per
// half group over the quad's four segments -- whose A operand row is x[m] and whose B
// operand column is W[n].  Neither the number of activation rows, nor the tile a row
// sits in, nor what the other rows hold enters that sequence: every M runs the same
// tiling (rows up to the next multiple of 16 are zero), and more than 128 rows are cut
// into launches of 128, which only repeats the same per-row arithmetic.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <string>
#include <vector>

#include <type_traits>

#include "fused_device.h"

namespace grf {
int set_error(int code, const std::string &what);                                          // decode_general.hip
// fused_gemv.hip; wave_units: the entry point takes GRF_TILE_WAVES tilings
enum TilingUse { kSlabTiling, kGemvTiling, kGemmTiling };  // what an entry point does with the tiling it is given
// pointers: also refuse null device pointers (a host-side validation has none to give)
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who, TilingUse use = kSlabTiling,
                      bool pointers = true);

// A kernel may ask for more than 64 KiB of dynamic LDS only after its limit has been raised;
// done once per kernel and device (not per launch: it is a driver call, and a launch that
// is being captured into a graph should consist of the launch alone).
template <auto Kernel>
int allow_full_lds() {
  static std::atomic<uint64_t> done{0};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev >= 0 && ((done.load(std::memory_order_relaxed) >> dev) & 1u)) return GRF_OK;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     160 * 1024);
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("LDS attribute: ") + hipGetErrorString(e));
  if (dev >= 0) done.fetch_or(1ull << dev, std::memory_order_relaxed);
  return GRF_OK;
}

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

// What a lane does with the words it decodes: multiply them into M activation rows, store
// them where the row lies in the dense matrix, or store them in the slot the row has in the
// tiling (row tile * R + r of a compact [n_tiles * R][cols] output: a gather of rows).
enum Sink : int { kDot = 0, kStore = 1, kGather = 2 };

// the walker to use for the same frame when its segments have 64 symbols and few enough
// activation rows leave it the registers (itself where there is no such variant)
template <class Walk>
struct ahead_of { using type = Walk; };
template <>
struct ahead_of<grf::SegmentWalk> { using type = grf::SegmentWalkAhead; };
constexpr uint32_t kAheadMaxRows = 4;
// a segment's residuals are 48 bytes, read as three 16-byte vectors
// (a segment's 48 residual bytes are contiguous only in the frame's own order)
// Position of a row in the residual array (grf_bctx_fused.row_pos; the row itself without one).
__device__ __forceinline__ uint32_t row_position(const grf_bctx_fused &f, uint32_t row) {
  return f.row_pos && row != grf::kNoRow ? f.row_pos[row] : row;
}

inline bool reads_ahead(const grf_bctx_fused &f) { return f.seg_len == 64 && !f.raw_interleaved && !((uintptr_t)f.raw6 & 15); }

// One workgroup's walk over tile `tile` of a frame.
template <class Walk, int M, int SINK>
__device__ __forceinline__ void fused_walk_body(uint8_t *lds, const grf_bctx_fused &f, const grf_fused_tiling &g,
                                                const uint16_t *x, uint32_t ldx, uint16_t *y, uint32_t ldy,
                                                const uint16_t *bias, uint16_t *out, int32_t *error, uint32_t tile) {
  constexpr bool STORE = SINK != kDot;
  const FusedLdsLayout L(f, g, STORE ? 0 : M);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
  const uint32_t P = g.lanes_per_row, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = g.tile_class[tile];
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f), f.whole_range};

  const uint32_t r = tid / P, p = tid % P;
  uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;
  if (row >= f.rows) row = grf::kNoRow;  // an empty slot, or a row the matrix does not have
  const uint32_t rpos = row_position(f, row);
  uint16_t *xs = reinterpret_cast<uint16_t *>(lds + L.xs);
  const uint32_t xpitch = S + grf::kXPad;
  const uint32_t width = P * S;
  float *part = reinterpret_cast<float *>(lds + L.part);      // [R][P][M] partials of one slab
  float *rowsum = reinterpret_cast<float *>(lds + L.rowsum);  // [R][M] running sums
  uint32_t bad = 0;

  // the first slab's byte range is two dependent global reads away (row, then offsets):
  // start them before the tables are copied so that the latencies overlap
  grf::PieceSpan span{0, 0};
  if (row != grf::kNoRow) span.fetch(f, row, rpos, 0, min(P, f.segs_per_row));
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
    const uint32_t col0 = (first_seg + p) * S;
    const uint64_t elem0 = (uint64_t)row * K + col0;
    Walk w;
    uint32_t a0 = 0;
    if (walks) w.prefetch(f, grf::fused_seg_slot(f, row, rpos, first_seg + p), (uint32_t)elem0, col0, first_seg + p, rpos);
    if (row != grf::kNoRow) {
      a0 = grf::fused_stage_piece(lds, piece_off, f, span, p, P);
      if (b + 1 < g.n_slabs)  // the next slab's byte range, while this one is walked
        span.fetch(f, row, rpos, first_seg + P, min(P, f.segs_per_row - first_seg - P));
    }
    __syncthreads();
    if (walks) {
      w.start(piece_off, a0);
      const uint16_t *xr = xs + p * xpitch;
      float acc[M];
#pragma unroll
      for (int m = 0; m < M; ++m) acc[m] = 0.f;
      if constexpr (STORE) {
        // a lane keeps two groups of 16 words and stores them as one 64-byte run: a line of
        // the output is then written in two visits, not four (four groups would finish the
        // line at once but cost the registers that keep two workgroups on a compute unit)
        constexpr int kHold = 2;
        const uint64_t at = SINK == kGather ? (uint64_t)(tile * R + r) * K + col0 : elem0;
        w.begin16(0, S);
        for (uint32_t t = 0; t < S; t += 16 * kHold) {
          uint32_t hold[kHold][8];
          const uint32_t groups = min((uint32_t)kHold, (S - t) / 16);
#pragma unroll
          for (int k = 0; k < kHold; ++k)
            if (k < groups) {
              w.template half<0>(q, reinterpret_cast<uint32_t(&)[4]>(hold[k][0]));
              w.template half<1>(q, reinterpret_cast<uint32_t(&)[4]>(hold[k][4]));
              // the loads of the group after this one leave before the stores below: memory
              // operations complete in order, so a wait for a load that followed the stores
              // would wait for them too
              if (t + 16 * (k + 1) < S) w.begin16(t + 16 * (k + 1), S);
            }
          uint4 *dst = reinterpret_cast<uint4 *>(out + at + t);
#pragma unroll
          for (int k = 0; k < kHold; ++k)
            if (k < groups) {
              dst[2 * k] = make_uint4(hold[k][0], hold[k][1], hold[k][2], hold[k][3]);
              dst[2 * k + 1] = make_uint4(hold[k][4], hold[k][5], hold[k][6], hold[k][7]);
            }
        }
      }
      for (uint32_t t = 0; !STORE && t < S; t += 16) {
        uint32_t pair[8];
        w.decode16(t, S, q, pair);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const uint4 *xm = reinterpret_cast<const uint4 *>(xr + m * P * xpitch + t);
          const uint4 xa = xm[0], xb = xm[1];
          const uint32_t xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
          for (int k = 0; k < 8; ++k) acc[m] = dot2_bf16(pair[k], xv[k], acc[m]);
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
      if (orow >= f.rows) continue;  // empty slot or no such row
      float sum = rowsum[i];
      if (bias) sum += __uint_as_float((uint32_t)bias[orow] << 16);
      y[(size_t)m * ldy + orow] = round_bf16(sum);
    }
  }
  if (bad) atomicOr(error, (int)bad);
}

// ---------------------------------------------------------------- GEMV over wave units
//
// GRF_TILE_WAVES: the unit of work is one wave: 64/P rows of the tile by P segments (one
// "slab" of the rows).  A wave copies the stream pieces of its rows itself, reads the
// activations straight from memory (they are small and stay in the caches), walks, and folds
// its rows' segment partials; the waves of a workgroup take the tile's units in turn and
// never wait for each other until the row sums are put together at the end.  What the
// slab-synchronous tiling loses -- every wave waiting for the slowest at two barriers per
// slab, copies that nothing overlaps because the workgroups of a compute unit run in step,
// lanes without a segment -- this one keeps busy: while one wave waits for its bytes the
// others walk.
//
// Reduction order of one output element: the S products of a segment as in the other GEMV;
// the segment partials of a row pairwise, neighbours first, over aligned blocks of 64 segments
// (a segment the row does not have counts as +0.0); the blocks' sums in increasing order;
// bias; one rounding.  A unit does the part of that tree that lies inside its P segments
// (lane distances 1, 2, 4, ...), the tile's last step the rest, so the bits of an output do not
// depend on P, on how rows are dealt to workgroups, on whether the matrix shares its launch
// with others, or on the activation row count (more than two rows run as passes of two).
struct WaveLdsLayout {
  uint32_t blocks, block_pitch, stream, sub, rows, total;
  __host__ __device__ WaveLdsLayout(const grf_bctx_fused &f, const grf_fused_tiling &g, uint32_t m) {
    const uint32_t waves = g.threads / 64, rpw = 64 / g.lanes_per_row;
    blocks = 0;
    block_pitch = grf::fused_table_bytes(f) + (1u << f.lognb);
    stream = grf::align_up(f.nc * block_pitch, 16);                   // [waves][64 / P] row pieces
    sub = grf::align_up(stream + waves * rpw * g.piece_cap, 16);      // [rows_per_tile][n_slabs][m] unit sums
    rows = grf::align_up(sub + g.rows_per_tile * g.n_slabs * m * 4, 16);  // [2][rows_per_tile] the tile's rows, their positions
    total = grf::align_up(rows + g.rows_per_tile * 8, 16);
  }
};

// Bytes of activations (all rows of a pass) above which the wave-unit GEMV numbers its units by
// slab first: half the first-level cache of a compute unit.
constexpr uint32_t kUnitsBySlabBytes = 16 * 1024;

// Product of two numbers below 2^24 whose product is below 2^32 (row and segment indices of a
// wave tiling: check_fused_frame holds rows and columns to that): the 24-bit multiply issues
// at full rate, the 32-bit one at a quarter of it.
__device__ __forceinline__ uint32_t mul24(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umul24(a, b);
#else
  return a * b;
#endif
}

// Sum over the P = 2^logp lanes of a row group, delivered in the group's first lane (other
// lanes end with partial sums).  Pairwise, neighbours first: ((l0 + l1) + (l2 + l3)) + ...; the
// first four levels stay inside a row of sixteen lanes and are lane-permuting adds (no LDS
// round trip), wider groups finish with wave shuffles.
__device__ __forceinline__ float group_sum_to_first_lane(float v, uint32_t logp) {
#if defined(__HIP_DEVICE_COMPILE__)
  auto moved = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF,
                                                                  0xF, false));
  };
  v += moved(v, std::integral_constant<int, 0xB1>{});                 // lanes i ^ 1 (quad permute 1,0,3,2)
  v += moved(v, std::integral_constant<int, 0x4E>{});                 // lanes i ^ 2 (quad permute 2,3,0,1)
  if (logp >= 3) v += moved(v, std::integral_constant<int, 0x141>{});  // mirror within 8: lane 0 takes lane 7's quad sum
  if (logp >= 4) v += moved(v, std::integral_constant<int, 0x140>{});  // mirror within 16: lane 0 takes lane 15's half sum
  if (logp >= 5) v += __shfl_xor(v, 16, 64);
  if (logp >= 6) v += __shfl_xor(v, 32, 64);
#else
  (void)logp;
#endif
  return v;
}

template <class Walk, int M, int SCAN>
__device__ __forceinline__ void fused_wave_body(uint8_t *lds, const grf_bctx_fused &f, const grf_fused_tiling &g,
                                                const uint16_t *x, uint32_t ldx, uint16_t *y, uint32_t ldy,
                                                const uint16_t *bias, int32_t *error, uint32_t tile) {
  const WaveLdsLayout L(f, g, M);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
  const uint32_t lane = tid % 64, nwaves = nthreads / 64;
#if defined(__HIP_DEVICE_COMPILE__)
  // the wave's number, told to the compiler as the scalar it is: the unit loop's counters
  // and branches then live in scalar registers
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
#else
  const uint32_t wave = tid / 64;
#endif
  const uint32_t P = g.lanes_per_row, rpw = 64 / P, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t cls = g.tile_class[tile];
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f), f.whole_range};
  const bool tables_by_dma = grf::fused_tables_by_dma(f);
  if (tables_by_dma) grf::fused_load_tables_dma(lds, L.blocks, L.block_pitch, f, cls, wave, nwaves, lane);
  // P is a power of two: lane coordinates by shift and mask.  A unit is (row group grp, slab b),
  // numbered u = grp * n_slabs + b or, for long rows, u = b * groups + grp; a wave steps through
  // its units u = wave, wave + nwaves, ... by adding (nwaves / n, nwaves % n) to the pair with a
  // carry, in scalar registers: divisions by values only known at run time cost some twenty
  // vector instructions each, and there were six of them per unit.
  // Which numbering: the waves of a compute unit work on neighbouring units, and every lane
  // reads its segment's 128 bytes of x in eight visits.  Numbered by row group first, twelve
  // waves are spread over every slab of the row, and once x outgrows the 32 KiB first-level
  // cache those lines come from the L2 again on most visits; numbered by slab first they share
  // two or three slabs' worth of x (5120 x 17408: 71 -> 65 us).  Short rows keep the first
  // numbering, where neighbouring waves also share the lines at the ends of their stream pieces.
  const uint32_t logp = 31 - __builtin_clz(P);
  const uint32_t rl = lane >> logp, p = lane & (P - 1);
  float *sub = reinterpret_cast<float *>(lds + L.sub);
  uint32_t *rows = reinterpret_cast<uint32_t *>(lds + L.rows);
  const uint32_t piece_off = L.stream + (wave * rpw + rl) * g.piece_cap;
  // The tile's real height: the slots up to its last row.  A tile with fewer rows than R --
  // the tail of a row class, or a tiling that gives the tiles of a small class fewer rows --
  // has that many row groups fewer to walk (its empty slots, kNoRow, are at the end).
  uint32_t r_real = 0;
  for (uint32_t i0 = 0; i0 < R; i0 += 64) {  // uniform
    const uint32_t i = i0 + lane;
    const uint64_t has = __ballot(i < R && g.tile_rows[tile * R + min(i, R - 1)] < f.rows);
    if (has) r_real = i0 + 64 - (uint32_t)__builtin_clzll(has);
  }
  const uint32_t groups = (r_real + rpw - 1) / rpw, units = groups * g.n_slabs;
  const bool by_slab = K * 2u * M > kUnitsBySlabBytes;
  const uint32_t n_minor = max(1u, by_slab ? groups : g.n_slabs);
  const uint32_t step_major = nwaves / n_minor, step_minor = nwaves % n_minor;
  uint32_t bad = 0;

  // The byte range [g0, g1) of a unit's row piece is the first of two dependent reads before
  // the piece can be copied, so it is read one unit ahead (and the first one before the
  // tables are copied).
  // (Loads in a branch that only some lanes take make the compiler wait for every load in
  // flight where the branch ends, so lanes without a row read the matrix's first entries and
  // discard them.)
  const uint32_t seg_step = grf::fused_seg_step(f);
  auto span_of = [&](uint32_t b, uint32_t row, uint32_t rpos, uint32_t &g0, uint32_t &g1) {
    const bool any = row != grf::kNoRow;
    const uint32_t first_seg = any ? b << logp : 0;
    const uint32_t slot = grf::fused_seg_slot<true>(f, any ? row : 0, any ? rpos : 0, first_seg);
    const uint32_t past = any ? min(P, f.segs_per_row - first_seg) : 0;
    g0 = grf::fused_index_entry(f.seg_offset, slot);
    g1 = grf::fused_index_entry(f.seg_offset, slot + mul24(past, seg_step));  // (no row: an empty range)
  };
  auto advance = [&](uint32_t &grp, uint32_t &b) {  // the unit nwaves further on
    uint32_t &major = by_slab ? b : grp, &minor = by_slab ? grp : b;
    major += step_major;
    minor += step_minor;
    if (minor >= n_minor) minor -= n_minor, ++major;
  };
  uint32_t grp = by_slab ? wave % n_minor : wave / n_minor, b = by_slab ? wave / n_minor : wave % n_minor;  // the first unit
  uint32_t row, rpos, g0, g1;
  {
    const uint32_t slot0 = grp * rpw + rl;
    row = (wave < units && slot0 < R) ? g.tile_rows[tile * R + slot0] : grf::kNoRow;
    if (row >= f.rows) row = grf::kNoRow;  // an empty slot, or a row the matrix does not have
    rpos = row_position(f, row);
    span_of(b, row, rpos, g0, g1);
  }
  for (uint32_t i = tid; i < R; i += nthreads) {
    uint32_t rw = g.tile_rows[tile * R + i];
    if (rw >= f.rows) rw = grf::kNoRow;
    rows[i] = rw;
    rows[R + i] = row_position(f, rw);
  }
  if (!tables_by_dma) grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the tables' copy has landed)
#endif
  __syncthreads();
  const uint32_t later_half = blockIdx.x >= gridDim.x / 2 ? 1u : 0u;
  uint32_t left = wave < units ? (units - 1 - wave) / nwaves : 0;  // units after the current one
  for (uint32_t u = wave; u < units; u += nwaves, --left) {  // wave-uniform
#if defined(__HIP_DEVICE_COMPILE__)
    // Waves with more units still to do go first.  Left alone the arbiter prefers the older
    // of the two workgroups that share a compute unit, which then finishes long before the
    // other and leaves it the unit at half occupancy.
    // Between walks a wave has a hundred-odd instructions to issue (row sums, addresses, the
    // loads of the next unit), each waiting on the one before; at the walking waves' priority
    // it got a turn so rarely that this took 3 us per unit.  It goes first, and back to its
    // walking priority when the walk starts.
    __builtin_amdgcn_s_setprio(3);
#endif
    const uint32_t slot = grp * rpw + rl;
    const uint32_t first_seg = b << logp;
    const uint32_t nseg = min(P, f.segs_per_row - first_seg);
    if (u != wave) {  // (read again: cheaper than registers over the walk)
      row = slot < R ? rows[slot] : grf::kNoRow;
      rpos = slot < R ? rows[R + slot] : 0;
    }
    const bool walks = row != grf::kNoRow && p < nseg;
    const uint32_t col0 = mul24(first_seg + p, S);
    // The copy of the pieces goes first: its byte ranges arrived during the walk before, while
    // a wait for them placed after this unit's other loads would wait for those as well.
    const uint32_t a0 = grf::fused_stage_piece_dma(lds, L.stream + wave * rpw * g.piece_cap, g.piece_cap, f, g0, g1, lane, logp, rpw);
    Walk w;
    {  // every lane loads (see span_of); lanes that do not walk read segment 0's entries
      const uint32_t seg = grf::fused_seg_slot<true>(f, walks ? row : 0, walks ? rpos : 0, walks ? first_seg + p : 0);
      w.prefetch(f, seg, walks ? mul24(row, K) + col0 : 0, walks ? col0 : 0, walks ? first_seg + p : 0, walks ? rpos : 0);
    }
    if (walks) w.start(piece_off, a0);
    const uint32_t slot_base = grp * rpw, slab = b;  // this unit's, kept while the counters move on
    {  // the next unit's byte range, on its way during this unit's walk
      advance(grp, b);
      const uint32_t sn = grp * rpw + rl;
      const bool more = u + nwaves < units && sn < R;
      span_of(b, more ? rows[sn] : grf::kNoRow, more ? rows[R + sn] : 0, g0, g1);
    }
    __builtin_amdgcn_wave_barrier();
#if defined(__HIP_DEVICE_COMPILE__)
    switch (min(3u, left + later_half)) {  // + the later-started half
      case 0: __builtin_amdgcn_s_setprio(0); break;
      case 1: __builtin_amdgcn_s_setprio(1); break;
      case 2: __builtin_amdgcn_s_setprio(2); break;
      default: __builtin_amdgcn_s_setprio(3); break;
    }
#endif
    float acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m) acc[m] = 0.f;
    if (walks) {
      // The activations are read eight columns (16 bytes per row) at a time, each load issued
      // while the eight symbols before it are decoded: two register sets, one for the first and
      // one for the second half of a group of 16, so nothing is copied between them.
      uint4 xa[M], xb[M];
      auto load_x = [&](uint4 (&xs)[M], uint32_t t) {  // (uniform base, 32-bit lane offset in bytes)
#pragma unroll
        for (int m = 0; m < M; ++m)
          xs[m] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint8_t *>(x) + ((uint32_t)m * ldx + col0 + t) * 2u);
      };
      auto contract = [&](const uint32_t (&pair)[4], const uint4 (&xs)[M]) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
          acc[m] = dot2_bf16(pair[0], xs[m].x, acc[m]);
          acc[m] = dot2_bf16(pair[1], xs[m].y, acc[m]);
          acc[m] = dot2_bf16(pair[2], xs[m].z, acc[m]);
          acc[m] = dot2_bf16(pair[3], xs[m].w, acc[m]);
        }
      };
      load_x(xa, 0);
      auto group = [&](uint32_t t) {
        uint32_t pair[4];
        load_x(xb, t + 8);
        w.begin16(t, S);
        w.template half<0, SCAN>(q, pair);
        contract(pair, xa);
        load_x(xa, min(t + 16, S - 8));  // the last group loads a half again rather than branch around the load
        w.template half<1, SCAN>(q, pair);
        contract(pair, xb);
      };
      // two groups per trip: the registers that carry the next group's residuals, classes and
      // activations then change roles twice and end where they began, without copies
      for (uint32_t t = 0; t < S; t += 32) {
        group(t);
        if (t + 16 < S) group(t + 16);
      }
      if (!w.ended_on_checkpoint(f)) bad |= GRF_ERR_CHECKPOINT;
    }
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_setprio(3);
#endif
    // The unit's sum of a row: its P segment partials (0 for lanes without a segment) added
    // pairwise, neighbours first -- lane distances 1, 2, 4, ...
    {
      // (the lane's coordinates are worked out again rather than kept in registers over the walk)
      uint32_t ln = __lane_id();
#if defined(__HIP_DEVICE_COMPILE__)
      asm volatile("" : "+v"(ln));
#endif
      const uint32_t p2 = ln & (P - 1), rl2 = ln >> logp;
      const uint32_t slot2 = slot_base + rl2;
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float sum = group_sum_to_first_lane(acc[m], logp);
        if (p2 == 0 && slot2 < R) sub[(slot2 * g.n_slabs + slab) * M + m] = sum;
      }
    }
  }
  __syncthreads();
  // A row's unit sums -> its output.  The order is the same for every tiling: the tree that a
  // unit began over its P segments is carried on over aligned blocks of 64 segments (64 / P
  // unit sums, pairwise, neighbours first; a unit the row does not have counts as +0.0, like
  // the lanes without a segment inside a unit), and the blocks' sums are added in
  // increasing order.
  const uint32_t per_block = 64u >> logp;  // unit sums of a row per block of 64 segments: 1..16
  for (uint32_t i = tid; i < R * M; i += nthreads) {
    const uint32_t rr = i / M, m = i % M;
    const uint32_t orow = rows[rr];
    if (orow == grf::kNoRow) continue;
    const float *sp = sub + (rr * g.n_slabs) * M + m;
    float sum = 0.f;
    for (uint32_t b0 = 0; b0 < g.n_slabs; b0 += per_block) {
      float v[16];
#pragma unroll
      for (uint32_t k = 0; k < 16; ++k) v[k] = (k < per_block && b0 + k < g.n_slabs) ? sp[(b0 + k) * M] : 0.f;
#pragma unroll
      for (uint32_t w = 1; w < 16; w <<= 1)
#pragma unroll
        for (uint32_t k = 0; k < 16; k += 2 * w)
          if (w < per_block) v[k] += v[k + w];
      sum = b0 ? sum + v[0] : v[0];
    }
    if (bias) sum += __uint_as_float((uint32_t)bias[orow] << 16);
    y[(size_t)m * ldy + orow] = round_bf16(sum);
  }
  if (bad) atomicOr(error, (int)bad);
}

// SCAN: the scan the step carries for lanes whose lookup byte names a neighbour of their symbol
// (grf::ScanKind); the launch picks the short one for frames without whole-range contexts.  (A
// choice inside the kernel was tried: after every symbol the two scans' registers have to be
// brought together again, which cost more than the short scan saves.)
template <class Walk, int M, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) __attribute__((amdgpu_waves_per_eu(6))) void fused_wave_kernel(
    grf_bctx_fused f, grf_fused_tiling g, const uint16_t *x, uint32_t ldx, uint16_t *y, uint32_t ldy,
    const uint16_t *bias, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  fused_wave_body<Walk, M, SCAN>(lds, f, g, x, ldx, y, ldy, bias, error, blockIdx.x);
}

template <class Walk, int M, int SCAN>
int launch_wave_scan(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint16_t *y,
                     uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  const WaveLdsLayout L(f, g, M);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  constexpr auto kernel = &fused_wave_kernel<Walk, M, SCAN>;
  if (L.total > 64 * 1024)
    if (int rc = allow_full_lds<kernel>()) return rc;
  hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(g.threads), L.total, s, f, g, x, ldx, y, ldy, bias, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused kernel: ") + hipGetErrorString(e));
  return GRF_OK;
}

template <class Walk, int M>
int launch_wave(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint16_t *y,
                uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  return f.whole_range ? launch_wave_scan<Walk, M, grf::kScanAny>(f, g, x, ldx, y, ldy, bias, error, s)
                       : launch_wave_scan<Walk, M, grf::kScanNoWholeRange>(f, g, x, ldx, y, ldy, bias, error, s);
}

// The wave-unit GEMV keeps the activations of a group of columns in registers: two rows per
// pass.  More rows run as further passes over the matrix with exactly the same arithmetic per
// row; batches beyond two belong to the matrix-core GEMM anyway.
constexpr uint32_t kWaveRowsPerPass = 2;

inline int check_wave_operands(const char *who, const grf_bctx_fused &f, const uint16_t *x, uint32_t ldx) {
  if (ldx > (1u << 29))  // the kernel addresses x with 32-bit byte offsets
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": leading dimension of x too large");
  if ((ldx & 7) || ((uintptr_t)x & 15))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          std::string(who) + ": wave units read x in 16-byte vectors (aligned, ldx a multiple of 8)");
  if (f.seg_len % 16 || f.cols % 16) return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": segment length");
  return GRF_OK;
}

template <class Walk>
int launch_wave_rows(const char *who, const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                     uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error, hipStream_t s) {
  if (int rc = check_wave_operands(who, f, x, ldx)) return rc;
  for (uint32_t m0 = 0; m0 < m_rows; m0 += kWaveRowsPerPass) {
    const uint16_t *xs = x + (size_t)m0 * ldx;
    uint16_t *ys = y + (size_t)m0 * ldy;
    const int rc = m_rows - m0 == 1 ? launch_wave<Walk, 1>(f, g, xs, ldx, ys, ldy, bias, error, s)
                                    : launch_wave<Walk, 2>(f, g, xs, ldx, ys, ldy, bias, error, s);
    if (rc) return rc;
  }
  return GRF_OK;
}


// Six waves per SIMD keep two 768-lane workgroups on a compute unit: the store sinks, which
// hold decoded words back, would otherwise take a few registers too many for that.
template <class Walk, int M, int SINK>
__global__ __launch_bounds__(grf::kFusedMaxThreads) __attribute__((amdgpu_waves_per_eu(6))) void fused_walk_kernel(grf_bctx_fused f, grf_fused_tiling g,
                                                                            const uint16_t *x, uint32_t ldx,
                                                                            uint16_t *y, uint32_t ldy,
                                                                            const uint16_t *bias, uint16_t *out,
                                                                            int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  fused_walk_body<Walk, M, SINK>(lds, f, g, x, ldx, y, ldy, bias, out, error, blockIdx.x);
}

// Several frames of one width in one launch (q/k/v, gate/up): the grid is the tiles of the
// members one after the other, every member with its own tiling, output and bias.  The
// tilings share one thread count; a member's rows see exactly the arithmetic of a launch of
// their own with that tiling.
constexpr uint32_t kMaxGroup = 4;
struct FusedGroup {
  grf_bctx_fused f[kMaxGroup];
  grf_fused_tiling g[kMaxGroup];
  uint16_t *y[kMaxGroup];
  const uint16_t *bias[kMaxGroup];
  uint32_t ldy[kMaxGroup];
  uint32_t first_tile[kMaxGroup + 1];  // first_tile[n] = tiles of the whole launch
  uint32_t n;
};

__device__ __forceinline__ uint32_t group_member(const FusedGroup &a, uint32_t block) {
  uint32_t i = 0;
#pragma unroll
  for (uint32_t k = 1; k < kMaxGroup; ++k)
    if (k < a.n && block >= a.first_tile[k]) i = k;
  return i;
}

template <class Walk, int M>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_walk_group_kernel(FusedGroup a, const uint16_t *x,
                                                                                  uint32_t ldx, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t i = group_member(a, blockIdx.x);
  fused_walk_body<Walk, M, kDot>(lds, a.f[i], a.g[i], x, ldx, a.y[i], a.ldy[i], a.bias[i], nullptr, error,
                                 blockIdx.x - a.first_tile[i]);
}

template <class Walk, int M, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) __attribute__((amdgpu_waves_per_eu(6))) void fused_wave_group_kernel(
    FusedGroup a, const uint16_t *x, uint32_t ldx, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t i = group_member(a, blockIdx.x);
  fused_wave_body<Walk, M, SCAN>(lds, a.f[i], a.g[i], x, ldx, a.y[i], a.ldy[i], a.bias[i], error,
                                 blockIdx.x - a.first_tile[i]);
}

template <class Walk, int M, int SINK>
int launch_walk(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                uint16_t *y,
                uint32_t ldy, const uint16_t *bias, uint16_t *out, int32_t *error, hipStream_t s) {
  const FusedLdsLayout L(f, g, SINK != kDot ? 0 : M);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  constexpr auto kernel = &fused_walk_kernel<Walk, M, SINK>;
  if (L.total > 64 * 1024)
    if (int rc = allow_full_lds<kernel>()) return rc;
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
  using Ahead = typename ahead_of<Walk>::type;
  if (g.scheme == GRF_TILE_WAVES) return launch_wave_rows<Walk>(who, f, g, x, ldx, m_rows, y, ldy, bias, error, s);
  if (!std::is_same<Ahead, Walk>::value && reads_ahead(f) && m_rows <= kAheadMaxRows) switch (m_rows) {
      case 1: return launch_walk<Ahead, 1, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
      case 2: return launch_walk<Ahead, 2, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
      case 3: return launch_walk<Ahead, 3, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
      default: return launch_walk<Ahead, 4, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    }
  switch (m_rows) {
    case 1: return launch_walk<Walk, 1, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 2: return launch_walk<Walk, 2, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 3: return launch_walk<Walk, 3, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 4: return launch_walk<Walk, 4, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 5: return launch_walk<Walk, 5, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 6: return launch_walk<Walk, 6, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    case 7: return launch_walk<Walk, 7, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
    default: return launch_walk<Walk, 8, kDot>(f, g, x, ldx, y, ldy, bias, nullptr, error, s);
  }
}

// ---------------------------------------------------------------- GEMM sink
//
// Nothing decoded ever leaves the registers.  A wave covers 16 rows of the tile and four
// lane-segments: lane l walks segment 4*quad + l/16 of row 16*block + l%16, and the eight
// words a lane decodes in half a group are, as they stand, its share of the B operand of
// v_mfma_f32_16x16x32_bf16 (column l%16, k-slots 8*(l/16)..+7).  The k-slots of one MFMA
// are therefore 8 consecutive columns out of each of four different segments; the A
// operand pairs them with the same columns of 16 activation rows, read with one 16-byte
// load per lane from a copy of the activations laid out for exactly that (column chunk
// major, see pack_activations_kernel).  No workgroup barrier inside a slab, no tile in LDS.
//
// At the end the waves of a row block (one per quad) hold partial sums over their
// segments; they are added through LDS in quad order.

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr uint32_t kMaxRowsPerLaunch = 128;  // eight 16-row activation tiles per launch
constexpr uint32_t kSumTiles = 4;            // tiles whose partial sums pass through LDS at a time

// Workgroup shape of the GEMM kernel for a tiling: row blocks x quads of lane-segments.
struct GemmShape {
  uint32_t row_blocks, quads, threads;
  __host__ __device__ explicit GemmShape(const grf_fused_tiling &g) {
    row_blocks = (g.rows_per_tile + 15) / 16;
    quads = (g.lanes_per_row + 3) / 4;
    threads = row_blocks * quads * 64;
  }
};

// Tables, then for every wave the pieces of its sixteen rows (piece_cap: the capacity of a
// piece of four segments); the same memory later holds the partial sums of every wave (1 KiB
// per wave and activation tile).
struct GemmLdsLayout {
  uint32_t blocks, block_pitch, stream, total;
  __host__ __device__ GemmLdsLayout(const grf_bctx_fused &f, const grf_fused_tiling &g) {
    blocks = 0;
    block_pitch = grf::fused_table_bytes(f) + (1u << f.lognb);
    stream = grf::align_up(f.nc * block_pitch, 16);
    const uint32_t waves = GemmShape(g).threads / 64;
    total = grf::align_up(stream + waves * 16 * g.piece_cap, 16);
    const uint32_t sums = waves * kSumTiles * 1024;
    if (total < sums) total = sums;
  }
};

// Activations in operand order: the 8 columns [8c, 8c+8) of row m at xp[c * m_pad + m]
// (16 bytes); rows m_rows..m_pad-1 are zero, and so is one more chunk after the last.  A
// group of 64 threads moves 8 chunks of 8 rows, reading 128-byte runs of x and writing
// 128-byte runs of xp.
static __global__ __launch_bounds__(256) void pack_activations_kernel(const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                                                                uint32_t m_pad, uint32_t chunks, uint4 *xp) {
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t cc = idx % 8, ml = (idx / 8) % 8, blk = idx / 64;
  const uint32_t m_blocks = m_pad / 8;
  const uint32_t m = (blk % m_blocks) * 8 + ml, c = (blk / m_blocks) * 8 + cc;
  if (c > chunks) return;
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (m < m_rows && c < chunks) {
    const uint2 *src = reinterpret_cast<const uint2 *>(x + (size_t)m * ldx + c * 8);
    const uint2 a = src[0], b = src[1];
    v = make_uint4(a.x, a.y, b.x, b.y);
  }
  xp[(size_t)c * m_pad + m] = v;
}

inline uint32_t gemm_tiles(uint32_t m_rows) { return m_rows <= 16 ? 1 : m_rows <= 32 ? 2 : m_rows <= 64 ? 4 : 8; }

inline void launch_pack(const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint32_t cols, uint32_t m_pad, uint4 *xp,
                        hipStream_t s) {
  const uint32_t chunks = cols / 8;
  const uint32_t pack_threads = (chunks + 1 + 7) / 8 * 8 * m_pad;  // the chunks and the chunk of zeros after them
  hipLaunchKernelGGL(pack_activations_kernel, dim3((pack_threads + 255) / 256), dim3(256), 0, s, x, ldx, m_rows, m_pad,
                     chunks, xp);
}

// The lane's A operands of one half group: tile j of the packed activations at byte offset
// `at` + 256 j of `xp`.  Up to four tiles: a uniform base and a 32-bit lane offset (the packed
// copy is a few MB), which keeps a 64-bit address out of the registers that the walk needs;
// with eight tiles the compiler does better with the address.
template <int MT>
__device__ __forceinline__ void gemm_load_x(uint4 (&xa)[MT], const uint4 *xp, uint32_t at) {
  const uint8_t *base = reinterpret_cast<const uint8_t *>(xp);
  if constexpr (MT <= 4) {
#pragma unroll
    for (int j = 0; j < MT; ++j) xa[j] = *reinterpret_cast<const uint4 *>(base + (at + (uint32_t)j * 256u));
  } else {
    const uint4 *xl = reinterpret_cast<const uint4 *>(base + (size_t)at);
#pragma unroll
    for (int j = 0; j < MT; ++j) xa[j] = xl[j * 16];
  }
}

template <int MT>
__device__ __forceinline__ void gemm_contract(float4v (&acc)[MT], const uint4 (&xa)[MT], const uint32_t (&w)[4]) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint4 wv = make_uint4(w[0], w[1], w[2], w[3]);
  const bf16x8_t b = __builtin_bit_cast(bf16x8_t, wv);
#pragma unroll
  for (int j = 0; j < MT; ++j)
    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[j]), b, acc[j], 0, 0, 0);
#else
  (void)acc;
  (void)xa;
  (void)w;
#endif
}

// MT: 16-row activation tiles of this launch (m_rows <= 16 * MT, xp packed with m_pad = 16 * MT)
// With g.k_parts > 1 the launch's tiles are k_parts copies of the row tiles, part-major: copy
// `part` walks the slabs [part * spp, (part + 1) * spp) with spp = ceil(n_slabs / k_parts) and
// leaves its sums as fp32 in `partials` [k_parts][m_rows][rows]; gemm_sum_parts_kernel adds the
// parts in order, then the bias, and rounds.  That lets a matrix with few rows be cut along K
// until its tiles fill the machine with full blocks of sixteen rows, in a fixed order of
// additions (the tiling is the matrix's, whatever the batch).
template <class Walk, int MT, int SCAN>
__device__ __forceinline__ void fused_gemm_body(uint8_t *lds, const grf_bctx_fused &f, const grf_fused_tiling &g,
                                                const uint4 *xp, uint32_t m_rows, uint16_t *y, uint32_t ldy,
                                                const uint16_t *bias, float *partials, int32_t *error,
                                                uint32_t launch_tile) {
  const GemmLdsLayout L(f, g);
  const GemmShape shape(g);
  const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
  const uint32_t P = g.lanes_per_row, R = g.rows_per_tile, S = f.seg_len, K = f.cols;
  const uint32_t parts = g.k_parts > 1 ? g.k_parts : 1u, row_tiles = g.n_tiles / parts;
  // (uniform: scalar divisions.  Part-major: with a tile's copies side by side instead, the same
  // launch at six rows took 5 % longer on 5120 x 17408 cut in three)
  const uint32_t part = launch_tile / row_tiles, tile = launch_tile - part * row_tiles;
  const uint32_t per_part = (g.n_slabs + parts - 1) / parts;
  const uint32_t b_first = part * per_part, b_past = min(g.n_slabs, b_first + per_part);
  const uint32_t cls = g.tile_class[tile];
  const grf::FusedParams q{f.shift, L.block_pitch, grf::fused_table_bytes(f), f.whole_range};
  constexpr uint32_t m_pad = MT * 16;

  const uint32_t lane = tid % 64;
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);  // (a scalar: the loop below branches on it)
#else
  const uint32_t wave = tid / 64;
#endif
  // (the tables' copy first: it is under way while the reads below follow one another)
  const bool tables_by_dma = grf::fused_tables_by_dma(f);
  if (tables_by_dma) grf::fused_load_tables_dma(lds, L.blocks, L.block_pitch, f, cls, wave, nthreads / 64, lane);
  const uint32_t rb = wave % shape.row_blocks, quad = wave / shape.row_blocks;
  const uint32_t r = rb * 16 + lane % 16, p4 = lane / 16;
  uint32_t row = r < R ? g.tile_rows[tile * R + r] : grf::kNoRow;
  if (row >= f.rows) row = grf::kNoRow;  // an empty slot, or a row the matrix does not have
  const uint32_t rpos = row_position(f, row);

  // A wave keeps its sixteen rows and its quad of lane-segments for the whole launch and goes
  // through the slabs on its own: in slab b it walks segments b * P + 4 * quad .. + 3 of every
  // row.  It copies the rows' pieces of those four segments to its own part of the LDS (the
  // loads write the LDS directly, one row per instruction), so the waves of a workgroup share
  // the tables and nothing else until their partial sums meet at the end.
  const uint32_t region = L.stream + wave * 16 * g.piece_cap;
  const uint32_t piece_off = region + (lane % 16) * g.piece_cap;
  // byte range of the lane's row piece in a slab; lanes without a row, and slabs past the row's
  // end, read the matrix's first entry and get an empty range (no load sits in a branch)
  auto span_of = [&](uint32_t b, uint32_t &g0, uint32_t &g1) {
    const uint32_t first = b * P + quad * 4;
    const bool any = row != grf::kNoRow && first < f.segs_per_row && quad * 4 < P;
    const uint32_t slot = grf::fused_seg_slot<true>(f, any ? row : 0, any ? rpos : 0, any ? first : 0);
    const uint32_t past = any ? min(4u, min(P - quad * 4, f.segs_per_row - first)) : 0;
    g0 = grf::fused_index_entry(f.seg_offset, slot);
    g1 = grf::fused_index_entry(f.seg_offset, slot + mul24(past, grf::fused_seg_step(f)));
  };
  uint32_t g0, g1;
  span_of(b_first, g0, g1);  // started before the table copy so that the latencies overlap
  if (!tables_by_dma) grf::fused_load_tables(lds, L.blocks, L.block_pitch, f, cls, tid, nthreads);

  float4v acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = (float4v){0.f, 0.f, 0.f, 0.f};
  uint32_t bad = 0;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the tables' copy has landed)
#endif
  __syncthreads();  // the tables are in place
  const uint32_t later_half = blockIdx.x >= gridDim.x / 2 ? 1u : 0u;

  for (uint32_t b = b_first; b < b_past; ++b) {
    const uint32_t first_seg = b * P + quad * 4;
    if (first_seg >= f.segs_per_row || quad * 4 >= P) break;  // uniform: this wave's quad has no segment from here on
    const uint32_t nseg = min(4u, min(P - quad * 4, f.segs_per_row - first_seg));
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_setprio(3);  // between walks a wave's few instructions go first
#endif
    const bool active = row != grf::kNoRow && p4 < nseg;
    const uint32_t col0 = mul24(first_seg + p4, S);
    // the pieces first: their ranges arrived during the walk before
    const uint32_t a0 = grf::fused_stage_piece_dma(lds, region, g.piece_cap, f, g0, g1, lane, 0, 16);
    Walk w;
    {
      const uint32_t seg = grf::fused_seg_slot<true>(f, active ? row : 0, active ? rpos : 0, active ? first_seg + p4 : 0);
      w.prefetch(f, seg, active ? mul24(row, K) + col0 : 0, active ? col0 : 0, active ? first_seg + p4 : 0, active ? rpos : 0);
    }
    if (active) w.start(piece_off, a0);  // (a0: of the lane's own row, which its four lanes share)
    span_of(b + 1, g0, g1);  // the next slab's byte range, on its way during this walk
    __builtin_amdgcn_wave_barrier();
#if defined(__HIP_DEVICE_COMPILE__)
    // walking priority as in the GEMV: the slabs still to do, + 1 for the later-started half of
    // the grid (left alone, the older of the two workgroups on a compute unit runs ahead and
    // leaves the other the unit at half occupancy)
    switch (min(3u, (b_past - 1 - b) + later_half)) {
      case 0: __builtin_amdgcn_s_setprio(0); break;
      case 1: __builtin_amdgcn_s_setprio(1); break;
      case 2: __builtin_amdgcn_s_setprio(2); break;
      default: __builtin_amdgcn_s_setprio(3); break;
    }
#endif
    if (__ballot(active) == 0) continue;  // nothing to walk in this wave (the branch is per wave)
    // A lane's k-slots are real columns when its segment exists, whether or not its own
    // row does; other lanes feed zeros (their weights are zero too, but 0 * NaN is not):
    // they read the chunk of zeros that ends the packed copy and never move on.  The load
    // after a segment's last half group reads the chunk that follows it, at most that one.
    const bool feeds = p4 < nseg;
    const uint32_t x_step = feeds ? m_pad * 16 : 0;  // bytes from one 8-column chunk to the next
    // (the lane's number is worked out again here rather than kept in a register over the walks)
    uint32_t ln = __lane_id();
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(ln));
#endif
    uint32_t xl = ((feeds ? col0 / 8 : K / 8) * m_pad + ln % 16) * 16;
    uint4 xa[MT];
    gemm_load_x<MT>(xa, xp, xl);
    for (uint32_t t = 0; t < S; t += 16) {
      uint32_t lo[4] = {0u, 0u, 0u, 0u}, hi[4] = {0u, 0u, 0u, 0u};
      if (active) {
        w.begin16(t, S);
        w.template half<0, SCAN>(q, lo);
      }
      gemm_contract<MT>(acc, xa, lo);
      xl += x_step;
      gemm_load_x<MT>(xa, xp, xl);
      if (active) w.template half<1, SCAN>(q, hi);
      gemm_contract<MT>(acc, xa, hi);
      xl += x_step;
      gemm_load_x<MT>(xa, xp, xl);
    }
    if (active && !w.ended_on_checkpoint(f)) bad |= GRF_ERR_CHECKPOINT;
  }
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_s_setprio(0);
#endif

  // partial sums of every wave -> LDS, then each output element adds its quads in order;
  // four activation tiles at a time, which is what the LDS allocation is sized for
  constexpr int CT = MT < (int)kSumTiles ? MT : (int)kSumTiles;
  float *sums = reinterpret_cast<float *>(lds);
  // (the thread's coordinates are worked out again rather than kept in registers, or spilled,
  // over the walk)
  uint32_t lane2 = __lane_id();
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(lane2));
#endif
  const uint32_t tid2 = wave * 64 + lane2;
#pragma unroll
  for (int c0 = 0; c0 < MT; c0 += CT) {
    __syncthreads();  // tables and stream bytes (or the previous chunk's sums) are done with
#pragma unroll
    for (int jj = 0; jj < CT; ++jj)
      if (c0 + jj < MT) {  // (six tiles: the second round holds two)
#pragma unroll
        for (int v = 0; v < 4; ++v) sums[((wave * CT + jj) * 4 + v) * 64 + lane2] = acc[c0 + jj][v];
      }
    __syncthreads();
    const uint32_t per_block = CT * 256;  // values of one row block: [tile jj][v][lane]
    for (uint32_t i = tid2; i < shape.row_blocks * per_block; i += nthreads) {
      const uint32_t blk = i / per_block, within = i % per_block;
      const uint32_t jj = within / 256, v = (within / 64) % 4, ln = within % 64;
      const uint32_t n_local = blk * 16 + ln % 16, m = (c0 + jj) * 16 + (ln / 16) * 4 + v;
      const uint32_t orow = n_local < R ? g.tile_rows[tile * R + n_local] : grf::kNoRow;
      if (orow >= f.rows || m >= m_rows || c0 + jj >= (uint32_t)MT) continue;  // empty slot, no such row, a padding row
      // wave index of (quad, block) is quad * row_blocks + block
      float sum = sums[(blk * CT) * 256 + within];
      for (uint32_t qd = 1; qd < shape.quads; ++qd) sum += sums[((qd * shape.row_blocks + blk) * CT) * 256 + within];
      if (parts > 1) {  // this part's share: the parts meet in gemm_sum_parts_kernel
        partials[((size_t)part * m_rows + m) * f.rows + orow] = sum;
        continue;
      }
      if (bias) sum += __uint_as_float((uint32_t)bias[orow] << 16);
      y[(size_t)m * ldy + orow] = round_bf16(sum);
    }
  }
  if (bad) atomicOr(error, (int)bad);
}

// Up to four activation tiles: 80 vector registers, six waves per SIMD.
template <class Walk, int MT, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) __attribute__((amdgpu_waves_per_eu(6))) void fused_gemm_kernel(
    grf_bctx_fused f, grf_fused_tiling g, const uint4 *xp, uint32_t m_rows, uint16_t *y, uint32_t ldy,
    const uint16_t *bias, float *partials, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  fused_gemm_body<Walk, MT, SCAN>(lds, f, g, xp, m_rows, y, ldy, bias, partials, error, blockIdx.x);
}

// Eight activation tiles: the accumulators and operands alone take 64 registers, so fewer
// waves are resident; still cheaper than decoding the matrix twice.
template <class Walk, int MT, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_gemm_wide_kernel(grf_bctx_fused f, grf_fused_tiling g,
                                                                                 const uint4 *xp, uint32_t m_rows,
                                                                                 uint16_t *y, uint32_t ldy,
                                                                                 const uint16_t *bias, float *partials, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  fused_gemm_body<Walk, MT, SCAN>(lds, f, g, xp, m_rows, y, ldy, bias, partials, error, blockIdx.x);
}

template <class Walk, int MT, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) __attribute__((amdgpu_waves_per_eu(6))) void fused_gemm_group_kernel(
    FusedGroup a, const uint4 *xp, uint32_t m_rows, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t i = group_member(a, blockIdx.x);
  fused_gemm_body<Walk, MT, SCAN>(lds, a.f[i], a.g[i], xp, m_rows, a.y[i], a.ldy[i], a.bias[i], nullptr, error,
                                  blockIdx.x - a.first_tile[i]);
}

template <class Walk, int MT, int SCAN>
__global__ __launch_bounds__(grf::kFusedMaxThreads) void fused_gemm_wide_group_kernel(FusedGroup a, const uint4 *xp,
                                                                                       uint32_t m_rows, int32_t *error) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t i = group_member(a, blockIdx.x);
  fused_gemm_body<Walk, MT, SCAN>(lds, a.f[i], a.g[i], xp, m_rows, a.y[i], a.ldy[i], a.bias[i], nullptr, error,
                                  blockIdx.x - a.first_tile[i]);
}

// y[m][n] = bf16(partials[0][m][n] + partials[1][m][n] + ... + bias[n]): the parts of a
// K-split launch, added in part order
static __global__ __launch_bounds__(256) void gemm_sum_parts_kernel(const float *partials, uint32_t parts, uint32_t m_rows,
                                                                    uint32_t rows, const uint16_t *bias, uint16_t *y,
                                                                    uint32_t ldy) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m_rows * rows) return;
  const uint32_t m = i / rows, n = i - m * rows;
  float sum = partials[i];
  for (uint32_t p = 1; p < parts; ++p) sum += partials[(size_t)p * m_rows * rows + i];
  if (bias) sum += __uint_as_float((uint32_t)bias[n] << 16);
  y[(size_t)m * ldy + n] = round_bf16(sum);
}

template <class Walk, int MT>
int launch_gemm_rows(const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                     uint16_t *y, uint32_t ldy, const uint16_t *bias, uint4 *xp, float *partials, int32_t *error,
                     hipStream_t s) {
  const GemmLdsLayout L(f, g);
  if (L.total > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused GEMM: LDS demand exceeds 160 KiB");
  if (x) launch_pack(x, ldx, m_rows, f.cols, MT * 16, xp, s);  // else the caller packed these rows already
  auto launch = [&](auto scan) -> int {
    constexpr int SCAN = decltype(scan)::value;
    constexpr auto kernel = [] {
      if constexpr (MT <= 4) return &fused_gemm_kernel<Walk, MT, SCAN>;
      else return &fused_gemm_wide_kernel<Walk, MT, SCAN>;
    }();
    if (L.total > 64 * 1024)
      if (int rc = allow_full_lds<kernel>()) return rc;
    hipLaunchKernelGGL(kernel, dim3(g.n_tiles), dim3(g.threads), L.total, s, f, g, xp, m_rows, y, ldy, bias, partials,
                       error);
    return GRF_OK;
  };
  if (int rc = f.whole_range ? launch(std::integral_constant<int, grf::kScanAny>{})
                             : launch(std::integral_constant<int, grf::kScanNoWholeRange>{}))
    return rc;
  if (g.k_parts > 1)
    hipLaunchKernelGGL(gemm_sum_parts_kernel, dim3((m_rows * f.rows + 255) / 256), dim3(256), 0, s, partials, g.k_parts,
                       m_rows, f.rows, bias, y, ldy);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused GEMM: ") + hipGetErrorString(e));
  return GRF_OK;
}

// bytes of the packed copy of the activations one launch needs
inline size_t gemm_workspace_bytes(uint32_t cols, uint32_t m_rows) {
  const uint32_t m = m_rows > kMaxRowsPerLaunch ? kMaxRowsPerLaunch : m_rows;
  return (size_t)(cols / 8 + 1) * gemm_tiles(m) * 16 * 16;
}
// ... and of the whole workspace of a launch cut into k_parts along K: the packed copy, then
// (from the next multiple of 256) the parts' fp32 sums [k_parts][rows of the launch][rows]
inline size_t gemm_partials_offset(uint32_t cols, uint32_t m_rows) {
  return (gemm_workspace_bytes(cols, m_rows) + 255) / 256 * 256;
}
inline size_t gemm_workspace_bytes_split(uint32_t cols, uint32_t rows, uint32_t k_parts, uint32_t m_rows) {
  if (k_parts <= 1) return gemm_workspace_bytes(cols, m_rows);
  const uint32_t m = m_rows > kMaxRowsPerLaunch ? kMaxRowsPerLaunch : m_rows;
  return gemm_partials_offset(cols, m_rows) + (size_t)k_parts * m * rows * 4;
}

// y = x W^T (+ bias) for any number of activation rows, 128 per launch.  `workspace` holds
// the packed activations of one launch; launches follow one another on the stream.  With
// x == nullptr the workspace already holds these rows (pack_rows, same cols and m_rows).
template <class Walk>
int launch_gemm(const char *who, const grf_bctx_fused &f, const grf_fused_tiling &g, const uint16_t *x, uint32_t ldx,
                uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, void *workspace,
                size_t workspace_bytes, int32_t *error, hipStream_t s) {
  if (!m_rows) return GRF_OK;
  if (ldy < f.rows) return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": ldy is smaller than the row count");
  if (!x && m_rows > kMaxRowsPerLaunch)
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": packed activations hold at most 128 rows");
  if (x && (ldx < f.cols || (ldx & 3) || ((uintptr_t)x & 7)))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) +
                                                ": x must be 8-byte aligned with a leading dimension that is a multiple of 4");
  if (GemmShape(g).threads != g.threads || g.threads > (uint32_t)grf::kFusedMaxThreads)
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) +
                                                ": tiling threads must be 64 x ceil(rows_per_tile / 16) x ceil(lanes_per_row / 4)");
  if (g.k_parts > 1 && (g.n_tiles % g.k_parts || g.k_parts > g.n_slabs))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": k_parts must divide n_tiles and be at most n_slabs");
  if (!workspace || ((uintptr_t)workspace & 15) ||
      workspace_bytes < gemm_workspace_bytes_split(f.cols, f.rows, g.k_parts, m_rows))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": workspace missing, misaligned or too small");
  uint4 *xp = static_cast<uint4 *>(workspace);
  float *partials = g.k_parts > 1 ? reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) +
                                                              gemm_partials_offset(f.cols, m_rows))
                                  : nullptr;
  for (uint32_t m0 = 0; m0 < m_rows; m0 += kMaxRowsPerLaunch) {
    const uint32_t m = m_rows - m0 < kMaxRowsPerLaunch ? m_rows - m0 : kMaxRowsPerLaunch;
    const uint16_t *xs = x ? x + (size_t)m0 * ldx : nullptr;
    uint16_t *ys = y + (size_t)m0 * ldy;
    int rc;
    if (m <= 16) rc = launch_gemm_rows<Walk, 1>(f, g, xs, ldx, m, ys, ldy, bias, xp, partials, error, s);
    else if (m <= 32) rc = launch_gemm_rows<Walk, 2>(f, g, xs, ldx, m, ys, ldy, bias, xp, partials, error, s);
    else if (m <= 64) rc = launch_gemm_rows<Walk, 4>(f, g, xs, ldx, m, ys, ldy, bias, xp, partials, error, s);
    else rc = launch_gemm_rows<Walk, 8>(f, g, xs, ldx, m, ys, ldy, bias, xp, partials, error, s);
    if (rc) return rc;
  }
  return GRF_OK;
}

// The rows of x in operand order into `workspace`, for products of several matrices with
// the same activations.
inline int pack_rows(const char *who, const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint32_t cols, void *workspace,
                     size_t workspace_bytes, hipStream_t s) {
  if (!x || !m_rows || m_rows > kMaxRowsPerLaunch || !cols || (cols & 15))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": 1..128 rows of a width that is a multiple of 16");
  if (ldx < cols || (ldx & 3) || ((uintptr_t)x & 7))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) +
                                                ": x must be 8-byte aligned with a leading dimension that is a multiple of 4");
  if (!workspace || ((uintptr_t)workspace & 15) || workspace_bytes < gemm_workspace_bytes(cols, m_rows))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": workspace missing, misaligned or too small");
  launch_pack(x, ldx, m_rows, cols, gemm_tiles(m_rows) * 16, static_cast<uint4 *>(workspace), s);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string(who) + ": " + hipGetErrorString(e));
  return GRF_OK;
}

// ---------------------------------------------------------------- grouped launches

struct GroupSpec {  // the arrays of a grouped entry point
  uint32_t n;
  const grf_bctx_fused *const *frames;
  const grf_fused_tiling *const *tilings;
  uint16_t *const *y;
  const uint32_t *ldy;
  const uint16_t *const *bias;  // may be null, and so may any of its elements
};

inline int build_group(const char *who, const GroupSpec &spec, bool gemm, FusedGroup &a) {
  auto bad = [&](const char *why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (spec.n < 1 || spec.n > kMaxGroup) return bad("a group has 1..4 members");
  if (!spec.frames || !spec.tilings || !spec.y || !spec.ldy) return bad("null argument");
  a = FusedGroup{};
  a.n = spec.n;
  for (uint32_t i = 0; i < spec.n; ++i) {
    if (!spec.frames[i] || !spec.tilings[i] || !spec.y[i]) return bad("null member");
    const grf_bctx_fused &f = *spec.frames[i];
    const grf_fused_tiling &g = *spec.tilings[i];
    if (int rc = grf::check_fused_frame(f, g, who, gemm ? kGemmTiling : kGemvTiling)) return rc;
    if (f.cols != spec.frames[0]->cols) return bad("members must have one width");
    if (g.threads != spec.tilings[0]->threads) return bad("member tilings must share one thread count");
    if (g.scheme != spec.tilings[0]->scheme) return bad("member tilings must share one scheme");
    if (g.k_parts > 1) return bad("grouped launches take tilings that are not cut along K (k_parts <= 1)");
    if (gemm && GemmShape(g).threads != g.threads)
      return bad("tiling threads must be 64 x ceil(rows_per_tile / 16) x ceil(lanes_per_row / 4)");
    if (spec.ldy[i] < f.rows) return bad("ldy is smaller than the row count");
    a.f[i] = f;
    a.g[i] = g;
    a.y[i] = spec.y[i];
    a.ldy[i] = spec.ldy[i];
    a.bias[i] = spec.bias ? spec.bias[i] : nullptr;
    a.first_tile[i + 1] = a.first_tile[i] + g.n_tiles;
  }
  return GRF_OK;
}

template <class Walk, int M>
int launch_walk_group(const FusedGroup &a, const uint16_t *x, uint32_t ldx, int32_t *error, hipStream_t s) {
  uint32_t lds = 0;
  for (uint32_t i = 0; i < a.n; ++i) lds = std::max(lds, FusedLdsLayout(a.f[i], a.g[i], M).total);
  if (lds > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
  constexpr auto kernel = &fused_walk_group_kernel<Walk, M>;
  if (lds > 64 * 1024)
    if (int rc = allow_full_lds<kernel>()) return rc;
  hipLaunchKernelGGL(kernel, dim3(a.first_tile[a.n]), dim3(a.g[0].threads), lds, s, a, x, ldx, error);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused kernel: ") + hipGetErrorString(e));
  return GRF_OK;
}

// y_i = x W_i^T (+ bias_i) for the members of a group, 1..8 activation rows, one launch
template <class Walk>
int launch_gemv_group(const char *who, const GroupSpec &spec, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                      int32_t *error, hipStream_t s) {
  FusedGroup a;
  if (int rc = build_group(who, spec, false, a)) return rc;
  if (m_rows < 1 || m_rows > 8) return grf::set_error(GRF_UNSUPPORTED, std::string(who) + ": 1 <= m_rows <= 8");
  if (!x || ldx < a.f[0].cols || (ldx & 1) || ((uintptr_t)x & 3))
    return grf::set_error(GRF_BAD_ARGUMENT,
                          std::string(who) + ": x must be 4-byte aligned with an even leading dimension");
  if (a.g[0].scheme == GRF_TILE_WAVES) {
    uint32_t lds = 0;
    for (uint32_t i = 0; i < a.n; ++i) {
      if (int rc = check_wave_operands(who, a.f[i], x, ldx)) return rc;
      lds = std::max(lds, WaveLdsLayout(a.f[i], a.g[i], kWaveRowsPerPass).total);
    }
    if (lds > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused kernel: LDS demand exceeds 160 KiB");
    bool whole = false;  // one member with a whole-range context: the scan that knows them, for all
    for (uint32_t i = 0; i < a.n; ++i) whole = whole || a.f[i].whole_range;
    for (uint32_t m0 = 0; m0 < m_rows; m0 += kWaveRowsPerPass) {
      FusedGroup part = a;
      for (uint32_t i = 0; i < a.n; ++i) part.y[i] = a.y[i] + (size_t)m0 * a.ldy[i];
      const uint16_t *xs = x + (size_t)m0 * ldx;
      const bool one = m_rows - m0 == 1;
      auto launch = [&](auto kernel_tag) -> int {
        constexpr auto kernel = decltype(kernel_tag)::value;
        if (lds > 64 * 1024)
          if (int rc = allow_full_lds<kernel>()) return rc;
        hipLaunchKernelGGL(kernel, dim3(a.first_tile[a.n]), dim3(a.g[0].threads), lds, s, part, xs, ldx, error);
        return GRF_OK;
      };
      using K1 = std::integral_constant<decltype(&fused_wave_group_kernel<Walk, 1, grf::kScanAny>),
                                        &fused_wave_group_kernel<Walk, 1, grf::kScanAny>>;
      using K2 = std::integral_constant<decltype(&fused_wave_group_kernel<Walk, 2, grf::kScanAny>),
                                        &fused_wave_group_kernel<Walk, 2, grf::kScanAny>>;
      using S1 = std::integral_constant<decltype(&fused_wave_group_kernel<Walk, 1, grf::kScanNoWholeRange>),
                                        &fused_wave_group_kernel<Walk, 1, grf::kScanNoWholeRange>>;
      using S2 = std::integral_constant<decltype(&fused_wave_group_kernel<Walk, 2, grf::kScanNoWholeRange>),
                                        &fused_wave_group_kernel<Walk, 2, grf::kScanNoWholeRange>>;
      const int rc = whole ? (one ? launch(K1{}) : launch(K2{})) : (one ? launch(S1{}) : launch(S2{}));
      if (rc) return rc;
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused kernel: ") + hipGetErrorString(e));
    }
    return GRF_OK;
  }
  using Ahead = typename ahead_of<Walk>::type;
  bool ahead = !std::is_same<Ahead, Walk>::value && m_rows <= kAheadMaxRows;
  for (uint32_t i = 0; i < a.n; ++i) ahead = ahead && reads_ahead(a.f[i]);
  if (ahead) switch (m_rows) {
      case 1: return launch_walk_group<Ahead, 1>(a, x, ldx, error, s);
      case 2: return launch_walk_group<Ahead, 2>(a, x, ldx, error, s);
      case 3: return launch_walk_group<Ahead, 3>(a, x, ldx, error, s);
      default: return launch_walk_group<Ahead, 4>(a, x, ldx, error, s);
    }
  switch (m_rows) {
    case 1: return launch_walk_group<Walk, 1>(a, x, ldx, error, s);
    case 2: return launch_walk_group<Walk, 2>(a, x, ldx, error, s);
    case 3: return launch_walk_group<Walk, 3>(a, x, ldx, error, s);
    case 4: return launch_walk_group<Walk, 4>(a, x, ldx, error, s);
    case 5: return launch_walk_group<Walk, 5>(a, x, ldx, error, s);
    case 6: return launch_walk_group<Walk, 6>(a, x, ldx, error, s);
    case 7: return launch_walk_group<Walk, 7>(a, x, ldx, error, s);
    default: return launch_walk_group<Walk, 8>(a, x, ldx, error, s);
  }
}

template <class Walk, int MT>
int launch_gemm_group_rows(const FusedGroup &a, uint32_t m_rows, const uint4 *xp, int32_t *error, hipStream_t s) {
  uint32_t lds = 0;
  for (uint32_t i = 0; i < a.n; ++i) lds = std::max(lds, GemmLdsLayout(a.f[i], a.g[i]).total);
  if (lds > 160 * 1024) return grf::set_error(GRF_UNSUPPORTED, "fused GEMM: LDS demand exceeds 160 KiB");
  bool whole = false;  // one member with a whole-range context: the scan that knows them, for all
  for (uint32_t i = 0; i < a.n; ++i) whole = whole || a.f[i].whole_range;
  auto launch = [&](auto scan) -> int {
    constexpr int SCAN = decltype(scan)::value;
    constexpr auto kernel = [] {
      if constexpr (MT <= 4) return &fused_gemm_group_kernel<Walk, MT, SCAN>;
      else return &fused_gemm_wide_group_kernel<Walk, MT, SCAN>;
    }();
    if (lds > 64 * 1024)
      if (int rc = allow_full_lds<kernel>()) return rc;
    hipLaunchKernelGGL(kernel, dim3(a.first_tile[a.n]), dim3(a.g[0].threads), lds, s, a, xp, m_rows, error);
    return GRF_OK;
  };
  if (int rc = whole ? launch(std::integral_constant<int, grf::kScanAny>{})
                     : launch(std::integral_constant<int, grf::kScanNoWholeRange>{}))
    return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return grf::set_error(GRF_LAUNCH_FAILED, std::string("fused GEMM: ") + hipGetErrorString(e));
  return GRF_OK;
}

// the same for any number of rows on the matrix cores, 128 rows per launch; x == nullptr:
// the workspace already holds the rows
template <class Walk>
int launch_gemm_group(const char *who, const GroupSpec &spec, const uint16_t *x, uint32_t ldx, uint32_t m_rows,
                      void *workspace, size_t workspace_bytes, int32_t *error, hipStream_t s) {
  FusedGroup a;
  if (int rc = build_group(who, spec, true, a)) return rc;
  if (!m_rows) return GRF_OK;
  const uint32_t cols = a.f[0].cols;
  if (!x && m_rows > kMaxRowsPerLaunch)
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": packed activations hold at most 128 rows");
  if (x && (ldx < cols || (ldx & 3) || ((uintptr_t)x & 7)))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) +
                                                ": x must be 8-byte aligned with a leading dimension that is a multiple of 4");
  if (!workspace || ((uintptr_t)workspace & 15) || workspace_bytes < gemm_workspace_bytes(cols, m_rows))
    return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": workspace missing, misaligned or too small");
  uint4 *xp = static_cast<uint4 *>(workspace);
  for (uint32_t m0 = 0; m0 < m_rows; m0 += kMaxRowsPerLaunch) {
    const uint32_t m = m_rows - m0 < kMaxRowsPerLaunch ? m_rows - m0 : kMaxRowsPerLaunch;
    FusedGroup part = a;
    for (uint32_t i = 0; i < a.n; ++i) part.y[i] = a.y[i] + (size_t)m0 * a.ldy[i];
    if (x) launch_pack(x + (size_t)m0 * ldx, ldx, m, cols, gemm_tiles(m) * 16, xp, s);
    int rc;
    if (m <= 16) rc = launch_gemm_group_rows<Walk, 1>(part, m, xp, error, s);
    else if (m <= 32) rc = launch_gemm_group_rows<Walk, 2>(part, m, xp, error, s);
    else if (m <= 64) rc = launch_gemm_group_rows<Walk, 4>(part, m, xp, error, s);
    else rc = launch_gemm_group_rows<Walk, 8>(part, m, xp, error, s);
    if (rc) return rc;
  }
  return GRF_OK;
}

inline uint32_t gemm_lds_bytes(const grf_bctx_fused &f, const grf_fused_tiling &g) { return GemmLdsLayout(f, g).total; }

}  // namespace grf
