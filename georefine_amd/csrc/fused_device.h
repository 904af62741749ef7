// The fused decoder: one walker over a checkpointed segment whose decoded BF16
// words go to a sink (FMA chain for the GEMV, LDS tile for the GEMM, global
// store for decode()).  Because every sink is fed by the same walker, words
// proven bit-exact through the store sink are the words the fused sinks consume.
//
// Work decomposition (mode 0 frames, segment length S divides the row length K):
//   * rows are grouped by row class; a workgroup ("tile") owns up to R rows of
//     ONE class, so only that class's nc column contexts are live and their
//     lookup tables fit in LDS;
//   * a row's K/S segments are walked P at a time ("slab"); lane (r, p) decodes
//     segment b*P + p of row r in slab b, so at step t every lane of the
//     workgroup is at column (b*P + p)*S + t and the x slab is P*S wide;
//   * the main-stream bytes of a slab are R contiguous pieces (one per row);
//     they are copied to LDS with 16-byte coalesced loads and each lane then
//     consumes its own sub-range with byte-granular LDS reads;
//   * the packed 6-bit residuals of a lane are 12 bytes per 16 symbols at a
//     position known in advance; they are loaded straight into registers.
//
// Symbol lookup: slot>>shift indexes a u8 table giving the sparse index of the
// symbol that owns the bucket's first slot; the 8-byte entries of that symbol
// and of its successor are read together and one compare picks between them.
// Entry: lo = start | (freq-1)<<16, hi = next_start (bits 0..16) | symbol<<21
// | small<<31 where `small` marks freq < bucket size (then the successor may
// still end inside the bucket and a short forward scan finishes the search).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "georefine_amd.h"
#include "rans_device.h"

namespace grf {

constexpr int kFusedThreads = 256;
constexpr uint32_t kNoRow = 0xFFFFFFFFu;

struct FusedLds {
  uint8_t *lut;       // nc << lognb bytes
  const uint2 *tab;   // (tabn + 1) * nc entries, index = sparse*nc + cc
  float *xs;          // M * P * (S + 4) floats
  uint8_t *cc8;       // P * S bytes: column class
  uint8_t *stream;    // R * piece_cap bytes
  float *part;        // R * P * M floats
};

__host__ __device__ inline uint32_t align_up(uint32_t v, uint32_t a) { return (v + a - 1) / a * a; }

// byte offsets of the LDS regions; shared by host (size) and device (carve)
struct FusedLdsLayout {
  uint32_t lut, tab, xs, cc8, stream, part, total;
  __host__ __device__ FusedLdsLayout(const grf_bctx_fused &f, uint32_t m) {
    uint32_t at = 0;
    lut = at;
    at = align_up(at + (f.nc << f.lognb), 16);
    tab = at;
    at = align_up(at + (f.tabn + 1) * f.nc * 8, 16);
    xs = at;
    at = align_up(at + m * f.lanes_per_row * (f.seg_len + 4) * 4, 16);
    cc8 = at;
    at = align_up(at + f.lanes_per_row * f.seg_len, 16);
    stream = at;
    at = align_up(at + f.rows_per_tile * f.piece_cap, 16);
    part = at;
    at = align_up(at + f.rows_per_tile * f.lanes_per_row * m * 4, 16);
    total = at;
  }
};

// One decode step of the main stream against LDS tables.
// Returns the selected table entry's hi word (symbol<<21 among other bits).
__device__ __forceinline__ uint32_t fused_symbol(uint32_t &state, uint32_t &ip, const uint8_t *lds_base,
                                                 uint32_t lut_off, uint32_t tab_off, uint32_t cc, uint32_t shift,
                                                 uint32_t lognb, uint32_t lognc) {
  const uint32_t slot = state & 0xFFFFu;
  const uint32_t la = (cc << lognb) | (slot >> shift);
  uint32_t idx = lds_base[lut_off + la];
  const uint2 *tab = reinterpret_cast<const uint2 *>(lds_base + tab_off);
  uint32_t ta = (idx << lognc) | cc;
  const uint2 e0 = tab[ta];
  const uint2 e1 = tab[ta + (1u << lognc)];
  const bool take1 = slot >= (e0.y & 0x1FFFFu);
  uint32_t lo = take1 ? e1.x : e0.x;
  uint32_t hi = take1 ? e1.y : e0.y;
  if (__builtin_expect((int32_t)hi < 0, 0)) {  // small symbol: successor may also end before slot
    ta += take1 ? (1u << lognc) : 0u;
    while (slot >= (hi & 0x1FFFFu)) {
      ta += 1u << lognc;
      const uint2 e = tab[ta];
      lo = e.x;
      hi = e.y;
    }
  }
  const uint32_t h = state >> 16;
  uint32_t x = (lo >> 16) * h + (slot + h - (lo & 0xFFFFu));
  // refill: at most two bytes; both are read unconditionally (the region has slack)
  uint16_t two;
  __builtin_memcpy(&two, lds_base + ip, 2);
  const uint32_t b0 = two & 0xFFu, b1 = two >> 8;
  const bool n1 = x < kLow;
  x = n1 ? ((x << 8) | b0) : x;
  ip += n1;
  const bool n2 = x < kLow;
  x = n2 ? ((x << 8) | b1) : x;
  ip += n2;
  state = x;
  return hi;
}

// Sixteen packed 6-bit residuals (12 bytes, MSB first) -> field k, k compile-time.
struct Raw6x16 {
  uint32_t w0, w1, w2;  // big-endian dwords
  __device__ __forceinline__ void load(const uint8_t *p) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
    w0 = __builtin_bswap32(q[0]);
    w1 = __builtin_bswap32(q[1]);
    w2 = __builtin_bswap32(q[2]);
  }
  template <int K>
  __device__ __forceinline__ uint32_t field() const {
    constexpr int bit = K * 6;          // position from the MSB of the 96-bit group
    constexpr int word = bit / 32, off = bit % 32;
    const uint32_t a = word == 0 ? w0 : (word == 1 ? w1 : w2);
    if constexpr (off + 6 <= 32) {
      return (a >> (32 - 6 - off)) & 63u;
    } else {
      const uint32_t b = word == 0 ? w1 : w2;
      return (uint32_t)((((uint64_t)a << 32 | b) >> (64 - 6 - off)) & 63u);
    }
  }
};

// fp32 bit pattern of the BF16 word (word << 16) from the entry's hi field and the residual
__device__ __forceinline__ uint32_t fused_value_bits(uint32_t hi, uint32_t r6) {
  return (hi & 0x7FE00000u) | ((r6 & 31u) << 16) | ((r6 >> 5) << 31);
}

}  // namespace grf
