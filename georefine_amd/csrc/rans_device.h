// Device-side building blocks shared by the decode, GEMV and GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "georefine_amd.h"

namespace grf {

constexpr uint32_t kLow = 1u << 23;

// BCTX: 10-bit main symbol + 6-bit residual -> BF16 word
// (inverse of GCR/bitexact_context_ans.cpp:9-12).
__device__ __forceinline__ uint32_t bctx_word(uint32_t main_sym, uint32_t res) {
  return (main_sym << 5) | (res & 31u) | ((res >> 5) << 15);
}
// PPCX: 11-bit main symbol (sign in bit 10) + 5-bit residual
// (GCR/bitexact_predictive_codec.py:248).
__device__ __forceinline__ uint32_t ppcx_word(uint32_t main_sym, uint32_t res) {
  return ((main_sym & 1024u) << 5) | ((main_sym & 1023u) << 5) | res;
}

// Packed fixed-width fields, most significant bit first: field i occupies bits
// [i*BITS, (i+1)*BITS) of the byte stream (GCR/bitexact_context_gpu_kernels.py:144-149).
template <int BITS>
__device__ __forceinline__ uint32_t packed_field(const uint8_t *p, uint32_t n_bytes, uint64_t i) {
  const uint64_t bit = i * BITS;
  const uint64_t byte = bit >> 3;
  const uint32_t hi = byte < n_bytes ? p[byte] : 0u;
  const uint32_t lo = byte + 1 < n_bytes ? p[byte + 1] : 0u;
  return (((hi << 8) | lo) >> (16 - BITS - (uint32_t)(bit & 7))) & ((1u << BITS) - 1);
}

// One rANS decode step against tables in global memory.  `cum` and `bucket`
// point at the rows of the symbol's context.  Never reads out of bounds
// whatever the stream holds; problems are OR-ed into `bad`.
__device__ __forceinline__ uint32_t rans_step_global(uint32_t &state, uint32_t &ip, const uint8_t *bytes,
                                                     uint32_t n_bytes, const uint32_t *cum,
                                                     const uint32_t *bucket, uint32_t &bad) {
  const uint32_t slot = state & 0xFFFFu;
  const uint32_t range = bucket[slot >> 8];
  uint32_t lo = range & 0xFFFFu, hi = range >> 16;
  while (lo < hi) {  // last symbol whose start is <= slot
    const uint32_t mid = (lo + hi + 1) >> 1;
    if (cum[mid] <= slot) lo = mid;
    else hi = mid - 1;
  }
  const uint32_t start = cum[lo];
  const uint32_t f = cum[lo + 1] - start;
  if (f == 0 || slot - start >= f) bad |= GRF_ERR_SYMBOL;
  state = f * (state >> 16) + (slot - start);
#pragma unroll
  for (int k = 0; k < 2; ++k) {  // a valid stream needs at most two refill bytes
    if (state < kLow) {
      uint32_t b = 0;
      if (ip < n_bytes) b = bytes[ip];
      else bad |= GRF_ERR_OVERRUN;
      state = (state << 8) | b;
      ++ip;
    }
  }
  if (state < kLow) bad |= GRF_ERR_UNDERFLOW;
  return lo;
}

// Ordinal key of a BF16 word and its bin among 15 monotone thresholds
// (GCR/bitexact_predictive_codec.py:106-110, device form
// GCR/bitexact_predictive_gpu_kernels.py:36-42): number of thresholds <= key.
__device__ __forceinline__ uint32_t ordinal_key(uint32_t word, uint32_t flip) {
  const uint32_t a = (word ^ (flip << 15)) & 0xFFFFu;
  return (a & 0x8000u) ? (~a & 0xFFFFu) : (a ^ 0x8000u);
}
__device__ __forceinline__ uint32_t threshold_bin(const uint16_t *th, uint32_t key) {
  uint32_t lo = 0, hi = 15;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (key >= th[mid]) lo = mid + 1;
      else hi = mid;
    }
  }
  return lo;
}

}  // namespace grf
