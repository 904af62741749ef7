// The fused decoder: one walker over a checkpointed segment whose decoded BF16
// words go to a sink (dot-product chain for the GEMV, LDS tile for the GEMM,
// global store for decode()).  Because every sink is fed by the same walker,
// words proven bit-exact through the store sink are the words the fused sinks
// consume.
//
// Work decomposition (packed-residual frames, segment length S divides the row
// length K):
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
//     position known in advance; they are loaded straight into registers, as are
//     the 16 column classes of the same columns.
//
// Symbol lookup: slot>>shift indexes a u8 table giving the sparse index of the
// symbol that owns the bucket's first slot; that symbol's 8-byte entry is read and
// assumed to own the slot.  Entry: low32 = start | (freq & 0xFFFF)<<16 (0 stands for 65536), high32 = symbol<<5
// (the symbol's bits in the BF16 word).  When a symbol boundary falls inside the
// bucket before the slot, a forward scan over the following entries finishes the search.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "georefine_amd.h"
#include "rans_device.h"

namespace grf {

constexpr int kFusedMaxThreads = 1024;
constexpr uint32_t kNoRow = 0xFFFFFFFFu;
constexpr uint32_t kXPad = 8;  // BF16 elements of padding per x segment in LDS (16 bytes)

__host__ __device__ inline uint32_t align_up(uint32_t v, uint32_t a) { return (v + a - 1) / a * a; }

// Per column class the LDS holds one block: the sparse symbol table first (kTabCap
// 8-byte entries), then the class's lookup bytes.  With the block base in a register
// the table read needs no further address arithmetic and the lookup read folds the
// constant table size into its offset field.
constexpr uint32_t kTabCap = 257;  // up to 256 symbols + the entry a forward scan stops on
constexpr uint32_t kTabBytes = kTabCap * 8;

// byte offsets of the LDS regions; shared by host (size) and device (carve).
struct FusedLdsLayout {
  uint32_t blocks, block_pitch, stream, xs, part, total;
  __host__ __device__ FusedLdsLayout(const grf_bctx_fused &f, const grf_fused_tiling &g, uint32_t m) {
    uint32_t at = 0;
    blocks = at;
    block_pitch = kTabBytes + (1u << f.lognb);
    at = align_up(at + f.nc * block_pitch, 16);
    stream = at;
    at = align_up(at + g.rows_per_tile * g.piece_cap, 16);
    xs = at;
    at = align_up(at + m * g.lanes_per_row * (f.seg_len + kXPad) * 2, 16);
    part = at;
    at = align_up(at + g.rows_per_tile * f.segs_per_row * m * 4, 16);
    total = at;
  }
};

typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef uint32_t v2u32 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2u32 lds_v2u32;

// LDS accesses by absolute byte offset (dynamic LDS starts at address 0 here:
// the kernels declare no static LDS)
__device__ __forceinline__ uint8_t lds_load_u8(uint32_t off) { return *reinterpret_cast<lds_u8 *>(off); }

struct FusedParams {  // uniform values the step needs, kept in scalar registers
  uint32_t shift, block_pitch;
};

// Slow twin of the step for the rare case that the slot lies beyond the looked-up symbol:
// scan forward from entry `e` at table address `ta` to the symbol that holds the slot, then
// update and refill in plain C.  Returns the entry's high word.
__device__ __forceinline__ uint32_t fused_symbol_scan(uint32_t &state, uint32_t &ip, uint32_t ta, v2u32 e,
                                                      uint32_t byte0, uint32_t byte1) {
  const uint32_t slot = state & 0xFFFFu;
  uint32_t freq = e.x >> 16;
  freq = freq ? freq : 65536u;
  while (slot - (e.x & 0xFFFFu) >= freq) {
    ta += 8;
    e = *reinterpret_cast<lds_v2u32 *>(ta);
    freq = e.x >> 16;
    freq = freq ? freq : 65536u;
  }
  uint32_t x = freq * (state >> 16) + (slot - (e.x & 0xFFFFu));
  if (x < kLow) {
    x = (x << 8) | byte0;
    ++ip;
    if (x < kLow) {
      x = (x << 8) | byte1;
      ++ip;
    }
  }
  state = x;
  return e.y;
}

// cc * pitch with cc = byte BYTE of `ccw`: one multiply whose operand select does the extraction
template <int BYTE>
__device__ __forceinline__ uint32_t fused_block_offset(uint32_t ccw, uint32_t pitch) {
  uint32_t block;
#if defined(__HIP_DEVICE_COMPILE__)
#define GRF_BLOCK(sel)                                                                                       \
  asm("v_mul_u32_u24_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:" sel \
      : "=v"(block)                                                                                          \
      : "s"(pitch), "v"(ccw))
  if constexpr (BYTE == 0) GRF_BLOCK("BYTE_0");
  if constexpr (BYTE == 1) GRF_BLOCK("BYTE_1");
  if constexpr (BYTE == 2) GRF_BLOCK("BYTE_2");
  if constexpr (BYTE == 3) GRF_BLOCK("BYTE_3");
#undef GRF_BLOCK
#else
  block = ((ccw >> (8 * BYTE)) & 0xFFu) * pitch;
#endif
  return block;
}

__device__ __forceinline__ uint32_t fused_lshl3_add(uint32_t a, uint32_t b) {  // (a << 3) + b in one instruction
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t r;
  asm("v_lshl_add_u32 %0, %1, 3, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
#else
  return (a << 3) + b;
#endif
}

// One decode step of the main stream against LDS tables, for the column class held in byte
// BYTE of `ccw`.  Returns the image of the symbol's bits in the BF16 word (symbol << 5).
//
// The lookup byte names the symbol that owns the first slot of the slot's bucket.  With
// buckets finer than almost every symbol, that symbol nearly always owns the slot itself,
// so the step reads only its entry and assumes it; a lane whose slot lies beyond the entry
// (a symbol boundary inside the bucket, or the 16-bit frequency field's 0 = 65536) redoes
// the step with a forward scan.
template <int BYTE>
__device__ __forceinline__ uint32_t fused_symbol(uint32_t &state, uint32_t &ip, uint32_t ccw, const FusedParams &q) {
  // The two possible refill bytes, fetched ahead of need with two byte reads.  (An unaligned
  // 16-bit LDS read stalls the LDS pipeline for tens of cycles on this hardware; aligned
  // dwords cost two vector instructions to address and shift.)
  const uint32_t b0 = lds_load_u8(ip), b1 = lds_load_u8(ip + 1);
  const uint32_t block = fused_block_offset<BYTE>(ccw, q.block_pitch);
  const uint32_t bucket = (state & 0xFFFFu) >> q.shift;
  const uint32_t idx = lds_load_u8(block + bucket + kTabBytes);
  const uint32_t ta = fused_lshl3_add(idx, block);
  const v2u32 e0 = *reinterpret_cast<lds_v2u32 *>(ta);
  const uint32_t state_in = state, ip_in = ip;
  uint32_t x, ipn, rel;
  uint64_t miss;  // lanes whose slot lies beyond the entry
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t t;
  // rel = slot - start; x = freq * (state >> 16) + rel; then up to two refills
  // (x << 8) | byte while x < 2^23, ip counting the bytes taken.  Operand halves are
  // addressed with operand selects instead of shifts and masks; v_perm builds (x << 8) | byte.
  // gfx950 needs two wait states between a VALU write of VCC and a VALU read of it.
  asm volatile(
      "v_sub_u32_sdwa %[rel], %[st], %[e0lo] dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_0\n\t"
      "v_mad_u32_u16 %[x], %[e0lo], %[st], %[rel] op_sel:[1,1,0,0]\n\t"
      "v_cmp_gt_u32 vcc, 0x800000, %[x]\n\t"
      "v_perm_b32 %[t], %[x], %[b0], %[sel]\n\t"
      "s_nop 0\n\t"
      "v_cndmask_b32 %[x], %[x], %[t], vcc\n\t"
      "v_addc_co_u32 %[ipo], vcc, 0, %[ipi], vcc\n\t"
      "v_cmp_gt_u32 vcc, 0x800000, %[x]\n\t"
      "v_perm_b32 %[t], %[x], %[b1], %[sel]\n\t"
      "s_nop 0\n\t"
      "v_cndmask_b32 %[x], %[x], %[t], vcc\n\t"
      "v_addc_co_u32 %[ipo], vcc, 0, %[ipo], vcc\n\t"
      "v_cmp_ge_u32_sdwa %[miss], %[rel], %[e0lo] src0_sel:DWORD src1_sel:WORD_1\n\t"
      : [x] "=&v"(x), [t] "=&v"(t), [rel] "=&v"(rel), [ipo] "=&v"(ipn), [miss] "=&s"(miss)
      : [st] "v"(state), [e0lo] "v"(e0.x), [b0] "v"(b0), [b1] "v"(b1), [sel] "s"(0x06050400u),
        [ipi] "v"(ip)
      : "vcc");
#else
  rel = e0.x + b0 + b1;  // host pass only parses this
  x = state;
  ipn = ip;
  miss = rel;
#endif
  state = x;
  ip = ipn;
  uint32_t hi = e0.y;
#if defined(__HIP_DEVICE_COMPILE__)
  const bool redo = __builtin_amdgcn_inverse_ballot_w64(miss);
#else
  const bool redo = miss != 0;
#endif
  if (__builtin_expect(redo, 0)) {
    // the slot lies beyond the entry: redo the step from the saved state with a forward scan
    state = state_in;
    ip = ip_in;
    hi = fused_symbol_scan(state, ip, ta, e0, b0, b1);
  }
  return hi;
}

// Sixteen packed 6-bit residuals (12 bytes, MSB first) -> field k, k compile-time.
struct Raw6x16 {
  uint32_t w0, w1, w2;  // big-endian dwords
  __device__ __forceinline__ void set(uint32_t a, uint32_t b, uint32_t c) {
    w0 = __builtin_bswap32(a);
    w1 = __builtin_bswap32(b);
    w2 = __builtin_bswap32(c);
  }
  template <int K>
  __device__ __forceinline__ uint32_t field() const {
    constexpr int bit = K * 6;  // position from the MSB of the 96-bit group
    constexpr int word = bit / 32, off = bit % 32;
    const uint32_t a = word == 0 ? w0 : (word == 1 ? w1 : w2);
    if constexpr (off + 6 <= 32) {
      return __builtin_amdgcn_ubfe(a, 32 - 6 - off, 6);
    } else {
      const uint32_t b = word == 0 ? w1 : w2;
      return __builtin_amdgcn_ubfe(__builtin_amdgcn_alignbit(a, b, 64 - 6 - off), 0, 6);
    }
  }
};

// ---- pieces of the tile walk shared by the GEMV and GEMM kernels ----

// this row class's lookup tables -> LDS, one block per column class: table, then lookup bytes
__device__ __forceinline__ void fused_load_tables(uint8_t *lds, uint32_t blocks, uint32_t block_pitch,
                                                  const grf_bctx_fused &f, uint32_t cls, uint32_t tid,
                                                  uint32_t nthreads) {
  const uint32_t nb = 1u << f.lognb, entries = f.tabn + 1;
  for (uint32_t c = 0; c < f.nc; ++c) {
    const uint4 *src = reinterpret_cast<const uint4 *>(f.lut + ((size_t)cls * f.nc + c) * nb);
    uint4 *dst = reinterpret_cast<uint4 *>(lds + blocks + c * block_pitch + kTabBytes);
    for (uint32_t i = tid; i < nb / 16; i += nthreads) dst[i] = src[i];
    const uint2 *ts = reinterpret_cast<const uint2 *>(f.tab) + ((size_t)cls * f.nc + c) * entries;
    uint2 *td = reinterpret_cast<uint2 *>(lds + blocks + c * block_pitch);
    for (uint32_t i = tid; i < entries; i += nthreads) td[i] = ts[i];
  }
}

// Copy the main-stream bytes of one row piece (segments [seg_base, seg_base+nseg)) to LDS
// at piece_off, keeping the 16-byte phase of the global address.  The P lanes of the row
// share the copy.  Returns the aligned global start so lanes can place their cursors.
__device__ __forceinline__ uint32_t fused_stage_piece(uint8_t *lds, uint32_t piece_off, const grf_bctx_fused &f,
                                                      uint32_t seg_base, uint32_t nseg, uint32_t p, uint32_t P) {
  const uint32_t g0 = f.seg_offset[seg_base], g1 = f.seg_offset[seg_base + nseg];
  const uint32_t a0 = g0 & ~15u;
  for (uint32_t o = a0 + p * 16; o < g1; o += P * 16)
    *reinterpret_cast<uint4 *>(lds + piece_off + (o - a0)) = *reinterpret_cast<const uint4 *>(f.main_bytes + o);
  return a0;
}

// A lane's position in its segment: rANS state, LDS cursor, and the registers that hold
// the packed residuals and column classes of the next 16 symbols.
struct SegmentWalk {
  uint32_t state, ip, ip0, gofs, seg;
  const uint32_t *rawp;
  const uint4 *ccp;
  uint32_t n0, n1, n2;
  uint4 nc4;

  __device__ __forceinline__ void open(const grf_bctx_fused &f, uint32_t seg_, uint32_t piece_off, uint32_t a0,
                                       uint64_t elem0, uint32_t col0) {
    seg = seg_;
    state = f.seg_state[seg];
    gofs = f.seg_offset[seg];
    ip0 = piece_off + (gofs - a0);
    ip = ip0;
    rawp = reinterpret_cast<const uint32_t *>(f.raw6 + elem0 / 4 * 3);
    ccp = reinterpret_cast<const uint4 *>(f.col_class + col0);
    n0 = rawp[0];
    n1 = rawp[1];
    n2 = rawp[2];
    nc4 = ccp[0];
  }

  // Decode symbols [t, t+16) of the segment into eight BF16 pairs (word k in the low half,
  // k+1 in the high half); loads the registers for the following group meanwhile.
  __device__ __forceinline__ void decode16(uint32_t t, uint32_t S, const FusedParams &q, uint32_t (&pair)[8]);

  // the segment must end exactly on the next checkpoint
  __device__ __forceinline__ bool ended_on_checkpoint(const grf_bctx_fused &f) const {
    return state == f.seg_state[seg + 1] && gofs + (ip - ip0) == f.seg_offset[seg + 1];
  }
};

// BF16 word in bits 0..15 (bits above are unspecified): symbol bits | mantissa low 5 bits
// | sign << 15.  r6 * (1 + 2^10) puts the five mantissa bits at 0..4 and the sign at 15
// (a 24-bit multiply); the mask drops the copies that land elsewhere.
__device__ __forceinline__ uint32_t fused_word_bits(uint32_t hi, uint32_t r6) {
  return ((r6 * 0x401u) & 0x801Fu) | hi;
}

__device__ __forceinline__ void SegmentWalk::decode16(uint32_t t, uint32_t S, const FusedParams &q,
                                                     uint32_t (&pair)[8]) {
  Raw6x16 rr;
  rr.set(n0, n1, n2);
  const uint32_t cw[4] = {nc4.x, nc4.y, nc4.z, nc4.w};
  if (t + 16 < S) {
    const uint32_t *nx = rawp + (t / 16 + 1) * 3;
    n0 = nx[0];
    n1 = nx[1];
    n2 = nx[2];
    nc4 = ccp[t / 16 + 1];
  }
  uint32_t bits[16];
#define GRF_STEP(k)                                                            \
  {                                                                            \
    const uint32_t hi = fused_symbol<(k) % 4>(state, ip, cw[(k) / 4], q);      \
    bits[k] = fused_word_bits(hi, rr.field<k>());                              \
  }
  GRF_STEP(0) GRF_STEP(1) GRF_STEP(2) GRF_STEP(3) GRF_STEP(4) GRF_STEP(5) GRF_STEP(6) GRF_STEP(7)
  GRF_STEP(8) GRF_STEP(9) GRF_STEP(10) GRF_STEP(11) GRF_STEP(12) GRF_STEP(13) GRF_STEP(14) GRF_STEP(15)
#undef GRF_STEP
#pragma unroll
  for (int k = 0; k < 8; ++k) pair[k] = __builtin_amdgcn_perm(bits[2 * k + 1], bits[2 * k], 0x05040100u);
}

}  // namespace grf
