// The fused decoder: one walker over a checkpointed segment whose decoded BF16
// words go to a sink (dot-product chain for the GEMV, LDS tile for the GEMM,
// global store for decode(); fused_kernels.h).  Because every sink is fed by the
// same walker, words proven bit-exact through the store sink are the words the
// fused sinks consume.
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
// symbol that owns most of the bucket's slots; that symbol's 8-byte entry is read and
// assumed to own the slot.  Entry: low32 = start | (freq & 0xFFFF)<<16 (0 stands for
// 65536), high32 = the symbol's bits in the BF16 word (symbol<<5 for this codec).  When a
// symbol boundary inside the bucket separates the slot from that symbol, a scan over the
// neighbouring entries finishes the search.
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

// Per column class the LDS holds one block: the sparse symbol table first (tabn + 1
// 8-byte entries: the symbols plus the entry a forward scan stops on), then the class's
// lookup bytes.  With the block base in a register the table read needs no further
// address arithmetic and the lookup read adds the uniform table size.
__host__ __device__ inline uint32_t fused_table_bytes(const grf_bctx_fused &f) { return align_up((f.tabn + 1) * 8, 16); }

// byte offsets of the LDS regions; shared by host (size) and device (carve).
struct FusedLdsLayout {
  uint32_t blocks, block_pitch, stream, xs, part, rowsum, total;
  __host__ __device__ FusedLdsLayout(const grf_bctx_fused &f, const grf_fused_tiling &g, uint32_t m) {
    uint32_t at = 0;
    blocks = at;
    block_pitch = fused_table_bytes(f) + (1u << f.lognb);
    at = align_up(at + f.nc * block_pitch, 16);
    stream = at;
    at = align_up(at + g.rows_per_tile * g.piece_cap, 16);
    xs = at;
    at = align_up(at + m * g.lanes_per_row * (f.seg_len + kXPad) * 2, 16);
    part = at;
    at = align_up(at + g.rows_per_tile * g.lanes_per_row * m * 4, 16);
    rowsum = at;
    at = align_up(at + g.rows_per_tile * m * 4, 16);
    total = at;
  }
};

typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef uint32_t v2u32 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2u32 lds_v2u32;

// LDS accesses by absolute byte offset (dynamic LDS starts at address 0 here:
// the kernels declare no static LDS)
__device__ __forceinline__ uint8_t lds_load_u8(uint32_t off) { return *reinterpret_cast<lds_u8 *>(off); }

struct FusedParams {  // uniform values the step needs, kept in scalar registers
  uint32_t shift, block_pitch, table_bytes;
  uint32_t whole_range;  // some context is one symbol of frequency 65536 (grf_bctx_fused.whole_range)
};
// Which scan the step carries for lanes that miss: the one that knows whole-range entries, or
// the shorter one for frames that promise to have none.
enum ScanKind : int { kScanAny = 0, kScanNoWholeRange = 1 };

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

// One decode step of the main stream against LDS tables.
//
// The lookup byte names the symbol that owns most slots of the slot's bucket.  With
// buckets finer than almost every symbol, that symbol nearly always owns the slot itself,
// so the step reads only its entry; a lane whose slot lies outside the entry (a symbol
// boundary inside the bucket, or the 16-bit frequency field's 0 = 65536) scans to the
// neighbouring entries before the state update, which all lanes then do together.
struct StepFetch {
  uint32_t win, ta;  // the next four stream bytes, first byte highest; table address of the entry
  v2u32 e0;
};

// A lane's position in one segment: rANS state and LDS cursor, the cursor in bits (eight times
// the byte address), which is the unit the refill's shift count comes in.
struct Cursor {
  uint32_t state, jb;
};

// `block` is the LDS offset of the column class's block (fused_block_offset).  The LDS
// returns data in issue order, so the lookup byte, on which the entry read waits, goes first.
__device__ __forceinline__ uint32_t fused_fetch_index(uint32_t state, uint32_t block, const FusedParams &q) {
  const uint32_t bucket = (state & 0xFFFFu) >> q.shift;
  return lds_load_u8(block + bucket + q.table_bytes);
}
// Refill bytes: one read of the two aligned dwords around the cursor serves two steps (they
// take at most four bytes); a funnel shift brings the byte at the cursor to the bottom and a
// byte permute turns the four around, so that `win` = stream bytes [ip, ip + 4) with the first
// byte highest: the order in which a refill shifts them into the state.  The lanes of a wave
// sit at scattered places of their pieces, so byte-wide reads (two per step) collide in the
// banks about as often as random addresses would, and were the largest share of the LDS time;
// a quarter as many reads leave the lookup and the entry read as the main LDS work.  (An
// unaligned 16- or 32-bit LDS read stalls the pipeline for tens of cycles on this hardware.)
typedef __attribute__((address_space(3))) uint32_t lds_u32;
__device__ __forceinline__ void fused_fetch_window(StepFetch &s, const Cursor &c) {
  const uint32_t a = (c.jb >> 3) & ~3u;
  const uint32_t lo = *reinterpret_cast<lds_u32 *>(a), hi = *reinterpret_cast<lds_u32 *>(a + 4);
  // the shift uses bits 0..4 of the cursor: (ip & 3) * 8
  s.win = __builtin_bswap32(__builtin_amdgcn_alignbit(hi, lo, c.jb));
}
// Keeps the window in the block that made it: left alone, the compiler sinks the funnel shift
// past the scan branch.
__device__ __forceinline__ void fused_pin_bytes(StepFetch &s) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(s.win));
#endif
}
__device__ __forceinline__ void fused_fetch_entry(StepFetch &s, uint32_t idx, uint32_t block) {
  s.ta = fused_lshl3_add(idx, block);
  s.e0 = *reinterpret_cast<lds_v2u32 *>(s.ta);
}

// rel = slot - start of the entry; `miss` = the lanes whose slot the entry does not hold
__device__ __forceinline__ uint32_t fused_locate(uint32_t state, uint32_t e_lo, uint64_t &miss) {
  uint32_t rel;
#if defined(__HIP_DEVICE_COMPILE__)
  asm("v_sub_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_0"
      : "=v"(rel)
      : "v"(state), "v"(e_lo));
  asm("v_cmp_ge_u32_sdwa %0, %1, %2 src0_sel:DWORD src1_sel:WORD_1" : "=s"(miss) : "v"(rel), "v"(e_lo));
#else
  rel = (state & 0xFFFFu) - (e_lo & 0xFFFFu);
  miss = rel >= (e_lo >> 16);
#endif
  return rel;
}

__device__ __forceinline__ bool fused_lane_in(uint64_t mask) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_inverse_ballot_w64(mask);
#else
  return mask != 0;
#endif
}

// For the lanes that missed: from the entry at `s.ta`, whose `rel` (slot - start, as a signed
// number) says which way to go, step to the entry that holds the slot; the entry in hand is
// known not to hold it, so the step comes first and the test after.  The tables cover every
// slot (the host checks that the frequencies of a context add up to 65536), so the scan ends;
// the trip limit only keeps a wave from spinning on tables that were overwritten.
constexpr uint32_t kScanTrips = 256;  // entries a table can have (its index is a byte)
__device__ __forceinline__ void fused_scan(uint32_t state, StepFetch &s, uint32_t &rel) {
  const uint32_t slot = state & 0xFFFFu;
  uint32_t ta = s.ta;
  v2u32 e = s.e0;
  uint32_t left = kScanTrips;
  do {
    ta += (int32_t)rel < 0 ? -8 : 8;
    e = *reinterpret_cast<lds_v2u32 *>(ta);
    rel = slot - (e.x & 0xFFFFu);
  } while (rel >= (e.x >> 16) && --left);
  s.e0 = e;
}
// The same for frames in which a context may be a single symbol of frequency 65536 (field 0,
// start 0): such an entry always reports a miss and is not left; it returns rel = state, so
// that the update freq16 * (state >> 16) + rel leaves the state as it is.
// The trip limit is the other scan's: a table has at most 256 entries, so a scan that has
// not ended by then is walking memory that is not a table; the segment then misses its
// checkpoint and the launch reports GRF_ERR_CHECKPOINT instead of spinning.
__device__ __forceinline__ void fused_scan_whole(uint32_t state, StepFetch &s, uint32_t &rel) {
  const uint32_t slot = state & 0xFFFFu;
  uint32_t ta = s.ta;
  v2u32 e = s.e0;
  for (uint32_t left = kScanTrips; left; --left) {
    const uint32_t freq = e.x >> 16;
    rel = slot - (e.x & 0xFFFFu);
    if (freq == 0) rel = state;
    if (freq == 0 || rel < freq) break;
    ta += (int32_t)rel < 0 ? -8 : 8;
    e = *reinterpret_cast<lds_v2u32 *>(ta);
  }
  s.e0 = e;
}

// state' = freq * (state >> 16) + rel, then the refill: n = 0, 1 or 2 bytes are shifted in
// while the state is below 2^23.  Without branches or condition registers: the state is
// below 2^31 and at least 2^7, so 8 n = (clz(state') - 1) & 24, and one 64-bit shift of
// state' : window by that count moves the bytes into the state and out of the window.
__device__ __forceinline__ void fused_advance(Cursor &c, StepFetch &s, uint32_t rel) {
  uint32_t x;
#if defined(__HIP_DEVICE_COMPILE__)
  asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[1,1,0,0]" : "=v"(x) : "v"(s.e0.x), "v"(c.state), "v"(rel));
#else
  x = (s.e0.x >> 16) * (c.state >> 16) + rel;
#endif
  const uint32_t bits = ((uint32_t)__builtin_clz(x) - 1u) & 24u;
  const uint64_t both = (((uint64_t)x << 32) | s.win) << bits;
  c.state = (uint32_t)(both >> 32);
  s.win = (uint32_t)both;
  c.jb += bits;
}

// Two consecutive steps of one segment, given the LDS offsets of their contexts' table blocks.
// Returns the images of the two symbols' bits in the BF16 word (symbol << 5).
template <int SCAN>
__device__ __forceinline__ uint32_t fused_finish_step(Cursor &c, StepFetch &s, uint32_t idx, uint32_t block) {
  fused_fetch_entry(s, idx, block);
  fused_pin_bytes(s);
  uint64_t miss;
  uint32_t rel = fused_locate(c.state, s.e0.x, miss);
  // a branch on the whole mask first: the common path then leaves EXEC alone
  if (__builtin_expect(miss != 0, 0)) {
    if (fused_lane_in(miss)) {
      if constexpr (SCAN == kScanNoWholeRange)
        fused_scan(c.state, s, rel);
      else
        fused_scan_whole(c.state, s, rel);
    }
  }
  fused_advance(c, s, rel);
  return s.e0.y;
}
template <int SCAN = kScanAny>
__device__ __forceinline__ void fused_symbol_pair_in(Cursor &c, uint32_t block0, uint32_t block1, const FusedParams &q,
                                                     uint32_t &hi0, uint32_t &hi1) {
  StepFetch s;
  const uint32_t idx0 = fused_fetch_index(c.state, block0, q);
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_sched_barrier(0);  // the lookup byte first: the LDS answers in issue order and the step waits for it
#endif
  fused_fetch_window(s, c);
  hi0 = fused_finish_step<SCAN>(c, s, idx0, block0);
  const uint32_t idx1 = fused_fetch_index(c.state, block1, q);
  hi1 = fused_finish_step<SCAN>(c, s, idx1, block1);
}
template <int K, int SCAN = kScanAny>
__device__ __forceinline__ void fused_symbol_pair(Cursor &c, uint32_t ccw, const FusedParams &q, uint32_t &hi0,
                                                  uint32_t &hi1) {
  fused_symbol_pair_in<SCAN>(c, fused_block_offset<K % 4>(ccw, q.block_pitch), fused_block_offset<K % 4 + 1>(ccw, q.block_pitch),
                       q, hi0, hi1);
}

// Sixteen packed 6-bit residuals (12 bytes, MSB first) -> field k, k compile-time, sign
// extended: bits 0..4 are the mantissa's low bits, every bit from 5 up copies the sign.
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
      return (uint32_t)__builtin_amdgcn_sbfe((int32_t)a, 32 - 6 - off, 6);
    } else {
      const uint32_t b = word == 0 ? w1 : w2;
      return (uint32_t)__builtin_amdgcn_sbfe((int32_t)__builtin_amdgcn_alignbit(a, b, 64 - 6 - off), 0, 6);
    }
  }
};

// ---- pieces of the tile walk shared by the GEMV and GEMM kernels ----

// Entry `i` of the segment index (states or offsets).  The arrays have at most 2^28 + 1 entries
// (a segment is at least 16 symbols), so the byte offset fits 32 bits: the load then takes the
// array's base from a scalar pair and the offset from one register, with no 64-bit address
// arithmetic per lane.
__device__ __forceinline__ uint32_t fused_index_entry(const uint32_t *index, uint32_t i) {
  return *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint8_t *>(index) + (i << 2));
}

// this row class's lookup tables -> LDS, one block per column class: table, then lookup bytes.
// A thread issues all of its loads of a pass (four 16-byte units of the lookups, four 8-byte
// entries) before it stores any of them: a loop whose trip count the compiler does not know
// runs its loads one round trip after the other, which cost a workgroup seven of them (about
// 5 us) before its first step.  Loads past the end read the last unit again; only the store
// is conditional.
__device__ __forceinline__ void fused_load_tables(uint8_t *lds, uint32_t blocks, uint32_t block_pitch,
                                                  const grf_bctx_fused &f, uint32_t cls, uint32_t tid,
                                                  uint32_t nthreads) {
  const uint32_t nb16 = (1u << f.lognb) / 16, entries = f.tabn + 1, tb = fused_table_bytes(f);
  const uint4 *lut = reinterpret_cast<const uint4 *>(f.lut + (size_t)cls * f.nc * (nb16 * 16));
  const uint2 *tab = reinterpret_cast<const uint2 *>(f.tab) + (size_t)cls * f.nc * entries;
  const uint32_t n16 = f.nc * nb16, n8 = f.nc * entries;
  constexpr int kInFlight = 4;
  for (uint32_t base = 0; base < max(n16, n8); base += kInFlight * nthreads) {  // uniform
    uint4 a[kInFlight];
    uint2 e[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      const uint32_t i = base + k * nthreads + tid;
      a[k] = lut[min(i, n16 - 1)];
      e[k] = tab[min(i, n8 - 1)];
    }
#if defined(__HIP_DEVICE_COMPILE__)
    // (keeps the loads above the stores: the compiler would sink each into its store's branch)
#pragma unroll
    for (int k = 0; k < kInFlight; ++k)
      asm volatile("" : "+v"(a[k].x), "+v"(a[k].y), "+v"(a[k].z), "+v"(a[k].w), "+v"(e[k].x), "+v"(e[k].y));
#endif
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      const uint32_t i = base + k * nthreads + tid;
      if (i < n16) *reinterpret_cast<uint4 *>(lds + blocks + (i / nb16) * block_pitch + tb + (i % nb16) * 16) = a[k];
      if (i < n8) *reinterpret_cast<uint2 *>(lds + blocks + (i / entries) * block_pitch + (i % entries) * 8) = e[k];
    }
  }
}

// The same tables copied without vector registers, by loads that write the LDS directly, the
// waves taking the copy's 1 KiB (lookup bytes) and 256-byte (entries, which are only 8-byte
// aligned) chunks in turn.  Nothing waits here: the copy is issued first thing in a workgroup
// and is under way while the reads that lead to the first unit's stream bytes follow one
// another; it is complete at the workgroup's barrier.  For lookups of at least 1 KiB a column
// class (a chunk must not straddle two classes' blocks).
__device__ __forceinline__ bool fused_tables_by_dma(const grf_bctx_fused &f) { return f.lognb >= 10; }
__device__ __forceinline__ void fused_load_tables_dma(uint8_t *lds, uint32_t blocks, uint32_t block_pitch,
                                                      const grf_bctx_fused &f, uint32_t cls, uint32_t wave,
                                                      uint32_t nwaves, uint32_t lane) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(3))) void lds_void;
  const uint32_t lut_bytes = 1u << f.lognb, tab_bytes = (f.tabn + 1) * 8, tb = fused_table_bytes(f);
  const uint8_t *lut = f.lut + (size_t)cls * f.nc * lut_bytes;
  const uint8_t *tab = reinterpret_cast<const uint8_t *>(f.tab) + (size_t)cls * f.nc * tab_bytes;
  const uint32_t lut_chunks = lut_bytes >> 10, tab_chunks = (tab_bytes + 255) >> 8;  // of one column class
  const uint32_t n_lut = f.nc * lut_chunks, n_tab = f.nc * tab_chunks;
  for (uint32_t c = wave; c < n_lut + n_tab; c += nwaves) {  // uniform
    if (c < n_lut) {
      const uint32_t cc = c / lut_chunks, k = c - cc * lut_chunks;
      __builtin_amdgcn_global_load_lds(lut + (cc * lut_bytes + k * 1024 + lane * 16),
                                       (lds_void *)(lds + (blocks + cc * block_pitch + tb + k * 1024)), 16, 0, 0);
    } else {
      const uint32_t t = c - n_lut, cc = t / tab_chunks, k = t - cc * tab_chunks;
      const uint32_t o = k * 256 + lane * 4;
      if (o < tab_bytes)
        __builtin_amdgcn_global_load_lds(tab + (cc * tab_bytes + o), (lds_void *)(lds + (blocks + cc * block_pitch + k * 256)),
                                         4, 0, 0);
    }
  }
#else
  (void)lds, (void)blocks, (void)block_pitch, (void)f, (void)cls, (void)wave, (void)nwaves, (void)lane;
#endif
}

// Where the checkpoint of a segment lies in the index arrays (seg_state, seg_offset).  In the
// frame's order (raw_interleaved == 0) segment s of row r is entry r * segs_per_row + s and its
// end is the entry after it.  In the blocked order the residuals have (raw_interleaved = B rows
// per block, rows by position) every row has segs_per_row + 1 entries -- the last one is the end
// of its stream -- and entry s of position q lies at ((q / B) * (segs_per_row + 1) + s) * B + q % B:
// the entries that a wave unit, or the sixteen rows of a GEMM wave, read at one visit are then
// one run of bytes, as its residuals are, instead of a few bytes out of every row's own line.
// `row`, rpos: the row and its position, s: the segment in its row.  The entry of the
// segment's end is fused_seg_step further on.  NARROW: rows and segments per row are below
// 2^24 (wave tilings), so the products take the full-rate 24-bit multiply.
template <bool NARROW = false>
__device__ __forceinline__ uint32_t fused_seg_slot(const grf_bctx_fused &f, uint32_t row, uint32_t rpos, uint32_t s) {
  auto mul = [](uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (NARROW) return (uint32_t)__umul24(a, b);
#endif
    return a * b;
  };
  if (!f.raw_interleaved) return mul(row, f.segs_per_row) + s;
  const uint32_t B = f.raw_interleaved, within = rpos & (B - 1);
  return mul(rpos - within, f.segs_per_row + 1) + mul(s, B) + within;
}
__device__ __forceinline__ uint32_t fused_seg_step(const grf_bctx_fused &f) {
  return f.raw_interleaved ? f.raw_interleaved : 1u;
}

// Byte range of one row piece (segments [s, s + nseg) of a row) in the main stream.  The
// kernels fetch it one slab ahead: it is the first of two dependent global reads before a
// slab's bytes can be copied.
struct PieceSpan {
  uint32_t g0, g1;
  __device__ __forceinline__ void fetch(const grf_bctx_fused &f, uint32_t row, uint32_t rpos, uint32_t s,
                                        uint32_t nseg) {
    const uint32_t slot = fused_seg_slot(f, row, rpos, s);
    g0 = fused_index_entry(f.seg_offset, slot);
    g1 = fused_index_entry(f.seg_offset, slot + nseg * fused_seg_step(f));
  }
};

// Copy the main-stream bytes of one row piece to LDS at piece_off, keeping the 16-byte
// phase of the global address.  The P lanes of the row share the copy.  Returns the
// aligned global start so lanes can place their cursors.
__device__ __forceinline__ uint32_t fused_stage_piece(uint8_t *lds, uint32_t piece_off, const grf_bctx_fused &f,
                                                      const PieceSpan &span, uint32_t p, uint32_t P) {
  const uint32_t a0 = span.g0 & ~15u;
  // read once: a streaming load, so that these bytes do not push the residual lines, which
  // a lane touches four times over a segment, out of the L2
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  for (uint32_t o = a0 + p * 16; o < span.g1; o += P * 16)
    *reinterpret_cast<u32x4 *>(lds + piece_off + (o - a0)) =
        __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(f.main_bytes + o));
  return a0;
}

// The same copy made by one wave for itself (wave-unit tiling), without vector registers: the
// loads write the LDS directly.  Such a load puts the 16 bytes of lane l at (base + 16 * l) of
// a wave-uniform base, whatever address the lane read, so one instruction moves up to 1 KiB of
// consecutive bytes: the rows of the unit take turns, all 64 lanes copying one row's piece
// (its byte range, which the row's own lanes hold, is handed to the others through scalar
// registers).  A piece longer than 1 KiB takes further rounds.  The bytes are in the LDS when
// the wave's vector-memory counter says so; lanes of the same wave read them afterwards.
// (Sixteen lanes per instruction, each row served by its own lanes, took four times as many
// instructions, and a wave spent 2 us per unit issuing them.)
__device__ __forceinline__ uint32_t fused_stage_piece_dma(uint8_t *lds, uint32_t region0, uint32_t cap,
                                                          const grf_bctx_fused &f, uint32_t g0, uint32_t g1, uint32_t lane,
                                                          uint32_t logp, uint32_t rows_per_wave) {
  typedef __attribute__((address_space(3))) void lds_void;
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t rounds = (cap + 1023) >> 10;  // uniform: a figure of the tiling
  for (uint32_t r = 0; r < rows_per_wave; ++r) {  // uniform
    const uint32_t s0 = __builtin_amdgcn_readlane(g0, r << logp) & ~15u, s1 = __builtin_amdgcn_readlane(g1, r << logp);
    for (uint32_t i = 0; i < rounds; ++i) {
      const uint32_t o = s0 + (i * 64 + lane) * 16;
      if (o < s1)
        __builtin_amdgcn_global_load_lds(f.main_bytes + o, (lds_void *)(lds + (region0 + r * cap + i * 1024)), 16, 0, 0);
    }
  }
#else
  (void)lds, (void)region0, (void)cap, (void)f, (void)g1, (void)lane, (void)logp, (void)rows_per_wave;
#endif
  return g0 & ~15u;
}

// BF16 word in bits 0..15 (bits above are unspecified): symbol bits | mantissa low 5 bits
// | sign << 15, from the sign-extended residual field: its copy of the sign at bit 15 and
// its low five bits are kept, one and-or.
__device__ __forceinline__ uint32_t fused_word_bits(uint32_t hi, uint32_t r6_sign_extended) {
  return (r6_sign_extended & 0x801Fu) | hi;
}

// A lane's walk over one segment: rANS cursor, plus the registers that hold the packed
// residuals and the column classes of the next 16 symbols.  AHEAD (segments of 64 symbols
// only): the residuals of the whole segment, 48 bytes, are read when the segment starts; a
// line of the residual section is then fetched once instead of on four visits a group
// apart, between which the L2 may have dropped it.
template <bool AHEAD>
struct SegmentWalkT {
  static constexpr bool kAhead = AHEAD;
  Cursor c;
  uint32_t gofs, eofs;        // byte offsets of this segment's and the next segment's checkpoints
  uint32_t end_state, end_jb;  // what the walk must end on: the next checkpoint's state, and its offset as an LDS cursor
  const uint8_t *raw_base, *cc_base;  // the frame's residual and class arrays (uniform)
  uint32_t raw_off, cc_off;           // byte offsets of this segment's first group in them
  uint32_t raw_stride;                // bytes from a group's residuals to the next group's
  uint32_t n0, n1, n2;             // !AHEAD: the next group's residual words
  uint32_t rw[AHEAD ? 12 : 1];     // AHEAD: the segment's residual words
  uint4 nc4;
  Raw6x16 rr;      // the group being decoded
  uint32_t cw[4];

  // Global reads for the segment whose checkpoint is entry `slot_` of the index arrays
  // (fused_seg_slot; elem0 / col0: its first element / column; seg_in_row = col0 / seg_len,
  // which the caller has without dividing; rpos: the row's position in the residual array,
  // f.row_pos[row] or the row itself), issued before the wait for the stream bytes so that
  // their latency overlaps it.
  // (A matrix has fewer than 2^32 elements, so element and byte offsets are 32-bit numbers.)
  __device__ __forceinline__ void prefetch(const grf_bctx_fused &f, uint32_t slot_, uint32_t elem0, uint32_t col0,
                                           uint32_t seg_in_row, uint32_t rpos) {
    const uint32_t slot = slot_, next = slot + fused_seg_step(f);
    gofs = fused_index_entry(f.seg_offset, slot);
    eofs = fused_index_entry(f.seg_offset, next);
    c.state = fused_index_entry(f.seg_state, slot);
    end_state = fused_index_entry(f.seg_state, next);
    // a uniform base plus a 32-bit lane offset: the loads then take their address from a scalar
    // pair and one vector register, and no 64-bit address is worked out per group
    raw_base = f.raw6;
    cc_base = f.col_class;
    if (f.raw_interleaved) {
      // blocks of B rows (by position); inside a block the groups by position in the segment,
      // then by segment, then by row: group t of segment s of position q at
      // ((q / B * G + t) * segs_per_row + s) * B + q % B, G = seg_len / 16 groups per segment
      const uint32_t B = f.raw_interleaved, within = rpos & (B - 1);
      const uint32_t group = (rpos - within) * (f.cols / 16) + seg_in_row * B + within;  // (once per segment)
      raw_off = ((group << 1) + group) << 2;  // * 12
      raw_stride = f.segs_per_row * B * 12;
    } else {
      raw_off = elem0 / 4 * 3;
      raw_stride = 12;
    }
    cc_off = col0;
    if constexpr (AHEAD) {
      const uint4 *r4 = reinterpret_cast<const uint4 *>(raw_base + raw_off);  // 48-byte groups: 16-byte aligned
      const uint4 a = r4[0], b = r4[1], d = r4[2];
      rw[0] = a.x, rw[1] = a.y, rw[2] = a.z, rw[3] = a.w;
      rw[4] = b.x, rw[5] = b.y, rw[6] = b.z, rw[7] = b.w;
      rw[8] = d.x, rw[9] = d.y, rw[10] = d.z, rw[11] = d.w;
    } else {
      const uint32_t *r = reinterpret_cast<const uint32_t *>(raw_base + raw_off);
      n0 = r[0];
      n1 = r[1];
      n2 = r[2];
    }
    nc4 = *reinterpret_cast<const uint4 *>(cc_base + cc_off);
  }
  // the row piece was staged at piece_off from global offset a0
  __device__ __forceinline__ void start(uint32_t piece_off, uint32_t a0) {
    c.jb = (piece_off + (gofs - a0)) << 3;
    end_jb = c.jb + ((eofs - gofs) << 3);
  }

  // Start the group of symbols [t, t+16): unpack its residuals and column classes, and load
  // the registers of the following group meanwhile.
  __device__ __forceinline__ void begin16(uint32_t t, uint32_t S) {
    cw[0] = nc4.x;
    cw[1] = nc4.y;
    cw[2] = nc4.z;
    cw[3] = nc4.w;
    // the last group loads itself again rather than branch around the loads
    const uint32_t next = min(t / 16 + 1, S / 16 - 1);
    nc4 = *reinterpret_cast<const uint4 *>(cc_base + (cc_off + next * 16));
    if constexpr (AHEAD) {  // the words of the groups still to come move down one group
      rr.set(rw[0], rw[1], rw[2]);
#pragma unroll
      for (int i = 0; i < 9; ++i) rw[i] = rw[i + 3];
    } else {
      rr.set(n0, n1, n2);
      const uint32_t *nx = reinterpret_cast<const uint32_t *>(raw_base + (raw_off + next * raw_stride));
      n0 = nx[0];
      n1 = nx[1];
      n2 = nx[2];
    }
  }
  // Half H (0 or 1) of the group: eight symbols into four BF16 pairs (word k in the low
  // half, k+1 in the high half).
  template <int H, int SCAN = kScanAny>
  __device__ __forceinline__ void half(const FusedParams &q, uint32_t (&pair)[4]) {
    uint32_t bits[8];
#define GRF_STEP2(i)                                                                   \
  {                                                                                    \
    uint32_t h0, h1;                                                                   \
    fused_symbol_pair<8 * H + (i), SCAN>(c, cw[(8 * H + (i)) / 4], q, h0, h1);         \
    bits[i] = fused_word_bits(h0, rr.field<8 * H + (i)>());                            \
    bits[(i) + 1] = fused_word_bits(h1, rr.field<8 * H + (i) + 1>());                  \
  }
    GRF_STEP2(0) GRF_STEP2(2) GRF_STEP2(4) GRF_STEP2(6)
#undef GRF_STEP2
#pragma unroll
    for (int k = 0; k < 4; ++k) pair[k] = __builtin_amdgcn_perm(bits[2 * k + 1], bits[2 * k], 0x05040100u);
  }
  // Symbols [t, t+16) of the segment into eight BF16 pairs.
  __device__ __forceinline__ void decode16(uint32_t t, uint32_t S, const FusedParams &q, uint32_t (&pair)[8]) {
    begin16(t, S);
    half<0>(q, reinterpret_cast<uint32_t (&)[4]>(pair[0]));
    half<1>(q, reinterpret_cast<uint32_t (&)[4]>(pair[4]));
  }

  // the segment must end exactly on the next checkpoint
  __device__ __forceinline__ bool ended_on_checkpoint(const grf_bctx_fused &f) const {
    (void)f;
    return c.state == end_state && c.jb == end_jb;
  }
};
using SegmentWalk = SegmentWalkT<false>;
using SegmentWalkAhead = SegmentWalkT<true>;

}  // namespace grf
