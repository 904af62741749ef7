// Context-codec entry points of the fused decode-GEMV (VALU dot products, 1 <= M <= 8)
// and of the store sink that backs decode() for fused frames.  Kernels: fused_kernels.h.
#include "fused_kernels.h"

namespace grf {
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who, TilingUse use, bool pointers) {
  auto bad = [&](const char *why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (pointers && (!f.main_bytes || !f.raw6 || !f.seg_state || !f.seg_offset || !g.tile_rows || !g.tile_class ||
                   !f.lut || !f.tab || !f.col_class))
    return bad("null pointer in frame");
  if (!f.rows || !f.cols || !g.n_tiles || !g.n_slabs) return bad("empty geometry");
  if (f.seg_len == 0 || f.seg_len % 16 || (uint64_t)f.seg_len * f.segs_per_row != f.cols)
    return bad("segment length must be a multiple of 16 that divides the row length");
  if (!g.threads || g.threads % 64 || g.threads > (uint32_t)grf::kFusedMaxThreads) return bad("thread count");
  // (row positions too stay below 2^24: they go up to the rows rounded up to 16, plus 16 per row class)
  if ((use == kGemmTiling || g.scheme == GRF_TILE_WAVES) &&
      ((uint64_t)f.rows + 16 + 16ull * f.nr >= (1u << 24) || f.cols >= (1u << 24)))
    return grf::set_error(GRF_UNSUPPORTED, std::string(who) + ": wave tilings take fewer than 2^24 rows and columns");
  if (use == kGemmTiling) {  // waves of 16 rows x 4 segments with their own stream pieces
    if (g.scheme != GRF_TILE_WAVES) return bad("the GEMM takes a wave tiling (piece_cap for pieces of four segments)");
    if (!g.lanes_per_row || !g.rows_per_tile) return bad("empty tile");
  } else if (g.scheme == GRF_TILE_WAVES) {
    if (use != kGemvTiling) return bad("this entry point takes slab tilings only");
    const uint32_t lanes = g.lanes_per_row;
    if (lanes < 4 || lanes > 64 || (lanes & (lanes - 1))) return bad("a wave unit has 4, 8, 16, 32 or 64 lanes per row");
    if (!g.rows_per_tile) return bad("empty tile");
  } else if (g.scheme != GRF_TILE_SLABS) {
    return bad("tiling scheme");
  } else if (!g.lanes_per_row || !g.rows_per_tile || g.lanes_per_row * g.rows_per_tile > g.threads) {
    return bad("tile does not fit one workgroup");
  }
  if (g.n_slabs != (f.segs_per_row + g.lanes_per_row - 1) / g.lanes_per_row) return bad("slab count mismatch");
  if (f.nc == 0 || f.nc > 16 || (f.nc & (f.nc - 1))) return bad("column class count");
  if (f.shift > 12 || f.lognb != 16 - f.shift) return bad("bucket shift");
  if (f.tabn == 0 || f.tabn > 255) return bad("sparse table size");
  if (g.piece_cap % 16 || g.piece_cap < 16) return bad("piece capacity");
  if ((uint64_t)f.rows * f.cols > 0xFFFFFFFFull) return bad("matrix too large");
  if (f.raw_interleaved > 16 || (f.raw_interleaved & (f.raw_interleaved - 1)))
    return bad("raw_interleaved is 0 or a block of 1, 2, 4, 8 or 16 rows");
  if (f.row_pos && !f.raw_interleaved) return bad("row positions belong to the interleaved residual order");
  return GRF_OK;
}

// What the kernels take on trust from the index and the tiling arrays, checked on host copies.
int validate_fused_host(const grf_bctx_fused &f, const grf_fused_tiling &g, TilingUse use, bool every_row,
                        const uint32_t *seg_offset, const uint32_t *tile_rows, const uint8_t *tile_class,
                        const uint8_t *row_class, const uint32_t *row_pos) {
  const char *who = "grf_bctx_fused_validate_host";
  auto bad = [&](const std::string &why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (int rc = check_fused_frame(f, g, who, use, false)) return rc;
  if (!seg_offset || !tile_rows || !tile_class) return bad("null array");
  const uint32_t spr = f.segs_per_row;
  // entry s (0..spr: the last is the row's end) of a row, in the order the frame structure says
  // the index has: the frame's own, or the blocked order of the residuals (fused_seg_slot)
  const uint32_t B = f.raw_interleaved;
  if (B && !row_pos) return bad("the blocked index order needs the rows' positions");
  if (row_pos) {  // positions first: the index is read through them
    const uint64_t limit = ((uint64_t)f.rows + 15) / 16 * 16 + 16ull * f.nr;  // every class may start on a multiple of 16
    for (uint32_t row = 0; row < f.rows; ++row)
      if (row_pos[row] >= limit) return bad("row " + std::to_string(row) + " has a position beyond the rows the order can hold");
  }
  auto entry = [&](uint32_t row, uint32_t s) -> uint32_t {
    if (!B) return seg_offset[(uint64_t)row * spr + s];
    const uint32_t q = row_pos[row], within = q % B;
    return seg_offset[(uint64_t)(q - within) * (spr + 1) + (uint64_t)s * B + within];
  };
  // the index: offsets never decrease, stay inside the stream and end on its length
  uint32_t lowest = 0xFFFFFFFFu, highest = 0;
  for (uint32_t row = 0; row < f.rows; ++row) {
    for (uint32_t s = 0; s < spr; ++s)
      if (entry(row, s) > entry(row, s + 1))
        return bad("segment offsets decrease at segment " + std::to_string(s) + " of row " + std::to_string(row));
    lowest = std::min(lowest, entry(row, 0));
    highest = std::max(highest, entry(row, spr));
  }
  if (lowest < 4) return bad("the first segment starts behind the stream's four-byte initial state");
  if (highest != f.main_n_bytes) return bad("the last index entry is not the stream's length");
  // the tiling: slots name rows of the matrix, every row once, one row class per tile
  const uint32_t k = use == kGemmTiling && g.k_parts > 1 ? g.k_parts : 1;
  if (g.n_tiles % k) return bad("tile count is not a multiple of k_parts");
  const uint32_t row_tiles = g.n_tiles / k;
  if (k > 1 && k > g.n_slabs) return bad("more parts than slabs");
  std::vector<uint8_t> seen(f.rows, 0);
  for (uint32_t t = 0; t < row_tiles; ++t) {
    if (tile_class[t] >= f.nr) return bad("tile class outside the frame's row classes");
    for (uint32_t r = 0; r < g.rows_per_tile; ++r) {
      const uint32_t row = tile_rows[(uint64_t)t * g.rows_per_tile + r];
      if (row == grf::kNoRow) continue;
      if (row >= f.rows) return bad("tile slot names row " + std::to_string(row) + ", which the matrix does not have");
      if (seen[row]++ && every_row) return bad("row " + std::to_string(row) + " appears in two slots");
      if (row_class && row_class[row] != tile_class[t])
        return bad("row " + std::to_string(row) + " is not of its tile's class");
    }
  }
  for (uint32_t row = 0; every_row && row < f.rows; ++row)
    if (!seen[row]) return bad("row " + std::to_string(row) + " is in no tile");
  // every stream piece a workgroup or wave stages fits the LDS reserved for it: from the
  // 16-byte aligned start of its first segment to the end of its last, plus the 8 bytes the
  // refill's window reads from the cursor on
  const uint32_t lanes = use == kGemmTiling ? 4u : g.lanes_per_row;
  std::vector<uint32_t> off(spr + 1);
  for (uint32_t row = 0; row < f.rows; ++row) {
    for (uint32_t s = 0; s <= spr; ++s) off[s] = entry(row, s);
    // the GEMM's waves start a piece of four segments at any multiple of four inside a slab,
    // and a slab at any multiple of lanes_per_row
    for (uint32_t b = 0; b < spr; b += g.lanes_per_row)
      for (uint32_t s = b; s < std::min(spr, b + g.lanes_per_row); s += lanes) {
        const uint32_t last = std::min(std::min(spr, b + g.lanes_per_row), s + lanes);
        const uint64_t span = (uint64_t)off[last] - (off[s] & ~15u) + 8;
        if (span > g.piece_cap)
          return bad("the stream piece of row " + std::to_string(row) + " from segment " + std::to_string(s) +
                     " needs " + std::to_string(span) + " bytes, piece_cap is " + std::to_string(g.piece_cap));
      }
  }
  if (row_pos) {  // one-to-one positions inside the residual array
    if (!f.raw_interleaved) return bad("row positions belong to the interleaved residual order");
    uint32_t top = 0;
    for (uint32_t row = 0; row < f.rows; ++row) top = std::max(top, row_pos[row]);
    if ((uint64_t)(top / f.raw_interleaved + 1) * f.raw_interleaved * f.cols > 0xFFFFFFFFull)
      return bad("row positions reach beyond a 32-bit element offset");
    std::vector<uint8_t> taken((size_t)top + 1, 0);
    for (uint32_t row = 0; row < f.rows; ++row)
      if (taken[row_pos[row]]++) return bad("two rows share residual position " + std::to_string(row_pos[row]));
  }
  uint32_t lds = 0;
  if (use == kGemmTiling) lds = GemmLdsLayout(f, g).total;
  else if (g.scheme == GRF_TILE_WAVES) lds = WaveLdsLayout(f, g, kWaveRowsPerPass).total;
  else lds = FusedLdsLayout(f, g, use == kGemvTiling ? 1 : 0).total;
  if (lds > 160 * 1024) return bad("the launch needs " + std::to_string(lds) + " bytes of LDS");
  return GRF_OK;
}
}  // namespace grf

extern "C" {

uint32_t grf_bctx_fused_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint32_t m_rows) {
  if (!frame || !tiling) return 0;
  if (tiling->scheme == GRF_TILE_WAVES)  // passes of at most two activation rows
    return grf::WaveLdsLayout(*frame, *tiling, m_rows < grf::kWaveRowsPerPass ? m_rows : grf::kWaveRowsPerPass).total;
  return grf::FusedLdsLayout(*frame, *tiling, m_rows).total;
}

int grf_bctx_fused_validate_host(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, int use,
                                 const uint32_t *seg_offset, const uint32_t *tile_rows, const uint8_t *tile_class,
                                 const uint8_t *row_class, const uint32_t *row_pos) {
  if (!frame || !tiling) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_validate_host: null argument");
  if (use < 0 || use > 3) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_validate_host: use is 0, 1, 2 or 3");
  try {
    const grf::TilingUse kind = use == 1 ? grf::kGemvTiling : use == 2 ? grf::kGemmTiling : grf::kSlabTiling;
    return grf::validate_fused_host(*frame, *tiling, kind, use != 3, seg_offset, tile_rows, tile_class, row_class,
                                    row_pos);
  } catch (...) {
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_validate_host: out of memory");
  }
}

int grf_bctx_gemv(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                  void *hip_stream) {
  if (!frame || !tiling || !x || !y || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv: null argument");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_gemv", grf::kGemvTiling)) return rc;
  return grf::launch_gemv<grf::SegmentWalk>("grf_bctx_gemv", *frame, *tiling, x, ldx, m_rows, y, ldy, bias, error,
                                            (hipStream_t)hip_stream);
}

int grf_bctx_fused_decode(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint16_t *out,
                          int32_t *error, void *hip_stream) {
  if (!frame || !tiling || !out || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_decode: null argument");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_fused_decode")) return rc;
  if (grf::reads_ahead(*frame))
    return grf::launch_walk<grf::SegmentWalkAhead, 1, grf::kStore>(*frame, *tiling, nullptr, 0, nullptr, 0, nullptr,
                                                                   out, error, (hipStream_t)hip_stream);
  return grf::launch_walk<grf::SegmentWalk, 1, grf::kStore>(*frame, *tiling, nullptr, 0, nullptr, 0, nullptr, out, error,
                                                            (hipStream_t)hip_stream);
}

int grf_bctx_fused_gather(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint16_t *out,
                          int32_t *error, void *hip_stream) {
  if (!frame || !tiling || !out || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_fused_gather: null argument");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_fused_gather")) return rc;
  return grf::launch_walk<grf::SegmentWalk, 1, grf::kGather>(*frame, *tiling, nullptr, 0, nullptr, 0, nullptr, out,
                                                             error, (hipStream_t)hip_stream);
}

}  // extern "C"
