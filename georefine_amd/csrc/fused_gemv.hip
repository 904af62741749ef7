// Context-codec entry points of the fused decode-GEMV (VALU dot products, 1 <= M <= 8)
// and of the store sink that backs decode() for fused frames.  Kernels: fused_kernels.h.
#include "fused_kernels.h"

namespace grf {
int check_fused_frame(const grf_bctx_fused &f, const grf_fused_tiling &g, const char *who, TilingUse use) {
  auto bad = [&](const char *why) { return grf::set_error(GRF_BAD_ARGUMENT, std::string(who) + ": " + why); };
  if (!f.main_bytes || !f.raw6 || !f.seg_state || !f.seg_offset || !g.tile_rows || !g.tile_class || !f.lut ||
      !f.tab || !f.col_class)
    return bad("null pointer in frame");
  if (!f.rows || !f.cols || !g.n_tiles || !g.n_slabs) return bad("empty geometry");
  if (f.seg_len == 0 || f.seg_len % 16 || (uint64_t)f.seg_len * f.segs_per_row != f.cols)
    return bad("segment length must be a multiple of 16 that divides the row length");
  if (!g.threads || g.threads % 64 || g.threads > (uint32_t)grf::kFusedMaxThreads) return bad("thread count");
  if ((use == kGemmTiling || g.scheme == GRF_TILE_WAVES) && (f.rows >= (1u << 24) || f.cols >= (1u << 24)))
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
}  // namespace grf

extern "C" {

uint32_t grf_bctx_fused_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, uint32_t m_rows) {
  if (!frame || !tiling) return 0;
  if (tiling->scheme == GRF_TILE_WAVES)  // passes of at most two activation rows
    return grf::WaveLdsLayout(*frame, *tiling, m_rows < grf::kWaveRowsPerPass ? m_rows : grf::kWaveRowsPerPass).total;
  return grf::FusedLdsLayout(*frame, *tiling, m_rows).total;
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
