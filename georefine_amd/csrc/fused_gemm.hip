// Context-codec entry points of the fused decode-GEMM on the matrix cores.  Kernels:
// fused_kernels.h.
#include "fused_kernels.h"

extern "C" {

uint32_t grf_bctx_gemm_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling) {
  if (!frame || !tiling) return 0;
  return grf::gemm_lds_bytes(*frame, *tiling);
}

size_t grf_gemm_workspace_bytes(uint32_t cols, uint32_t m_rows) { return grf::gemm_workspace_bytes(cols, m_rows); }

int grf_pack_activations(const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint32_t cols, void *workspace,
                         size_t workspace_bytes, void *hip_stream) {
  return grf::pack_rows("grf_pack_activations", x, ldx, m_rows, cols, workspace, workspace_bytes,
                        (hipStream_t)hip_stream);
}

int grf_bctx_gemm(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                  uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, void *workspace,
                  size_t workspace_bytes, int32_t *error, void *hip_stream) {
  if (!frame || !tiling || !y || !error)  // x may be null: rows packed by grf_pack_activations
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm: null argument");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_gemm")) return rc;
  return grf::launch_gemm<grf::SegmentWalk>("grf_bctx_gemm", *frame, *tiling, x, ldx, m_rows, y, ldy, bias, workspace,
                                            workspace_bytes, error, (hipStream_t)hip_stream);
}

int grf_bctx_gemv_group(uint32_t n, const grf_bctx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint16_t *const *y, const uint32_t *ldy,
                        const uint16_t *const *bias, int32_t *error, void *hip_stream) {
  if (!error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemv_group: null argument");
  const grf::GroupSpec spec{n, frames, tilings, y, ldy, bias};
  return grf::launch_gemv_group<grf::SegmentWalk>("grf_bctx_gemv_group", spec, x, ldx, m_rows, error,
                                                  (hipStream_t)hip_stream);
}

int grf_bctx_gemm_group(uint32_t n, const grf_bctx_fused *const *frames, const grf_fused_tiling *const *tilings,
                        const uint16_t *x, uint32_t ldx, uint32_t m_rows, uint16_t *const *y, const uint32_t *ldy,
                        const uint16_t *const *bias, void *workspace, size_t workspace_bytes, int32_t *error,
                        void *hip_stream) {
  if (!error) return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm_group: null argument");
  const grf::GroupSpec spec{n, frames, tilings, y, ldy, bias};
  return grf::launch_gemm_group<grf::SegmentWalk>("grf_bctx_gemm_group", spec, x, ldx, m_rows, workspace,
                                                  workspace_bytes, error, (hipStream_t)hip_stream);
}

}  // extern "C"
