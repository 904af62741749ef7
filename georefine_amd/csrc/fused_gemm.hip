// Context-codec entry points of the fused decode-GEMM on the matrix cores.  Kernels:
// fused_kernels.h.
#include "fused_kernels.h"

namespace {

// Scratch of the entry point that allocates nothing: the packed activations of one launch.
// Every GPU the library runs on holds its own copy of this array from the moment the code
// object is loaded there until the process ends.
constexpr size_t kScratchBytes = 8u << 20;
static __device__ __align__(256) uint8_t scratch[kScratchBytes];

// The array's address on the current device.  In host code `scratch` is only a stand-in for
// the symbol, not a device address: the address is asked for once per device and kept.
int scratch_address(void **out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void *> address[kMaxDevices];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return grf::set_error(GRF_LAUNCH_FAILED, "grf_bctx_gemm_noalloc: no current device");
  void *ptr = address[dev].load(std::memory_order_acquire);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return grf::set_error(GRF_LAUNCH_FAILED,
                            std::string("grf_bctx_gemm_noalloc: scratch address: ") + hipGetErrorString(e));
    address[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return GRF_OK;
}

}  // namespace

extern "C" {

uint32_t grf_bctx_gemm_lds_bytes(const grf_bctx_fused *frame, const grf_fused_tiling *tiling) {
  if (!frame || !tiling) return 0;
  return grf::gemm_lds_bytes(*frame, *tiling);
}

size_t grf_gemm_workspace_bytes(uint32_t cols, uint32_t m_rows) { return grf::gemm_workspace_bytes(cols, m_rows); }
size_t grf_gemm_workspace_bytes_split(uint32_t cols, uint32_t rows, uint32_t k_parts, uint32_t m_rows) {
  return grf::gemm_workspace_bytes_split(cols, rows, k_parts, m_rows);
}

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
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_gemm", grf::kGemmTiling)) return rc;
  return grf::launch_gemm<grf::SegmentWalk>("grf_bctx_gemm", *frame, *tiling, x, ldx, m_rows, y, ldy, bias, workspace,
                                            workspace_bytes, error, (hipStream_t)hip_stream);
}

size_t grf_gemm_noalloc_limit_bytes(void) { return kScratchBytes; }

int grf_bctx_gemm_noalloc(const grf_bctx_fused *frame, const grf_fused_tiling *tiling, const uint16_t *x, uint32_t ldx,
                          uint32_t m_rows, uint16_t *y, uint32_t ldy, const uint16_t *bias, int32_t *error,
                          void *hip_stream) {
  if (!frame || !tiling || !x || !y || !error)
    return grf::set_error(GRF_BAD_ARGUMENT, "grf_bctx_gemm_noalloc: null argument");
  if (grf::gemm_workspace_bytes_split(frame->cols, frame->rows, tiling->k_parts, m_rows) > kScratchBytes)
    return grf::set_error(GRF_UNSUPPORTED,
                          "grf_bctx_gemm_noalloc: the packed activations (and partial sums) of one launch exceed the "
                          "8 MiB scratch (grf_gemm_workspace_bytes_split(cols, rows, k_parts, m_rows) > "
                          "grf_gemm_noalloc_limit_bytes()); use grf_bctx_gemm with a workspace");
  if (int rc = grf::check_fused_frame(*frame, *tiling, "grf_bctx_gemm_noalloc", grf::kGemmTiling)) return rc;
  void *ptr = nullptr;
  if (int rc = scratch_address(&ptr)) return rc;
  // every launch writes all it reads of the scratch (its rows, zero rows up to the tile, the
  // chunk of zeros after the last column), so nothing of an earlier call shows through
  return grf::launch_gemm<grf::SegmentWalk>("grf_bctx_gemm_noalloc", *frame, *tiling, x, ldx, m_rows, y, ldy, bias, ptr,
                                            kScratchBytes, error, (hipStream_t)hip_stream);
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
