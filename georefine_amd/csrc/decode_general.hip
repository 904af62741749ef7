// General decode kernels: one lane per checkpointed segment, any stride, any
// geometry (segments may cross rows), every frame mode.  These are the
// always-correct paths behind decode() and gather_rows(); the fused kernels
// cover the aligned shapes the linear layers use.
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "georefine_amd.h"
#include "rans_device.h"

namespace grf {
thread_local std::string g_error;
int set_error(int code, const std::string &what) {
  g_error = what;
  return code;
}
}  // namespace grf

namespace {

int fail(int code, const std::string &what) { return grf::set_error(code, what); }

constexpr int kThreads = 256;

// MODE128: residual is a second rANS stream whose context is the main symbol.
// Index of element (row, col) among the packed 6-bit fields: the frame's own order, or, for
// a tensor that keeps them for the fused kernels, groups of 16 in blocks of rows, ordered by
// their position in the segment, the segment's number and the row inside the block.
__device__ __forceinline__ uint64_t raw6_index(const grf_bctx_frame &f, uint32_t row, uint32_t col) {
  if (!f.raw6_segment) return (uint64_t)row * f.cols + col;
  const uint32_t S = f.raw6_segment, spr = f.cols / S, B = f.raw6_block_rows ? f.raw6_block_rows : 1;
  const uint32_t q = f.raw6_row_pos ? f.raw6_row_pos[row] : row, within = q % B;
  const uint64_t group = (uint64_t)(q - within) * (f.cols / 16) + ((uint64_t)((col % S) / 16) * spr + col / S) * B + within;
  return group * 16 + col % 16;
}

template <bool MODE128>
__global__ __launch_bounds__(kThreads) void bctx_decode_kernel(grf_bctx_frame f, const int64_t *block_ids,
                                                                uint32_t count, uint16_t *out, int32_t *error) {
  const uint32_t lane = blockIdx.x * kThreads + threadIdx.x;
  if (lane >= count) return;
  const uint64_t n = (uint64_t)f.rows * f.cols;
  const uint64_t segments = (n + f.stride - 1) / f.stride;
  uint64_t block = block_ids ? (uint64_t)block_ids[lane] : lane;
  uint32_t bad = 0;
  if (block >= segments) {  // caller error: decode nothing, flag it
    atomicOr(error, GRF_ERR_CHECKPOINT);
    return;
  }
  const uint64_t start = block * f.stride;
  uint32_t row = (uint32_t)(start / f.cols), col = (uint32_t)(start % f.cols);
  uint32_t state = f.main.states[block], ip = f.main.offsets[block];
  uint32_t rstate = 0, rip = 0;
  if (MODE128) {
    rstate = f.residual.states[block];
    rip = f.residual.offsets[block];
  }
  const uint32_t steps = (uint32_t)(start + f.stride <= n ? f.stride : n - start);
  uint16_t *dst = out + (uint64_t)lane * f.stride;
  for (uint32_t t = 0; t < steps; ++t) {
    const uint32_t ctx = (uint32_t)f.row_class[row] * f.nc + f.col_class[col];
    const uint32_t m = grf::rans_step_global(state, ip, f.main.bytes, f.main.n_bytes,
                                             f.main.cum + (size_t)ctx * 1025, f.main.bucket + (size_t)ctx * 256, bad);
    uint32_t r;
    if (MODE128)
      r = grf::rans_step_global(rstate, rip, f.residual.bytes, f.residual.n_bytes,
                                f.residual.cum + (size_t)m * 65, f.residual.bucket + (size_t)m * 256, bad);
    else
      r = grf::packed_field<6>(f.residual.bytes, f.residual.n_bytes, raw6_index(f, row, col));
    dst[t] = (uint16_t)grf::bctx_word(m, r);
    if (++col == f.cols) {
      col = 0;
      ++row;
    }
  }
  // the segment must end exactly where the next one begins
  const bool last = block + 1 == segments;
  const uint32_t want_state = last ? grf::kLow : f.main.states[block + 1];
  const uint32_t want_ip = last ? f.main.n_bytes : f.main.offsets[block + 1];
  if (state != want_state || ip != want_ip) bad |= GRF_ERR_CHECKPOINT;
  if (MODE128) {
    const uint32_t rs = last ? grf::kLow : f.residual.states[block + 1];
    const uint32_t ro = last ? f.residual.n_bytes : f.residual.offsets[block + 1];
    if (rstate != rs || rip != ro) bad |= GRF_ERR_CHECKPOINT;
  }
  if (bad) atomicOr(error, (int)bad);
}

// Index of element (row, col) among the packed 5-bit fields: the frame's own order, or, for a
// tensor that keeps them for the fused kernels, records of 32 in blocks of rows, ordered by their
// position in the segment, the segment's number and the row inside the block.
__device__ __forceinline__ uint64_t raw5_index(const grf_ppcx_frame &f, uint32_t row, uint32_t col) {
  if (!f.raw5_segment) return (uint64_t)row * f.cols + col;
  const uint32_t S = f.raw5_segment, spr = f.cols / S, B = f.raw5_block_rows ? f.raw5_block_rows : 1;
  const uint32_t q = f.raw5_row_pos ? f.raw5_row_pos[row] : row, within = q % B;
  const uint64_t record = (uint64_t)(q - within) * (f.cols / 32) + ((uint64_t)((col % S) / 32) * spr + col / S) * B + within;
  return record * 32 + col % 32;
}

// MODE1: residual is a second rANS stream (vocab 32) whose context is the main symbol.
template <bool MODE1>
__global__ __launch_bounds__(kThreads) void ppcx_decode_kernel(grf_ppcx_frame f, const uint16_t *reference,
                                                                uint16_t *out, int32_t *error) {
  const uint64_t n = (uint64_t)f.rows * f.cols;
  const uint64_t segments = (n + f.stride - 1) / f.stride;
  const uint64_t block = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
  if (block >= segments) return;
  uint32_t bad = 0;
  const uint64_t start = block * f.stride;
  uint32_t row = (uint32_t)(start / f.cols), col = (uint32_t)(start % f.cols);
  uint32_t state = f.main.states[block], ip = f.main.offsets[block];
  uint32_t rstate = 0, rip = 0;
  if (MODE1) {
    rstate = f.residual.states[block];
    rip = f.residual.offsets[block];
  }
  uint16_t th[15];
#pragma unroll
  for (int k = 0; k < 15; ++k) th[k] = f.thresholds[k];
  const uint32_t steps = (uint32_t)(start + f.stride <= n ? f.stride : n - start);
  uint16_t *dst = out + block * f.stride;
  uint32_t label = f.labels[row], flip = f.flips[row];
  for (uint32_t t = 0; t < steps; ++t) {
    const uint32_t key = grf::ordinal_key(reference[start + t], flip);
    const uint32_t ctx = label * 16 + grf::threshold_bin(th, key);
    const uint32_t m = grf::rans_step_global(state, ip, f.main.bytes, f.main.n_bytes,
                                             f.main.cum + (size_t)ctx * 2049, f.main.bucket + (size_t)ctx * 256, bad);
    uint32_t r;
    if (MODE1)
      r = grf::rans_step_global(rstate, rip, f.residual.bytes, f.residual.n_bytes,
                                f.residual.cum + (size_t)m * 33, f.residual.bucket + (size_t)m * 256, bad);
    else
      r = grf::packed_field<5>(f.residual.bytes, f.residual.n_bytes, raw5_index(f, row, col));
    dst[t] = (uint16_t)grf::ppcx_word(m, r);
    if (++col == f.cols) {
      col = 0;
      ++row;
      if (row < f.rows) {
        label = f.labels[row];
        flip = f.flips[row];
      }
    }
  }
  const bool last = block + 1 == segments;
  if (state != (last ? grf::kLow : f.main.states[block + 1]) ||
      ip != (last ? f.main.n_bytes : f.main.offsets[block + 1]))
    bad |= GRF_ERR_CHECKPOINT;
  if (MODE1) {
    if (rstate != (last ? grf::kLow : f.residual.states[block + 1]) ||
        rip != (last ? f.residual.n_bytes : f.residual.offsets[block + 1]))
      bad |= GRF_ERR_CHECKPOINT;
  }
  if (bad) atomicOr(error, (int)bad);
}

// fl32(fl32(u*c0) + fl32(g*c1)) + c2, no contraction, truncated to 16 bits.
__global__ __launch_bounds__(kThreads) void mix_predict_kernel(const uint16_t *up, const uint16_t *gate,
                                                                const uint16_t *coeff, uint16_t *out,
                                                                uint32_t rows, uint32_t cols, int32_t *error) {
  const uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= (uint64_t)rows * cols) return;
  const uint32_t row = (uint32_t)(i / cols);
  const uint32_t uw = up[i], gw = gate[i];
  const uint32_t c0 = coeff[row * 3], c1 = coeff[row * 3 + 1], c2 = coeff[row * 3 + 2];
  const float a = __fmul_rn(__uint_as_float(uw << 16), __uint_as_float(c0 << 16));
  const float b = __fmul_rn(__uint_as_float(gw << 16), __uint_as_float(c1 << 16));
  const float y = __fadd_rn(__fadd_rn(a, b), __uint_as_float(c2 << 16));
  const uint32_t word = __float_as_uint(y) >> 16;
  auto nonfinite = [](uint32_t w) { return (w & 0x7F80u) == 0x7F80u; };
  if (nonfinite(uw) || nonfinite(gw) || nonfinite(c0) || nonfinite(c1) || nonfinite(c2) || nonfinite(word))
    atomicOr(error, GRF_ERR_SYMBOL);
  out[i] = (uint16_t)word;
}

bool stream_ok(const grf_stream &s, bool coded) {
  if (!s.bytes) return false;
  if (!coded) return true;
  return s.cum && s.bucket && s.states && s.offsets && s.n_bytes >= 4;
}

int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(GRF_LAUNCH_FAILED, std::string(what) + ": " + hipGetErrorString(e));
  return GRF_OK;
}

}  // namespace

namespace grf {
// One lane writes the two device counters -- the constant-rate one and the shader clock's --
// and where it ran: shader-clock counters of different parts of the chip do not share a zero,
// so only two readings taken at one place may be subtracted.
__global__ void timestamp_kernel(uint64_t *slot) {
  if (threadIdx.x == 0) {
    slot[0] = wall_clock64();
    slot[1] = clock64();
    slot[2] = __smid();
  }
}
}  // namespace grf

extern "C" {

const char *grf_last_error(void) { return grf::g_error.c_str(); }
int grf_abi_version(void) { return 3; }

int grf_wall_clock_khz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

int grf_timestamp(uint64_t *slot, void *hip_stream) {
  if (!slot) return fail(GRF_BAD_ARGUMENT, "grf_timestamp: null argument");
  hipLaunchKernelGGL(grf::timestamp_kernel, dim3(1), dim3(64), 0, (hipStream_t)hip_stream, slot);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(GRF_LAUNCH_FAILED, std::string("grf_timestamp: ") + hipGetErrorString(e));
  return GRF_OK;
}

int grf_bctx_decode(const grf_bctx_frame *frame, const int64_t *block_ids, uint32_t count, uint16_t *out,
                    int32_t *error, void *hip_stream) {
  if (!frame || !out || !error) return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: null argument");
  const grf_bctx_frame &f = *frame;
  if (!f.rows || !f.cols || !f.stride || f.stride > 65536 || !f.nc || f.nc > 16 || !f.row_class || !f.col_class)
    return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: bad geometry");
  if (f.mode != 0 && f.mode != 128) return fail(GRF_UNSUPPORTED, "grf_bctx_decode: mode must be 0 or 128");
  if (!stream_ok(f.main, true) || !stream_ok(f.residual, f.mode == 128))
    return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: incomplete stream descriptor");
  const uint64_t n = (uint64_t)f.rows * f.cols;
  // (in the fused kernels' order the array may hold rows beyond the matrix's: positions no row has)
  if (f.mode == 0 && (f.raw6_segment ? f.residual.n_bytes < (n * 6 + 7) / 8 : f.residual.n_bytes != (n * 6 + 7) / 8))
    return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: packed residual length mismatch");
  if (f.mode == 0 && f.raw6_segment &&
      (f.raw6_segment % 16 || f.cols % f.raw6_segment || f.raw6_block_rows > 16 ||
       (f.raw6_block_rows & (f.raw6_block_rows - 1))))
    return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: residual order (segment length, block rows)");
  const uint64_t segments = (n + f.stride - 1) / f.stride;
  if (!count) return GRF_OK;
  if (!block_ids && count > segments) return fail(GRF_BAD_ARGUMENT, "grf_bctx_decode: count exceeds segments");
  const dim3 grid((count + kThreads - 1) / kThreads), block(kThreads);
  hipStream_t s = (hipStream_t)hip_stream;
  if (f.mode == 128)
    hipLaunchKernelGGL(bctx_decode_kernel<true>, grid, block, 0, s, f, block_ids, count, out, error);
  else
    hipLaunchKernelGGL(bctx_decode_kernel<false>, grid, block, 0, s, f, block_ids, count, out, error);
  return launch_status("grf_bctx_decode");
}

int grf_ppcx_decode(const grf_ppcx_frame *frame, const uint16_t *reference, uint16_t *out, int32_t *error,
                    void *hip_stream) {
  if (!frame || !reference || !out || !error) return fail(GRF_BAD_ARGUMENT, "grf_ppcx_decode: null argument");
  const grf_ppcx_frame &f = *frame;
  if (!f.rows || !f.cols || !f.stride || f.stride > 65536 || !f.labels || !f.flips || !f.thresholds)
    return fail(GRF_BAD_ARGUMENT, "grf_ppcx_decode: bad geometry");
  if (f.mode > 1) return fail(GRF_UNSUPPORTED, "grf_ppcx_decode: mode must be 0 or 1");
  if (!stream_ok(f.main, true) || !stream_ok(f.residual, f.mode == 1))
    return fail(GRF_BAD_ARGUMENT, "grf_ppcx_decode: incomplete stream descriptor");
  const uint64_t n = (uint64_t)f.rows * f.cols;
  if (f.mode == 0 && (f.raw5_segment ? f.residual.n_bytes < (n * 5 + 7) / 8 : f.residual.n_bytes != (n * 5 + 7) / 8))
    return fail(GRF_BAD_ARGUMENT, "grf_ppcx_decode: packed residual length mismatch");
  if (f.mode == 0 && f.raw5_segment &&
      (f.raw5_segment % 32 || f.cols % f.raw5_segment || f.raw5_block_rows > 16 ||
       (f.raw5_block_rows & (f.raw5_block_rows - 1))))
    return fail(GRF_BAD_ARGUMENT, "grf_ppcx_decode: residual order (segment length, block rows)");
  const uint64_t segments = (n + f.stride - 1) / f.stride;
  const dim3 grid((unsigned)((segments + kThreads - 1) / kThreads)), block(kThreads);
  hipStream_t s = (hipStream_t)hip_stream;
  if (f.mode == 1)
    hipLaunchKernelGGL(ppcx_decode_kernel<true>, grid, block, 0, s, f, reference, out, error);
  else
    hipLaunchKernelGGL(ppcx_decode_kernel<false>, grid, block, 0, s, f, reference, out, error);
  return launch_status("grf_ppcx_decode");
}

int grf_mix_predict(const uint16_t *up, const uint16_t *gate, const uint16_t *coeff, uint16_t *out,
                    uint32_t rows, uint32_t cols, int32_t *error, void *hip_stream) {
  if (!up || !gate || !coeff || !out || !error || !rows || !cols)
    return fail(GRF_BAD_ARGUMENT, "grf_mix_predict: null or empty argument");
  const uint64_t n = (uint64_t)rows * cols;
  const dim3 grid((unsigned)((n + kThreads - 1) / kThreads)), block(kThreads);
  hipLaunchKernelGGL(mix_predict_kernel, grid, block, 0, (hipStream_t)hip_stream, up, gate, coeff, out, rows, cols,
                     error);
  return launch_status("grf_mix_predict");
}

}  // extern "C"
