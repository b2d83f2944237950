// Entry points of the LDS-streamed Q4_K decode GEMV (kernel and design notes: ttq_gemv_q4k_stream.h).
#include "ttq_gemv_q4k_stream.h"

namespace ttq {

// ------------------------------------------------------------------------------ launch
bool gemv_q4k_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  if (format != kQ4_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  if (n_in != 4096 && n_in != 2048) return false;
  const int64_t blocks = (((int64_t)st_rows_per_wg(n_out, nullptr) + 15) / 16) * (n_in / 2048);
  // byte offsets into the weight buffer are 32-bit in the kernel; with fewer than 16 rows per
  // compute unit the register-streamed kernel, which splits a row group over its wavefronts, is faster
  return n_out >= 16 * device_num_cus() && blocks <= kStMaxBlocks && n_out * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

// The gate || up form: n_ff outputs from 2 n_ff weight rows.  At least 8 outputs per compute unit (16 weight rows),
// and the two parts' row groups together within the block table.
bool gemv_q4k_stream_fused_supported(int x_dtype, int64_t n_ff, int64_t n_in) {
  if (!(x_dtype == kBF16 || x_dtype == kF16)) return false;
  if (n_in != 4096 && n_in != 2048) return false;
  const int64_t blocks = 2 * (((int64_t)st_rows_per_wg(n_ff, nullptr) + 15) / 16) * (n_in / 2048);
  return n_ff >= 8 * device_num_cus() && blocks <= kStMaxBlocks && 2 * n_ff * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

template <typename XT>
static hipError_t st_launch_fused_x(const void* w, const void* x, void* y, int y_dtype, int64_t m, int64_t n_ff,
                                    int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return st_launch_xy<XT, float, 0, true>(w, x, y, nullptr, 0, m, n_ff, n_in, s);
    case kF16: return st_launch_xy<XT, f16_tag, 0, true>(w, x, y, nullptr, 0, m, n_ff, n_in, s);
    case kBF16: return st_launch_xy<XT, bf16_tag, 0, true>(w, x, y, nullptr, 0, m, n_ff, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemv_q4k_stream_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                        int64_t n_ff, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return st_launch_fused_x<bf16_tag>(w, x, y, y_dtype, m, n_ff, n_in, s);
  if (x_dtype == kF16) return st_launch_fused_x<f16_tag>(w, x, y, y_dtype, m, n_ff, n_in, s);
  return hipErrorInvalidValue;
}

// add + RMSNorm in front (and optionally silu_and_mul behind) on the same kernel
template <typename XT, bool FUSE>
static hipError_t st_launch_norm_x(const void* w, const void* x, void* y, int y_dtype, int64_t m, int64_t n_out,
                                   int64_t n_in, const GemvNormArgs& na, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return st_launch_xy<XT, float, 0, FUSE, true>(w, x, y, nullptr, 0, m, n_out, n_in, s, na);
    case kF16: return st_launch_xy<XT, f16_tag, 0, FUSE, true>(w, x, y, nullptr, 0, m, n_out, n_in, s, na);
    case kBF16: return st_launch_xy<XT, bf16_tag, 0, FUSE, true>(w, x, y, nullptr, 0, m, n_out, n_in, s, na);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemv_q4k_stream_norm(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                       int64_t n_out, int64_t n_in, bool silu_mul, const void* norm_residual,
                                       const void* norm_gamma, float norm_eps, void* new_residual_out,
                                       void* normed_out, hipStream_t s) {
  GemvNormArgs na{};
  na.residual = static_cast<const uint16_t*>(norm_residual);
  na.gamma = static_cast<const uint16_t*>(norm_gamma);
  na.new_residual = static_cast<uint16_t*>(new_residual_out);
  na.normed = static_cast<uint16_t*>(normed_out);
  na.eps = norm_eps;
  if (x_dtype == kBF16)
    return silu_mul ? st_launch_norm_x<bf16_tag, true>(w, x, y, y_dtype, m, n_out, n_in, na, s)
                    : st_launch_norm_x<bf16_tag, false>(w, x, y, y_dtype, m, n_out, n_in, na, s);
  if (x_dtype == kF16)
    return silu_mul ? st_launch_norm_x<f16_tag, true>(w, x, y, y_dtype, m, n_out, n_in, na, s)
                    : st_launch_norm_x<f16_tag, false>(w, x, y, y_dtype, m, n_out, n_in, na, s);
  return hipErrorInvalidValue;
}

template <typename XT>
static hipError_t st_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                              int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return st_launch_xy<XT, float, 0>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return st_launch_xy<XT, f16_tag, 0>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return st_launch_xy<XT, bf16_tag, 0>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemv_q4k_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return st_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return st_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
