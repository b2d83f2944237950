// Entry points of the LDS-streamed Q6_K decode GEMV (kernel and design notes: ttq_gemv_q6k_stream.h).
#include "ttq_gemv_q6k_stream.h"

namespace ttq {

namespace {

template <typename XT>
hipError_t q6_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                       int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q6_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return q6_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return q6_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool gemv_q6k_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  if (format != kQ6_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  return q6_plan(n_out, n_in).ok;
}

hipError_t launch_gemv_q6k_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return q6_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return q6_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
