// Prefill GEMM over a packed copy of the activations (kernel: ttq_gemm_pcd.h): the instantiations behind
// launch_gemm_pc's choice of tile, and the packing pass.
#include "ttq_gemm_pcd.h"

namespace ttq {

namespace {

template <int FMT, bool FUSE, class XT>
hipError_t packed_fmt(int tile, const uint8_t* wb, const uint16_t* xp, void* y, int y_dtype, const void* bias,
                      int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp, hipStream_t s,
                      const float* row_scale) {
  switch (tile) {
    case 0: return launch_pcd_grid<FMT, 4, 7, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case 1: return launch_pcd_grid<FMT, 4, 4, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case 2: return launch_pcd_grid<FMT, 2, 7, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case 3: return launch_pcd_grid<FMT, 2, 4, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case 4: return launch_pcd_grid<FMT, 1, 7, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case 5: return launch_pcd_grid<FMT, 1, 4, FUSE, 0, 4, XT>(wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_gemm_packed(int format, bool fuse, int tile, const uint8_t* wb, const uint16_t* xp, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp,
                              hipStream_t s, bool x_f16, const float* row_scale) {
  // (no fused gate||up form here: its epilogue does not fit beside three steps of A fragments, and registers that
  // are the target of asynchronous requests must not be spilled)
  if (fuse) return hipErrorInvalidValue;
  if (x_f16) {
    switch (format) {
      case kQ4_K: return packed_fmt<kQ4_K, false, f16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
      case kQ6_K: return packed_fmt<kQ6_K, false, f16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
      case kQ8_0: return packed_fmt<kQ8_0, false, f16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
      default: return hipErrorInvalidValue;
    }
  }
  switch (format) {
    case kQ4_K: return packed_fmt<kQ4_K, false, bf16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case kQ6_K: return packed_fmt<kQ6_K, false, bf16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    case kQ8_0: return packed_fmt<kQ8_0, false, bf16_tag>(tile, wb, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, row_scale);
    default: return hipErrorInvalidValue;
  }
}

size_t gemm_packed_activation_bytes(int64_t m, int64_t n_in) { return packed_activation_bytes(m, n_in); }

hipError_t launch_gemm_pack_activations(const void* x, int x_dtype, uint16_t* xp, int64_t m, int64_t n_in, hipStream_t s,
                                        bool keep_f16) {
  return launch_pack_activations(x, x_dtype, xp, m, n_in, s, keep_f16);
}

hipError_t launch_gemm_pack_activations_scaled(const float* x, uint16_t* xp, float* row_scale, int64_t m, int64_t n_in,
                                               hipStream_t s) {
  return launch_pack_activations_scaled(x, xp, row_scale, m, n_in, s);
}

}  // namespace ttq
