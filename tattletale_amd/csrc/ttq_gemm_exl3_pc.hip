// Trellis-coded linear layer for many rows as a producer/consumer GEMM (kernel: ttq_gemm_exl3_pc.h): the
// instantiations per (bits, codebook, rows per tile).
#include "ttq_gemm_exl3_pc.h"

namespace ttq {

namespace {

template <int BITS, int CB>
hipError_t xg_mb(int mb, const uint8_t* trellis, const uint16_t* svh, const uint16_t* xp, void* y, int y_dtype,
                 const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp, hipStream_t s) {
  if (mb == 1) return launch_exl3_pc_grid<BITS, CB, 1>(trellis, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
  if (mb == 4) return launch_exl3_pc_grid<BITS, CB, 4>(trellis, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
  return launch_exl3_pc_grid<BITS, CB, 2>(trellis, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
}

template <int BITS>
hipError_t xg_cb(int cb, int mb, const uint8_t* trellis, const uint16_t* svh, const uint16_t* xp, void* y, int y_dtype,
                 const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp, hipStream_t s) {
  return cb == 0 ? xg_mb<BITS, 0>(mb, trellis, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s)
                 : xg_mb<BITS, 1>(mb, trellis, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
}

}  // namespace

// xp: the rotated activations (fp16) in fragment order; mb: 16-row blocks per consumer (1, 2 or 4: tiles of 64, 128 or 256 rows)
hipError_t launch_gemm_exl3_pc(int bits, int cb, int mb, const uint16_t* trellis, const uint16_t* svh, const uint16_t* xp,
                               void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                               int64_t n_in, PcSplit sp, hipStream_t s) {
  const uint8_t* t = reinterpret_cast<const uint8_t*>(trellis);
  switch (bits) {
    case 1: return xg_cb<1>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 2: return xg_cb<2>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 3: return xg_cb<3>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 4: return xg_cb<4>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 5: return xg_cb<5>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 6: return xg_cb<6>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 7: return xg_cb<7>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    case 8: return xg_cb<8>(cb, mb, t, svh, xp, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ttq
