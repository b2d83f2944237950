// Measurement ladder for the Q4_K prefill GEMM: what each role of the producer/consumer kernels costs on its own
// and what the roles cost together, on the 256 x 112 tile of the headline shape.
//
// Not part of libttq_hip.so.  bench.py --only ladder_gemm builds libttq_ladder.so on demand and times the rungs;
// a rocprofv3 kernel trace of that command names every rung by its kernel and its ABL template argument.
//
// kernel 0: gemm_pcd_kernel (ttq_gemm_pcd.h; activations from their packed copy straight into the consumers' registers)
//   ABL 31    barriers, prologue and epilogue only
//   ABL 4124  consumers alone: A requests, B reads, MFMA (real values put in the W tile once, at the start)
//   ABL 4104  ... and the W producers' global loads and LDS stores, without the dequantization arithmetic
//   ABL 0     the whole kernel
//   ABL 3     W producers alone (loads, dequantization, LDS stores)
//   ABL 2     consumers without their A requests (zero activations) and W producers
//   ABL 1024  the whole kernel without its barriers: every role at its own pace (results are garbage)
// kernel 1: gemm_pc_kernel (ttq_gemm_pc.h; activations staged through LDS by four mover wavefronts)
//   ABL 31    barriers, prologue and epilogue only
//   ABL 4126  consumers alone (real values put in LDS once, at the start)
//   ABL 4124  consumers and X movers
//   ABL 0     the whole kernel
//   ABL 29    X movers alone
//   ABL 1024  the whole kernel without its barriers
//   ABL 2048  the whole kernel with X moved by global_load_lds into rings of four stages (+ an L2 prefetch)
// kernel 2: gemm_pcr_kernel (ttq_gemm_pcr.h; kernel 0 as a persistent workgroup per compute unit, a ring of W stages
//   with counters in LDS in place of the step barrier)
//   ABL 0     the whole kernel
// ttq_ladder_gemm_pack is the packing pass of kernels 0 and 2 on its own.
#include "ttq_gemm_pcr.h"

namespace {

template <int KERNEL, int ABL>
hipError_t rung(const uint8_t* wb, const uint16_t* x, void* y, int64_t m, int64_t n_out, int64_t n_in, ttq::PcSplit sp,
                hipStream_t s) {
  using namespace ttq;
  if (KERNEL == 2) {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    return launch_pcr_grid<kQ4_K, 4, 7, false>(wb, x, y, kBF16, nullptr, 0, m, n_out, n_in, cus, s);
  }
  if (KERNEL == 0) return launch_pcd_grid<kQ4_K, 4, 7, false, ABL>(wb, x, y, kBF16, nullptr, 0, m, n_out, n_in, sp, s);
  return launch_pc_grid<kQ4_K, 4, 7, false, ABL>(wb, x, y, kBF16, nullptr, 0, m, n_out, n_in, sp, s);
}

bool args_ok(const void* w, const void* x, const void* y, int64_t m, int64_t n_out, int64_t n_in) {
  return w && x && y && m > 0 && n_out > 0 && n_in > 0 && n_in % 1024 == 0 && m * n_in * 2 < ((int64_t)1 << 32);
}

}  // namespace

#define TTQ_RUNGS(EXTRA)                                                                                      \
  switch (kernel * 100000 + abl) {                                                                            \
    TTQ_RUNG(0, 31 + EXTRA) TTQ_RUNG(0, 4124 + EXTRA) TTQ_RUNG(0, 4104 + EXTRA) TTQ_RUNG(0, 0 + EXTRA)        \
    TTQ_RUNG(0, 3 + EXTRA) TTQ_RUNG(0, 2 + EXTRA) TTQ_RUNG(0, 1024 + EXTRA)                                   \
    TTQ_RUNG(1, 31 + EXTRA) TTQ_RUNG(1, 4126 + EXTRA) TTQ_RUNG(1, 4124 + EXTRA) TTQ_RUNG(1, 0 + EXTRA)        \
    TTQ_RUNG(1, 29 + EXTRA) TTQ_RUNG(1, 1024 + EXTRA) TTQ_RUNG(1, 2048 + EXTRA)                               \
    default: return -1;                                                                                       \
  }

extern "C" __attribute__((visibility("default")))
int ttq_ladder_gemm_pack(const void* x_bf16, void* xp, int64_t m, int64_t n_in, void* stream) {
  if (!x_bf16 || !xp || m <= 0 || n_in <= 0 || n_in % 256 != 0) return -1;
  return ttq::launch_pack_activations(x_bf16, ttq::kBF16, static_cast<uint16_t*>(xp), m, n_in,
                                      static_cast<hipStream_t>(stream)) == hipSuccess ? 0 : -7;
}

// x_bf16: the activations for kernel 1, their packed copy (ttq_ladder_gemm_pack) for kernels 0 and 2
extern "C" __attribute__((visibility("default")))
int ttq_ladder_gemm_launch(int kernel, int abl, const void* w, const void* x_bf16, void* y_bf16, int64_t m, int64_t n_out,
                           int64_t n_in, void* stream) {
  if (!args_ok(w, x_bf16, y_bf16, m, n_out, n_in)) return -1;
  const ttq::PcSplit sp{1, 0, nullptr, nullptr};
  hipError_t e = hipErrorInvalidValue;
#define TTQ_RUNG(K, A)                                                                                                 \
  case K * 100000 + (A):                                                                                               \
    e = rung<K, (A)>(static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x_bf16), y_bf16, m, n_out, n_in, sp, \
                     static_cast<hipStream_t>(stream));                                                                \
    break;
  if (kernel == 2 && abl == 0) {
    e = rung<2, 0>(static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x_bf16), y_bf16, m, n_out, n_in, sp,
                   static_cast<hipStream_t>(stream));
    return e == hipSuccess ? 0 : -7;
  }
  TTQ_RUNGS(0)
#undef TTQ_RUNG
  return e == hipSuccess ? 0 : -7;
}

// The same rungs with the wavefronts' clocks read around every step barrier (ABL + 512): trace receives, for
// workgroup b and wavefront v (0-3 consumers, 4-7 W producers, 8-11 X movers of kernel 1), at [(b * 12 + v) * 4 ...]:
// shader cycles from kernel entry to the end of the K loop, cycles spent at the barriers, cycles the DMA movers
// waited for their requests, and the first span again in ticks of the 100 MHz clock.  trace holds 4 * 12 words per
// workgroup of the launch.
extern "C" __attribute__((visibility("default")))
int ttq_ladder_gemm_trace(int kernel, int abl, const void* w, const void* x_bf16, void* y_bf16, int64_t m, int64_t n_out,
                          int64_t n_in, uint32_t* trace, void* stream) {
  if (!args_ok(w, x_bf16, y_bf16, m, n_out, n_in) || !trace) return -1;
  const ttq::PcSplit sp{1, 0, nullptr, trace};
  hipError_t e = hipErrorInvalidValue;
  abl += 512;
#define TTQ_RUNG(K, A)                                                                                                 \
  case K * 100000 + (A):                                                                                               \
    e = rung<K, (A)>(static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x_bf16), y_bf16, m, n_out, n_in, sp, \
                     static_cast<hipStream_t>(stream));                                                                \
    break;
  TTQ_RUNGS(512)
#undef TTQ_RUNG
  return e == hipSuccess ? 0 : -7;
}
