// C-ABI layer of libttq_hip.so: argument validation, GEMV/GEMM dispatch, error codes.
// Declarations and the reference interfaces they replace are in include/ttq.h.
//
// The dispatch in ttq_linear_forward mirrors the reference's Linear.forward
// (workspace/transformers/src/layers/linear.nim:45-57): one operator, bias optional, the
// number of activation rows decides between the decode (GEMV) and prefill (GEMM) kernels.
#include "../../include/ttq.h"
#include "ttq_internal.h"

#include <stdlib.h>

namespace ttq {

int device_num_cus() {
  static std::atomic<int> cached[64];     // by device ordinal; 0 = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  std::atomic<int>& slot = cached[dev & 63];
  int cus = slot.load(std::memory_order_relaxed);
  if (cus == 0) {
    hipDeviceProp_t prop;
    cus = (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
              ? prop.multiProcessorCount : 256;
    slot.store(cus, std::memory_order_relaxed);
  }
  return cus;
}

thread_local RouteProbe* t_route_probe = nullptr;

hipError_t allow_large_lds(const void* kernel, LargeLds& state) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (state.done.load(std::memory_order_relaxed) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e != hipSuccess) return e;
  state.done.fetch_or(bit, std::memory_order_relaxed);
  return hipSuccess;
}

}  // namespace ttq

namespace {

thread_local int g_last_hip_error = 0;

int hip_status(hipError_t e) {
  if (e == hipSuccess) return TTQ_OK;
  g_last_hip_error = (int)e;
  return TTQ_ERR_HIP;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
int64_t dtype_size(int d) { return d == TTQ_F32 ? 4 : 2; }
// do [a, a + an) and [b, b + bn) share a byte?  (null pointers never overlap anything)
bool overlaps(const void* a, int64_t an, const void* b, int64_t bn) {
  if (!a || !b || an <= 0 || bn <= 0) return false;
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return pa < pb + (uintptr_t)bn && pb < pa + (uintptr_t)an;
}
bool valid_dtype(int d) { return d == TTQ_F32 || d == TTQ_F16 || d == TTQ_BF16; }

// Shape rules of each format along n_in / n_out.
int check_shape(int format, int64_t m, int64_t n_out, int64_t n_in, int bits, int cb) {
  if (m < 0 || n_out < 0 || n_in <= 0) return TTQ_ERR_SHAPE;
  if (n_out > 0x7FFFFFFF || n_in > 0x7FFFFFFF || m > 0x7FFFFFFF) return TTQ_ERR_UNSUPPORTED;
  switch (format) {
    case TTQ_Q8_0: return (n_in % 32 == 0) ? TTQ_OK : TTQ_ERR_SHAPE;
    case TTQ_Q4_K:
    case TTQ_Q6_K: return (n_in % 256 == 0) ? TTQ_OK : TTQ_ERR_SHAPE;
    case TTQ_EXL3:
      if (bits < 1 || bits > 8) return TTQ_ERR_FORMAT;
      if (cb != TTQ_CB_3INST && cb != TTQ_CB_MCG) return TTQ_ERR_FORMAT;
      return (n_in % 128 == 0 && n_out % 128 == 0) ? TTQ_OK : TTQ_ERR_SHAPE;
    default: return TTQ_ERR_FORMAT;
  }
}


// grid dimensions y and z end at 65535: the trellis GEMV puts groups of 8 activation rows on z, the fused decode
// kernels and RMSNorm one row per workgroup on y
constexpr int64_t kMaxExl3GemvRows = 8 * 65535, kMaxGridRows = 65535;

// launch_gemv puts the activation rows (or passes over them) on gridDim.y, which ends at 65535
hipError_t launch_gemv_any_m(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                             const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                             hipStream_t s) {
  constexpr int64_t kChunk = 65520;   // a multiple of the 4, 8 and 16 rows the few-row kernels take per pass
  const char* xb = static_cast<const char*>(x);
  char* yb = static_cast<char*>(y);
  for (int64_t r = 0; r < m; r += kChunk) {
    const int64_t rows = m - r < kChunk ? m - r : kChunk;
    const hipError_t e = ttq::launch_gemv(format, w, xb + r * n_in * dtype_size(x_dtype), x_dtype,
                                          yb + r * n_out * dtype_size(y_dtype), y_dtype, bias, bias_dtype, rows,
                                          n_out, n_in, s);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

int gemv_block(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
               const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
               void* stream) {
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype)) return TTQ_ERR_DTYPE;
  if (bias && !valid_dtype(bias_dtype)) return TTQ_ERR_DTYPE;
  int rc = check_shape(format, m, n_out, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;  // empty output: nothing to read or write
  if (!w || !x || !y) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(x) || !aligned16(y)) return TTQ_ERR_ALIGN;
  return hip_status(launch_gemv_any_m(format, w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in,
                                      static_cast<hipStream_t>(stream)));
}

int dequant_block(int format, const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in,
                  void* stream) {
  if (!valid_dtype(out_dtype)) return TTQ_ERR_DTYPE;
  const int rc = check_shape(format, 1, n_out, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (n_out == 0) return TTQ_OK;  // empty matrix
  if (!w || !out) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(out)) return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_dequant(format, w, out, out_dtype, n_out, n_in,
                                        static_cast<hipStream_t>(stream)));
}

}  // namespace

extern "C" {

int ttq_version(void) { return TTQ_VERSION; }

const char* ttq_strerror(int status) {
  switch (status) {
    case TTQ_OK: return "ok";
    case TTQ_ERR_NULL: return "required pointer is NULL";
    case TTQ_ERR_SHAPE: return "bad shape: dimension negative or not a multiple of the block size";
    case TTQ_ERR_ALIGN: return "base pointer is not 16-byte aligned";
    case TTQ_ERR_DTYPE: return "unknown or unsupported dtype";
    case TTQ_ERR_FORMAT: return "unknown format, bit width or codebook";
    case TTQ_ERR_UNSUPPORTED: return "request outside the supported size limits";
    case TTQ_ERR_HIP: return "HIP runtime error (see ttq_last_hip_error)";
    case TTQ_ERR_ALIAS: return "output buffer overlaps an input where that is not allowed";
    case TTQ_ERR_WORKSPACE: return "caller-owned workspace is NULL, misaligned or smaller than ttq_workspace_bytes says";
    default: return "unknown status";
  }
}

int ttq_last_hip_error(void) { return g_last_hip_error; }

int64_t ttq_packed_nbytes(int format, int64_t n_out, int64_t n_in, int bits) {
  const int rc = check_shape(format, 1, n_out, n_in, bits, TTQ_CB_MCG);
  if (rc != TTQ_OK) return rc;
  switch (format) {
    case TTQ_Q8_0: return n_out * (n_in / 32) * 34;
    case TTQ_Q4_K: return n_out * (n_in / 256) * 144;
    case TTQ_Q6_K: return n_out * (n_in / 256) * 210;
    case TTQ_EXL3: return (n_out / 16) * (n_in / 16) * 32 * bits;
    default: return TTQ_ERR_FORMAT;
  }
}

int ttq_gemv_q8_0(const void* w, const void* x, int x_dtype, float* y, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemv_block(TTQ_Q8_0, w, x, x_dtype, y, TTQ_F32, nullptr, 0, m, n_out, n_in, stream);
}
int ttq_gemv_q4_k(const void* w, const void* x, int x_dtype, float* y, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemv_block(TTQ_Q4_K, w, x, x_dtype, y, TTQ_F32, nullptr, 0, m, n_out, n_in, stream);
}
int ttq_gemv_q6_k(const void* w, const void* x, int x_dtype, float* y, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemv_block(TTQ_Q6_K, w, x, x_dtype, y, TTQ_F32, nullptr, 0, m, n_out, n_in, stream);
}

int ttq_gemv_exl3(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                  const uint16_t* x_f16, float* y, int64_t m, int64_t n_out, int64_t n_in, int bits,
                  int codebook, void* stream) {
  const int rc = check_shape(TTQ_EXL3, m, n_out, n_in, bits, codebook);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;
  if (!trellis || !suh_f16 || !svh_f16 || !x_f16 || !y) return TTQ_ERR_NULL;
  if (!aligned16(trellis) || !aligned16(x_f16) || !aligned16(y) || !aligned8(suh_f16) || !aligned8(svh_f16))
    return TTQ_ERR_ALIGN;
  if (m > kMaxExl3GemvRows) return TTQ_ERR_UNSUPPORTED;
  return hip_status(ttq::launch_gemv_exl3(trellis, suh_f16, svh_f16, x_f16, TTQ_F16, y, TTQ_F32,
                                          nullptr, 0, m, n_out, n_in, bits, codebook,
                                          static_cast<hipStream_t>(stream)));
}

int ttq_gemv_exl3_noalloc(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                          const uint16_t* x_f16, float* y, int64_t m, int64_t n_out, int64_t n_in, int bits,
                          int codebook, void* stream) {
  const int rc = check_shape(TTQ_EXL3, m, n_out, n_in, bits, codebook);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;
  if (!trellis || !suh_f16 || !svh_f16 || !x_f16 || !y) return TTQ_ERR_NULL;
  if (!aligned16(trellis) || !aligned16(x_f16) || !aligned16(y) || !aligned8(suh_f16) || !aligned8(svh_f16))
    return TTQ_ERR_ALIGN;
  if (m > 8) return TTQ_ERR_UNSUPPORTED;        // one group of activation rows: the decode case
  const ttq::Exl3Plan plan = ttq::exl3_mfma_plan(m, n_out, n_in);
  if (plan.accum_words > ttq::exl3_resident_words()) return TTQ_ERR_UNSUPPORTED;
  unsigned long long* accum = nullptr;
  if (plan.slices > 1) {
    const hipError_t e = ttq::exl3_resident_workspace(&accum);
    if (e != hipSuccess) return hip_status(e);
  }
  return hip_status(ttq::launch_gemv_exl3_mfma(plan, trellis, suh_f16, svh_f16, x_f16, TTQ_F16, y, TTQ_F32, nullptr, 0, m,
                                               n_out, n_in, bits, codebook, accum,
                                               static_cast<hipStream_t>(stream)));
}

int ttq_gemm_exl3(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16, const void* x,
                  int x_dtype, float* y, int64_t m, int64_t n_out, int64_t n_in, int bits, int codebook,
                  void* stream) {
  if (!valid_dtype(x_dtype)) return TTQ_ERR_DTYPE;
  const int rc = check_shape(TTQ_EXL3, m, n_out, n_in, bits, codebook);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;
  if (!trellis || !suh_f16 || !svh_f16 || !x || !y) return TTQ_ERR_NULL;
  if (!aligned16(trellis) || !aligned16(x) || !aligned16(y) || !aligned8(suh_f16) || !aligned8(svh_f16))
    return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_gemm_exl3(trellis, suh_f16, svh_f16, x, x_dtype, y, TTQ_F32, nullptr, 0, m, n_out, n_in, bits,
                                          codebook, static_cast<hipStream_t>(stream)));
}

int ttq_silu_and_mul(const void* in, void* out, int dtype, int64_t m, int64_t h, void* stream) {
  if (!valid_dtype(dtype)) return TTQ_ERR_DTYPE;
  if (m < 0 || h < 0) return TTQ_ERR_SHAPE;
  if (m == 0 || h == 0) return TTQ_OK;
  if (!in || !out) return TTQ_ERR_NULL;
  if (!aligned16(in) || !aligned16(out)) return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_silu_and_mul(in, out, dtype, m, h, static_cast<hipStream_t>(stream)));
}

int ttq_gemv_q4_k_silu_mul(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                           int64_t n_ff, int64_t n_in, void* stream) {
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype)) return TTQ_ERR_DTYPE;
  if (n_ff < 0 || n_ff > (INT64_MAX >> 2)) return TTQ_ERR_SHAPE;
  const int rc = check_shape(TTQ_Q4_K, m, 2 * n_ff, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_ff == 0) return TTQ_OK;
  if (!w || !x || !y) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(x) || !aligned16(y)) return TTQ_ERR_ALIGN;
  // two to four rows: one pass over the weights for all of them; more rows: four at a time
  if (m >= 2 && ttq::gemv_q4k_stream4_fused_supported(x_dtype, m < 4 ? m : 4, n_ff, n_in) &&
      ttq::gemv_q4k_stream_fused_supported(x_dtype, n_ff, n_in)) {
    const char* xb = static_cast<const char*>(x);
    char* yb = static_cast<char*>(y);
    for (int64_t r0 = 0; r0 < m; r0 += 4) {
      const int64_t rows = m - r0 < 4 ? m - r0 : 4;
      const void* xr = xb + r0 * n_in * dtype_size(x_dtype);
      void* yr = yb + r0 * n_ff * dtype_size(y_dtype);
      const hipError_t e = rows >= 2 ? ttq::launch_gemv_q4k_stream4_fused(w, xr, x_dtype, yr, y_dtype, rows, n_ff, n_in,
                                                                          static_cast<hipStream_t>(stream))
                                     : ttq::launch_gemv_q4k_stream_fused(w, xr, x_dtype, yr, y_dtype, rows, n_ff, n_in,
                                                                         static_cast<hipStream_t>(stream));
      if (e != hipSuccess) return hip_status(e);
    }
    return TTQ_OK;
  }
  if (m <= 4 && ttq::gemv_q4k_stream_fused_supported(x_dtype, n_ff, n_in))
    return hip_status(ttq::launch_gemv_q4k_stream_fused(w, x, x_dtype, y, y_dtype, m, n_ff, n_in,
                                                        static_cast<hipStream_t>(stream)));
  if (!ttq::gemv_fused_supported(TTQ_Q4_K, x_dtype, n_ff, n_in, true) || m > kMaxGridRows) return TTQ_ERR_UNSUPPORTED;
  return hip_status(ttq::launch_gemv_fused(w, x, x_dtype, y, y_dtype, nullptr, 0, m, n_ff, n_in, true, nullptr,
                                           nullptr, 0.f, nullptr, nullptr, static_cast<hipStream_t>(stream)));
}

int ttq_rmsnorm(const void* x, const void* residual, const void* gamma, float eps, int dtype,
                void* new_residual_out, void* normed_out, int64_t m, int64_t n, void* stream) {
  if (!valid_dtype(dtype)) return TTQ_ERR_DTYPE;
  if (m < 0 || n < 0 || !(eps >= 0.f)) return TTQ_ERR_SHAPE;
  if (m == 0 || n == 0) return TTQ_OK;
  if (m > kMaxGridRows) return TTQ_ERR_UNSUPPORTED;
  if (!x || !gamma || !normed_out) return TTQ_ERR_NULL;
  if (!aligned16(x) || !aligned16(gamma) || !aligned16(normed_out) || (residual && !aligned16(residual)) ||
      (new_residual_out && !aligned16(new_residual_out)))
    return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_rmsnorm(x, residual, gamma, eps, dtype, new_residual_out, normed_out, m, n,
                                        static_cast<hipStream_t>(stream)));
}

int ttq_gemv_q4_k_rmsnorm(const void* w, const void* x, const void* residual, const void* gamma, float eps,
                          int x_dtype, void* new_residual_out, void* normed_out, void* y, int y_dtype,
                          int64_t m, int64_t n_out, int64_t n_in, int silu_mul, void* stream) {
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype)) return TTQ_ERR_DTYPE;
  if (n_out < 0 || n_out > (INT64_MAX >> 2) || !(eps >= 0.f)) return TTQ_ERR_SHAPE;
  const int rc = check_shape(TTQ_Q4_K, m, silu_mul ? 2 * n_out : n_out, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;
  if (!w || !x || !gamma || !y) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(x) || !aligned16(gamma) || !aligned16(y) || (residual && !aligned16(residual)) ||
      (new_residual_out && !aligned16(new_residual_out)) || (normed_out && !aligned16(normed_out)))
    return TTQ_ERR_ALIGN;
  // every workgroup re-reads x and residual while workgroup 0 writes the two outputs: in-place use
  // (allowed for ttq_rmsnorm) would race here
  {
    const int64_t nb = m * n_in * dtype_size(x_dtype);
    if (overlaps(new_residual_out, nb, x, nb) || overlaps(new_residual_out, nb, residual, nb) ||
        overlaps(normed_out, nb, x, nb) || overlaps(normed_out, nb, residual, nb) ||
        overlaps(normed_out, nb, new_residual_out, nb))
      return TTQ_ERR_ALIAS;
  }
  // two to four rows: the normalization as a launch of its own (it writes the rows the caller asked for anyway),
  // then one pass over the weights for all rows -- the one-launch form below reads the weights once per row
  if (m >= 2 && m <= 4 && normed_out &&
      (silu_mul ? ttq::gemv_q4k_stream4_fused_supported(x_dtype, m, n_out, n_in)
                : ttq::gemv_q4k_stream4_supported(TTQ_Q4_K, x_dtype, m, n_out, n_in))) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = ttq::launch_rmsnorm(x, residual, gamma, eps, x_dtype, new_residual_out, normed_out, m, n_in, s);
    if (e != hipSuccess) return hip_status(e);
    e = silu_mul ? ttq::launch_gemv_q4k_stream4_fused(w, normed_out, x_dtype, y, y_dtype, m, n_out, n_in, s)
                 : ttq::launch_gemv_q4k_stream4(w, normed_out, x_dtype, y, y_dtype, nullptr, 0, m, n_out, n_in, s);
    return hip_status(e);
  }
  if (m <= 4 && (silu_mul ? ttq::gemv_q4k_stream_fused_supported(x_dtype, n_out, n_in)
                          : ttq::gemv_q4k_stream_supported(TTQ_Q4_K, x_dtype, n_out, n_in)))
    return hip_status(ttq::launch_gemv_q4k_stream_norm(w, x, x_dtype, y, y_dtype, m, n_out, n_in, silu_mul != 0, residual,
                                                       gamma, eps, new_residual_out, normed_out,
                                                       static_cast<hipStream_t>(stream)));
  if (!ttq::gemv_fused_supported(TTQ_Q4_K, x_dtype, n_out, n_in, silu_mul != 0) || m > kMaxGridRows) return TTQ_ERR_UNSUPPORTED;
  return hip_status(ttq::launch_gemv_fused(w, x, x_dtype, y, y_dtype, nullptr, 0, m, n_out, n_in, silu_mul != 0,
                                           residual, gamma, eps, new_residual_out, normed_out,
                                           static_cast<hipStream_t>(stream)));
}

int ttq_gemm_q4_k_silu_mul(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_ff,
                           int64_t n_in, void* stream) {
  const int rc = check_shape(TTQ_Q4_K, m, n_ff, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (n_ff > 0x3FFFFFFF) return TTQ_ERR_UNSUPPORTED;
  if (m == 0 || n_ff == 0) return TTQ_OK;
  if (!w || !x_bf16 || !y_bf16) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(x_bf16) || !aligned16(y_bf16)) return TTQ_ERR_ALIGN;
  // up to 64 rows: the few-row kernel where it is estimated to be faster than the tiled one
  const bool pc_ok = ttq::gemm_pc_supported(TTQ_Q4_K, m, 2 * n_ff, n_in, 112);
  if (ttq::gemm_skinny_silu_mul_supported(m, n_ff, n_in) &&
      (!pc_ok || ttq::gemm_skinny_silu_mul_estimate_us(m, n_ff, n_in) <
                     ttq::gemm_pc_estimate_us(TTQ_Q4_K, m, 2 * n_ff, n_in)))
    return hip_status(ttq::launch_gemm_skinny_silu_mul(w, x_bf16, y_bf16, TTQ_BF16, nullptr, 0, m, n_ff, n_in,
                                                       static_cast<hipStream_t>(stream)));
  if (!pc_ok) return TTQ_ERR_UNSUPPORTED;
  return hip_status(ttq::launch_gemm_pc_silu_mul(w, x_bf16, y_bf16, TTQ_BF16, nullptr, 0, m, n_ff, n_in,
                                                 static_cast<hipStream_t>(stream)));
}

static int gemm_block(int format, const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                      int64_t n_out, int64_t n_in, void* stream) {
  const int rc = check_shape(format, m, n_out, n_in, 0, 0);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || n_out == 0) return TTQ_OK;    // empty output: nothing to read or write
  if (!w || !x_bf16 || !y_bf16) return TTQ_ERR_NULL;
  if (!aligned16(w) || !aligned16(x_bf16) || !aligned16(y_bf16)) return TTQ_ERR_ALIGN;
  if (!ttq::gemm_supported(format, m, n_out, n_in)) return TTQ_ERR_UNSUPPORTED;
  return hip_status(ttq::launch_gemm(format, w, x_bf16, y_bf16, TTQ_BF16, nullptr, 0, m, n_out, n_in,
                                     static_cast<hipStream_t>(stream)));
}
int ttq_gemm_q4_k(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemm_block(TTQ_Q4_K, w, x_bf16, y_bf16, m, n_out, n_in, stream);
}
int ttq_gemm_q6_k(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemm_block(TTQ_Q6_K, w, x_bf16, y_bf16, m, n_out, n_in, stream);
}
int ttq_gemm_q8_0(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                  int64_t n_in, void* stream) {
  return gemm_block(TTQ_Q8_0, w, x_bf16, y_bf16, m, n_out, n_in, stream);
}

int ttq_dequant_q8_0(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream) {
  return dequant_block(TTQ_Q8_0, w, out, out_dtype, n_out, n_in, stream);
}
int ttq_dequant_q4_k(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream) {
  return dequant_block(TTQ_Q4_K, w, out, out_dtype, n_out, n_in, stream);
}
int ttq_dequant_q6_k(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream) {
  return dequant_block(TTQ_Q6_K, w, out, out_dtype, n_out, n_in, stream);
}

int ttq_dequant_exl3(const uint16_t* trellis, uint16_t* out_f16, int64_t n_out, int64_t n_in, int bits,
                     int codebook, void* stream) {
  if (!trellis || !out_f16) return TTQ_ERR_NULL;
  const int rc = check_shape(TTQ_EXL3, 1, n_out, n_in, bits, codebook);
  if (rc != TTQ_OK) return rc;
  if (!aligned16(trellis) || !aligned16(out_f16)) return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_dequant_exl3(trellis, out_f16, n_out, n_in, bits, codebook,
                                             static_cast<hipStream_t>(stream)));
}

int ttq_hadamard128_f32(float* v, const uint16_t* pre_f16, const uint16_t* post_f16, int64_t n,
                        void* stream) {
  if (!v) return TTQ_ERR_NULL;
  if (n < 0 || n % 128 != 0) return TTQ_ERR_SHAPE;
  if (!aligned16(v)) return TTQ_ERR_ALIGN;
  return hip_status(ttq::launch_hadamard128(v, pre_f16, post_f16, n, static_cast<hipStream_t>(stream)));
}

int ttq_linear_forward(const ttq_qlinear* layer, const void* x, int x_dtype, int64_t m, void* y,
                       int y_dtype, void* stream) {
  if (!layer) return TTQ_ERR_NULL;
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype)) return TTQ_ERR_DTYPE;
  if (layer->bias && !valid_dtype(layer->bias_dtype)) return TTQ_ERR_DTYPE;
  if (layer->precision != TTQ_PRECISION_AUTO && layer->precision != TTQ_PRECISION_F32_SCALES &&
      layer->precision != TTQ_PRECISION_BF16_OK)
    return TTQ_ERR_FORMAT;
  const int rc = check_shape(layer->format, m, layer->n_out, layer->n_in, layer->bits, layer->codebook);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || layer->n_out == 0) return TTQ_OK;   // an empty batch gives an empty output, as F.linear does
  if (!x || !y || !layer->qweight) return TTQ_ERR_NULL;
  if (!aligned16(layer->qweight) || !aligned16(x) || !aligned16(y)) return TTQ_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n_out = layer->n_out, n_in = layer->n_in;

  if (layer->format == TTQ_EXL3) {
    if (!layer->suh || !layer->svh) return TTQ_ERR_NULL;
    if (!aligned8(layer->suh) || !aligned8(layer->svh)) return TTQ_ERR_ALIGN;
    // many rows: rotate the activations once (rounded to fp16) and decode every weight once per 64 rows
    if (layer->precision != TTQ_PRECISION_F32_SCALES && ttq::gemm_exl3_preferred(m, n_out, n_in))
      return hip_status(ttq::launch_gemm_exl3(
          static_cast<const uint16_t*>(layer->qweight), static_cast<const uint16_t*>(layer->suh),
          static_cast<const uint16_t*>(layer->svh), x, x_dtype, y, y_dtype, layer->bias, layer->bias_dtype, m, n_out,
          n_in, layer->bits, layer->codebook, s));
    if (m > kMaxExl3GemvRows) return TTQ_ERR_UNSUPPORTED;
    return hip_status(ttq::launch_gemv_exl3(
        static_cast<const uint16_t*>(layer->qweight), static_cast<const uint16_t*>(layer->suh),
        static_cast<const uint16_t*>(layer->svh), x, x_dtype, y, y_dtype, layer->bias,
        layer->bias_dtype, m, n_out, n_in, layer->bits, layer->codebook, s));
  }

  // Several rows of bf16 activations: the prefill GEMM (weights rounded to bf16) or a few passes of
  // the decode kernels (fp32 scales), whichever the shape makes cheaper.  Up to four rows always
  // decode.
  // (fp16 outputs from bf16 activations: every GEMM kernel but the single-role one, which only more than 4 GiB of
  // activations reach, stores them)
  const bool gemm_ok = x_dtype == TTQ_BF16 &&
                       (y_dtype == TTQ_BF16 || y_dtype == TTQ_F32 ||
                        (y_dtype == TTQ_F16 && (ttq::gemm_skinny_supported(layer->format, m, n_out, n_in) ||
                                                ttq::gemm_pc_supported(layer->format, m, n_out, n_in, 112)))) &&
                       (layer->format == TTQ_Q4_K || layer->format == TTQ_Q6_K || layer->format == TTQ_Q8_0) &&
                       ttq::gemm_supported(layer->format, m, n_out, n_in);
  // TTQ_FORWARD_ROUTE (developer builds, A/B measurements): 1 = always the decode kernels, 2 = the GEMM whenever it exists
  static const int knob = ttq::dev_knob("TTQ_FORWARD_ROUTE", 0);
  const int route = layer->precision == TTQ_PRECISION_F32_SCALES ? 1 : knob;
  if (gemm_ok && m >= 5 && route != 1) {
    if (route == 2 ||
        ttq::gemm_estimate_us(layer->format, m, n_out, n_in) < ttq::gemv_estimate_us(layer->format, x_dtype, m, n_out, n_in))
      return hip_status(ttq::launch_gemm(layer->format, layer->qweight, static_cast<const uint16_t*>(x), y, y_dtype,
                                         layer->bias, layer->bias_dtype, m, n_out, n_in, s));
  }
  const bool block_fmt = layer->format == TTQ_Q4_K || layer->format == TTQ_Q6_K || layer->format == TTQ_Q8_0;
  // fp16 activations, five rows or more: the operator computes in the type of x, so the weights are rounded to fp16
  // (11 bits: the result stays in the 1e-3 class of the decode kernels) and multiplied on the fp16 matrix cores --
  // by the few-row kernel (64 rows per launch) or, from where it is cheaper, by the prefill GEMM over a packed fp16
  // copy of the activations -- unless passes of the decode kernels are cheaper still.
  if (x_dtype == TTQ_F16 && block_fmt && m >= 5 && route != 1) {
    float us_few = 1e30f, us_gemm = 1e30f;
    if (ttq::gemm_skinny_supported(layer->format, m < 64 ? m : 64, n_out, n_in)) {
      const int64_t full = m / 64, rest = m % 64;
      us_few = (float)full * ttq::gemm_skinny_estimate_us(layer->format, 64, n_out, n_in);
      if (rest) us_few += ttq::gemm_skinny_estimate_us(layer->format, rest, n_out, n_in);
    }
    if (m > 64 && ttq::gemm_pc_supported(layer->format, m < 8192 ? m : 8192, n_out, n_in, 112))
      us_gemm = ttq::gemm_pc_estimate_us(layer->format, m, n_out, n_in) + 2.5f + (float)(m * n_in * 4) / 3.0e6f;
    const float us_gemv = ttq::gemv_estimate_us(layer->format, x_dtype, m, n_out, n_in);
    // (several launches of the few-row kernel against one short round of the tiled kernel: the margin of the bf16
    // chooser, whose estimate for the tiled kernel is fitted to full rounds and about a third too high for a short one)
    if (us_gemm < (m > 64 ? us_few / 0.65f : us_few) && (route == 2 || us_gemm < us_gemv))
      return hip_status(ttq::launch_gemm_pc_x(layer->format, layer->qweight, x, x_dtype, y, y_dtype, layer->bias,
                                              layer->bias_dtype, m, n_out, n_in, s, true));
    if (us_few < 1e29f && (route == 2 || us_few < us_gemv)) {
      if (ttq::route_probe(ttq::kRouteGemmSkinnyChunked)) return TTQ_OK;
      return hip_status(ttq::launch_gemm_skinny_chunked(layer->format, layer->qweight, static_cast<const uint16_t*>(x),
                                                        x_dtype, y, y_dtype, layer->bias, layer->bias_dtype, m, n_out,
                                                        n_in, s));
    }
  }
  // fp32 activations, 256 rows or more, and only where the layer says that bf16 activations will do
  // (TTQ_PRECISION_BF16_OK): the prefill GEMM's packing pass rounds them to bf16 on the way into its workspace
  // (weights and activations rounded to bf16: the 2e-2 class, like the GEMM entry points)
  if (x_dtype == TTQ_F32 && block_fmt && m >= 256 && route != 1 && n_in % 8 == 0 &&
      layer->precision == TTQ_PRECISION_BF16_OK &&
      ttq::gemm_pc_supported(layer->format, m < 8192 ? m : 8192, n_out, n_in, 112)) {
    return hip_status(ttq::launch_gemm_pc_x(layer->format, layer->qweight, x, x_dtype, y, y_dtype, layer->bias,
                                            layer->bias_dtype, m, n_out, n_in, s));
  }
  // fp32 activations, five rows or more: the fp16 form of the prefill GEMM over a copy in which every row has been
  // scaled by a power of two (its largest magnitude to 2^14) and rounded to fp16, the factor undone on the sums.
  // With the weights rounded to fp16 as well the result stays in the 1e-3 class of the decode kernels (about 2e-4
  // measured), which take these activations as 15-bit block fixed point themselves, at a fraction of the time of
  // their passes (14336 x 4096 at 512 rows: 2.2 ms in passes of four rows).
  // A few rows take the few-row kernel in fp16 over a row-major copy scaled the same way (one pass of a workgroup
  // per row), as fp16 activations do: 14336 x 4096 at 8 rows 17 us against 28 us of the GEMM.  From two rows on
  // that also beats passes of the decode kernels where those have no kernel of several rows for fp32 activations
  // (Q6_K 14336 x 4096 at four rows: 20 us against 49; the 128256 x 4096 head 149 against 408).
  if (x_dtype == TTQ_F32 && block_fmt && m >= 2 && route != 1) {
    float us_few = 1e30f, us_gemm = 1e30f;
    // (up to 8192 rows: the scaled copy of all rows sits in the workspace at once)
    if (m <= 8192 && ttq::gemm_skinny_supported(layer->format, m < 64 ? m : 64, n_out, n_in)) {
      // (the scaling pass: a workgroup per row walks it twice -- 3 us on rows of 4096 values, 4.3 us on 14336)
      const int64_t full = m / 64, rest = m % 64;
      us_few = (float)full * ttq::gemm_skinny_estimate_us(layer->format, 64, n_out, n_in) + 2.5f + (float)n_in * 0.13e-3f;
      if (rest) us_few += ttq::gemm_skinny_estimate_us(layer->format, rest, n_out, n_in);
    }
    if (m >= 5 && ttq::gemm_pc_supported(layer->format, m < 8192 ? m : 8192, n_out, n_in, 112))
      us_gemm = ttq::gemm_pc_estimate_us(layer->format, m, n_out, n_in) + 5.f + (float)(m * n_in * 10) / 3.0e6f;
    const float us_gemv = ttq::gemv_estimate_us(layer->format, x_dtype, m, n_out, n_in);
    if ((m > 64 ? us_few / 0.65f : us_few) < us_gemm && (route == 2 || us_few < us_gemv)) {
      if (ttq::route_probe(ttq::kRouteGemmSkinnyF32ScaledF16)) return TTQ_OK;
      return hip_status(ttq::launch_gemm_skinny_f32(layer->format, layer->qweight, static_cast<const float*>(x), y, y_dtype,
                                                    layer->bias, layer->bias_dtype, m, n_out, n_in, s));
    }
    if (us_gemm < 1e29f && (route == 2 || us_gemm < us_gemv))
      return hip_status(ttq::launch_gemm_pc_x(layer->format, layer->qweight, x, x_dtype, y, y_dtype, layer->bias,
                                              layer->bias_dtype, m, n_out, n_in, s, true));
  }
  return hip_status(launch_gemv_any_m(layer->format, layer->qweight, x, x_dtype, y, y_dtype, layer->bias,
                                      layer->bias_dtype, m, n_out, n_in, s));
}

// ---- which kernel family ttq_linear_forward would launch
int ttq_route(const ttq_qlinear* layer, int64_t m, int x_dtype, int y_dtype) {
  if (!layer) return TTQ_ERR_NULL;
  // the dispatch itself, with a probe bound to this thread (nothing is launched, allocated or dereferenced) and
  // stand-ins for the buffers
  ttq_qlinear probe_layer = *layer;
  alignas(16) static char stand_in[16];
  probe_layer.qweight = stand_in;
  if (probe_layer.format == TTQ_EXL3) {
    probe_layer.suh = stand_in;
    probe_layer.svh = stand_in;
  }
  if (layer->bias) probe_layer.bias = stand_in;
  ttq::RouteProbe probe{0};
  ttq::t_route_probe = &probe;
  const int rc = ttq_linear_forward(&probe_layer, stand_in, x_dtype, m, stand_in, y_dtype, nullptr);
  ttq::t_route_probe = nullptr;
  return rc != TTQ_OK ? rc : probe.route;
}

const char* ttq_route_name(int route) {
  switch (route) {
    case TTQ_ROUTE_NONE: return "none (empty call)";
    case TTQ_ROUTE_GEMV_Q4K_STREAM: return "gemv_q4k_stream";
    case TTQ_ROUTE_GEMV_Q4K_STREAM4: return "gemv_q4k_stream4";
    case TTQ_ROUTE_GEMV_Q4K_SLICE: return "gemv_q4k_slice";
    case TTQ_ROUTE_GEMV_Q4K_BATCH4: return "gemv_q4k_batch4";
    case TTQ_ROUTE_GEMV_Q4K_BATCH: return "gemv_q4k_batch";
    case TTQ_ROUTE_GEMV_Q4K_MFMA: return "gemv_q4k_mfma";
    case TTQ_ROUTE_GEMV_Q6K_STREAM: return "gemv_q6k_stream";
    case TTQ_ROUTE_GEMV_Q6K_STREAM4: return "gemv_q6k_stream4";
    case TTQ_ROUTE_GEMV_Q8_STREAM: return "gemv_q8_stream";
    case TTQ_ROUTE_GEMV_Q8_WIN: return "gemv_q8_win";
    case TTQ_ROUTE_GEMV_Q8_MFMA: return "gemv_q8_mfma";
    case TTQ_ROUTE_GEMV_DOT2: return "gemv_dot2";
    case TTQ_ROUTE_GEMV_DOT2_MULTI: return "gemv_dot2_multi";
    case TTQ_ROUTE_GEMV_GENERIC: return "gemv_generic";
    case TTQ_ROUTE_GEMV_LONG: return "gemv_long";
    case TTQ_ROUTE_GEMM_SKINNY_F32_SCALED_F16: return "gemm_skinny_f32_scaled_f16";
    case TTQ_ROUTE_GEMM_PC: return "gemm_pc";
    case TTQ_ROUTE_GEMM_PC_SPLIT_K: return "gemm_pc_split_k";
    case TTQ_ROUTE_GEMM_SKINNY: return "gemm_skinny";
    case TTQ_ROUTE_GEMM_SKINNY_CHUNKED: return "gemm_skinny_chunked";
    case TTQ_ROUTE_GEMM_Q4K_TILES: return "gemm_q4k_tiles";
    case TTQ_ROUTE_GEMM_PC_BF16_COPY: return "gemm_pc_bf16_copy";
    case TTQ_ROUTE_GEMM_PC_PACKED: return "gemm_pc_packed";
    case TTQ_ROUTE_GEMM_PC_F16: return "gemm_pc_f16";
    case TTQ_ROUTE_GEMM_PC_F32_SCALED_F16: return "gemm_pc_f32_scaled_f16";
    case TTQ_ROUTE_GEMM_PC_PACKED_SPLIT_K: return "gemm_pc_packed_split_k";
    case TTQ_ROUTE_EXL3_GEMV: return "exl3_gemv";
    case TTQ_ROUTE_EXL3_GEMV_SLICED: return "exl3_gemv_sliced";
    case TTQ_ROUTE_EXL3_GEMM: return "exl3_gemm";
    case TTQ_ROUTE_EXL3_GEMV_TWO_LAUNCHES: return "exl3_gemv_two_launches";
    default: return "unknown route";
  }
}

// ---- caller-owned workspaces
int64_t ttq_workspace_bytes(const ttq_qlinear* layer, int64_t m, int x_dtype) {
  if (!layer) return TTQ_ERR_NULL;
  if (!valid_dtype(x_dtype)) return TTQ_ERR_DTYPE;
  const int rc = check_shape(layer->format, m, layer->n_out, layer->n_in, layer->bits, layer->codebook);
  if (rc != TTQ_OK) return rc;
  if (m == 0 || layer->n_out == 0) return 0;
  const int64_t n_out = layer->n_out, n_in = layer->n_in;
  const int64_t header = (int64_t)ttq::caller_workspace_header_bytes();
  constexpr int64_t kExl3Rows = 4096, kGemmRows = 8192;   // rows whose rotated / packed copy is in the workspace at a time
  if (layer->format == TTQ_EXL3) {              // hand-off words; the rotated activations of the many-row form
    const int64_t block_rows = ((m < kExl3Rows ? m : kExl3Rows) + 15) / 16 * 16;   // whole blocks of 16 rows
    const int64_t partials = (int64_t)ttq::gemm_exl3_partials_bytes(m, n_out, n_in);
    return header + ((block_rows * n_in * 2 + 255) & ~(int64_t)255) + ((partials + 255) & ~(int64_t)255);
  }
  // the decode kernels take no workspace (two to four rows of fp32 activations may take the few-row kernel over a
  // scaled fp16 copy)
  if (m < 5 && !(x_dtype == TTQ_F32 && m >= 2)) return 0;
  // the packed bf16 copy of the activations where the prefill GEMM wants one, then the partial sums of a launch
  // split along K: the prefill GEMM's exact size for every row count it can be called with here, and the few-row
  // kernel's bound (one 64 x 64 tile of sums per compute unit)
  const int64_t block_rows = m < kGemmRows ? m : kGemmRows;
  // (fp16 activations beyond 64 rows may take the prefill GEMM over a packed fp16 copy; fp32 ones over a scaled
  // fp16 copy, or a bf16 copy where the layer allows it)
  const int copy_dtype = (x_dtype == TTQ_F16 && m > 64) || x_dtype == TTQ_F32 ? x_dtype : TTQ_BF16;
  int64_t scratch = ((int64_t)ttq::gemm_pc_packed_bytes(m, n_out, n_in, copy_dtype) + 255) & ~(int64_t)255;
  int64_t partials = (int64_t)ttq::device_num_cus() * (16 * 4 * (16 * 4 + 1) * 4);
  const int64_t rows[3] = {m, block_rows, m % kGemmRows};
  for (int64_t r : rows) {
    if (r <= 0) continue;
    const int64_t p = (int64_t)ttq::gemm_pc_partials_bytes(r, n_out, n_in);
    if (p > partials) partials = p;
  }
  return header + scratch + ((partials + 255) & ~(int64_t)255);
}

static int ws_check(void* ws, int64_t ws_bytes) {
  if (ws_bytes < 0 || (ws_bytes > 0 && (!ws || !aligned16(ws)))) return TTQ_ERR_WORKSPACE;
  return TTQ_OK;
}
// the status of a call that ran with a caller-owned workspace bound
static int ws_status(int rc, const ttq::CallerWsScope& scope) { return scope.too_small() ? TTQ_ERR_WORKSPACE : rc; }

int ttq_linear_forward_ws(const ttq_qlinear* layer, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
                          void* ws, int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(ttq_linear_forward(layer, x, x_dtype, m, y, y_dtype, stream), scope);
}

int ttq_gemm_q4_k_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                     int64_t n_in, void* ws, int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(gemm_block(TTQ_Q4_K, w, x_bf16, y_bf16, m, n_out, n_in, stream), scope);
}
int ttq_gemm_q6_k_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                     int64_t n_in, void* ws, int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(gemm_block(TTQ_Q6_K, w, x_bf16, y_bf16, m, n_out, n_in, stream), scope);
}
int ttq_gemm_q8_0_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m, int64_t n_out,
                     int64_t n_in, void* ws, int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(gemm_block(TTQ_Q8_0, w, x_bf16, y_bf16, m, n_out, n_in, stream), scope);
}
int ttq_gemm_exl3_ws(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16, const void* x,
                     int x_dtype, float* y, int64_t m, int64_t n_out, int64_t n_in, int bits, int codebook, void* ws,
                     int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(ttq_gemm_exl3(trellis, suh_f16, svh_f16, x, x_dtype, y, m, n_out, n_in, bits, codebook, stream), scope);
}
int ttq_gemv_exl3_ws(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16, const uint16_t* x_f16,
                     float* y, int64_t m, int64_t n_out, int64_t n_in, int bits, int codebook, void* ws,
                     int64_t ws_bytes, void* stream) {
  const int rc = ws_check(ws, ws_bytes);
  if (rc != TTQ_OK) return rc;
  ttq::CallerWsScope scope(ws, (size_t)ws_bytes);
  return ws_status(ttq_gemv_exl3(trellis, suh_f16, svh_f16, x_f16, y, m, n_out, n_in, bits, codebook, stream), scope);
}

int ttq_release_workspaces(void) { return hip_status(ttq::release_stream_workspaces()); }

int ttq_debug_set_exl3_poll_limit(int limit) { return ttq::exl3_set_poll_limit(limit); }

}  // extern "C"
