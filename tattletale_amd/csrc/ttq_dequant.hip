// Device dequantizers for the block formats: packed bytes -> dense (n_out, n_in) values.
// They make the bit-exactness contract observable on the GPU: with out_dtype fp32 the
// result must equal the canonical CPU dequantizer bit for bit; with bf16 it is that value
// rounded to nearest-even, i.e. what the prefill GEMM feeds to the matrix cores.
//
// The dense tensor produced here is what the reference's Linear would have stored as
// `weight` (workspace/transformers/src/layers/linear.nim:19-27).
#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {

// ---- Q8_0: { f16 d; i8 qs[32]; } -> y[i] = f32(d) * qs[i].  One thread per 4 weights.
template <typename OT>
__global__ void __launch_bounds__(256) dequant_q8_0_kernel(const uint8_t* __restrict__ w,
                                                           OT* __restrict__ out, int64_t nquads) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= nquads) return;
  const int64_t b = g >> 3;
  const int part = (int)(g & 7);
  const uint8_t* p = w + 34 * b;
  const float d = f16_bits_to_f32(load2(p));
  const int8_t* qs = reinterpret_cast<const int8_t*>(p + 2 + 4 * part);
#pragma unroll
  for (int i = 0; i < 4; i++) YElem<OT>::store(out, 32 * b + 4 * part + i, d * (float)qs[i]);
}

// ---- Q4_K: { f16 d; f16 dmin; u8 scales[12]; u8 qs[128]; }.  One thread per qs dword:
// 4 low-nibble weights of sub-block 2c and 4 high-nibble weights of sub-block 2c+1.
template <typename OT>
__global__ void __launch_bounds__(256) dequant_q4_k_kernel(const uint8_t* __restrict__ w,
                                                           OT* __restrict__ out, int64_t nthreads) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= nthreads) return;
  const int64_t b = g >> 5;
  const int t = (int)(g & 31);
  const int c = t >> 3, i = t & 7;
  const uint32_t* p = reinterpret_cast<const uint32_t*>(w + 144 * b);
  const uint32_t dm = p[0], s0 = p[1], s1 = p[2], s2 = p[3];
  const float d = f16_bits_to_f32((uint16_t)(dm & 0xFFFF));
  const float dmin = f16_bits_to_f32((uint16_t)(dm >> 16));
  uint32_t sc1, mn1, sc2, mn2;
  q4k_scale_min(s0, s1, s2, 2 * c, sc1, mn1);
  q4k_scale_min(s0, s1, s2, 2 * c + 1, sc2, mn2);
  const float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
  const float d2 = d * (float)sc2, m2 = dmin * (float)mn2;
  const uint32_t q = p[4 + 8 * c + i];
  const int64_t o = 256 * b + 64 * c + 4 * i;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t byte = (q >> (8 * k)) & 0xFFu;
    const float lo = d1 * (float)(byte & 0xFu);
    const float hi = d2 * (float)(byte >> 4);
    YElem<OT>::store(out, o + k, lo - m1);
    YElem<OT>::store(out, o + 32 + k, hi - m2);
  }
}

// ---- Q6_K: { u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d; }.  One thread per
// (block, half h, l-quad): 4 positions l, each yielding 4 weights (l, l+32, l+64, l+96).
template <typename OT>
__global__ void __launch_bounds__(256) dequant_q6_k_kernel(const uint8_t* __restrict__ w,
                                                           OT* __restrict__ out, int64_t nthreads) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= nthreads) return;
  const int64_t b = g >> 4;
  const int t = (int)(g & 15);
  const int h = t >> 3, l0 = (t & 7) * 4;
  const uint8_t* p = w + 210 * b;
  const uint8_t* ql = p + 64 * h;
  const uint8_t* qh = p + 128 + 32 * h;
  const int8_t* sc = reinterpret_cast<const int8_t*>(p + 192 + 8 * h);
  const float d = f16_bits_to_f32(load2(p + 208));
  const int is = l0 >> 4;
  const float s1 = d * (float)sc[is + 0], s2 = d * (float)sc[is + 2];
  const float s3 = d * (float)sc[is + 4], s4 = d * (float)sc[is + 6];
  const int64_t o = 256 * b + 128 * h + l0;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const int l = l0 + k;
    const uint32_t a = ql[l], bq = ql[l + 32], hq = qh[l];
    const int q1 = (int)((a & 0xF) | (((hq >> 0) & 3) << 4)) - 32;
    const int q2 = (int)((bq & 0xF) | (((hq >> 2) & 3) << 4)) - 32;
    const int q3 = (int)((a >> 4) | (((hq >> 4) & 3) << 4)) - 32;
    const int q4 = (int)((bq >> 4) | (((hq >> 6) & 3) << 4)) - 32;
    YElem<OT>::store(out, o + k, s1 * (float)q1);
    YElem<OT>::store(out, o + k + 32, s2 * (float)q2);
    YElem<OT>::store(out, o + k + 64, s3 * (float)q3);
    YElem<OT>::store(out, o + k + 96, s4 * (float)q4);
  }
}

template <typename OT>
static hipError_t launch_dequant_t(int format, const void* w, OT* out, int64_t n_out, int64_t n_in,
                                   hipStream_t s) {
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  const int64_t nelem = n_out * n_in;
  if (nelem == 0) return hipSuccess;
  int64_t nthreads;
  switch (format) {
    case kQ8_0: nthreads = nelem / 4; break;
    case kQ4_K: nthreads = nelem / 8; break;
    case kQ6_K: nthreads = nelem / 16; break;
    default: return hipErrorInvalidValue;
  }
  const int64_t nblocks = (nthreads + 255) / 256;
  if (nblocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)nblocks), block(256);
  switch (format) {
    case kQ8_0: hipLaunchKernelGGL(dequant_q8_0_kernel<OT>, grid, block, 0, s, wb, out, nthreads); break;
    case kQ4_K: hipLaunchKernelGGL(dequant_q4_k_kernel<OT>, grid, block, 0, s, wb, out, nthreads); break;
    case kQ6_K: hipLaunchKernelGGL(dequant_q6_k_kernel<OT>, grid, block, 0, s, wb, out, nthreads); break;
  }
  return hipGetLastError();
}

hipError_t launch_dequant(int format, const void* w, void* out, int out_dtype, int64_t n_out,
                          int64_t n_in, hipStream_t s) {
  switch (out_dtype) {
    case kF32: return launch_dequant_t<float>(format, w, static_cast<float*>(out), n_out, n_in, s);
    case kF16: return launch_dequant_t<f16_tag>(format, w, static_cast<f16_tag*>(out), n_out, n_in, s);
    case kBF16: return launch_dequant_t<bf16_tag>(format, w, static_cast<bf16_tag*>(out), n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ttq
