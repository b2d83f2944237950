// Prefill GEMM for Q4_K weights on gfx950:  Y (m, n_out) = X (m, n_in) * W^T.
//
// Replaces F.linear(x, weight) for a multi-row bf16 activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81; the prefill case of
//  workspace/transformers/src/layers/attn.nim:154-156).
//
// Each workgroup owns a 128 x 128 tile of Y.  Per K step of 64 it
//   - loads 32 packed bytes per weight row straight from the Q4_K super-block (one chunk:
//     low nibbles = sub-block 2c, high nibbles = sub-block 2c+1), dequantizes them in
//     registers with the canonical arithmetic d*sc*q - dmin*m, rounds to bf16
//     (nearest-even) and writes the tile to LDS,
//   - copies the matching 128 x 64 slab of X to LDS,
//   - multiplies with v_mfma_f32_32x32x16_bf16, fp32 accumulators in registers.
// LDS rows are padded by 16 bytes so the 16-byte fragment reads of 32 consecutive rows hit
// distinct banks.
#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kLdsStride = BK + 8;  // bf16 elements per LDS row (144 bytes)
constexpr int kGemmThreads = 256;

__device__ __forceinline__ bf16x8_t lds_frag(const uint16_t* base, int row, int kofs) {
  return *reinterpret_cast<const bf16x8_t*>(base + row * kLdsStride + kofs);
}

template <typename YT>
__global__ void __launch_bounds__(kGemmThreads)
gemm_q4k_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in) {
  __shared__ __attribute__((aligned(16))) uint16_t sx[BM * kLdsStride];
  __shared__ __attribute__((aligned(16))) uint16_t sw[BN * kLdsStride];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;  // wave tile origin inside the block tile
  const int64_t row_bytes = (int64_t)(n_in >> 8) * 144;

  // loader roles: thread -> (tile row, 16-byte half)
  const int lrow = tid >> 1, lhalf = tid & 1;
  const bool w_ok = (n0 + lrow) < n_out;
  const bool x_ok = (m0 + lrow) < m;
  const uint8_t* wrow = w + row_bytes * (int64_t)(w_ok ? n0 + lrow : 0);
  const uint16_t* xrow = x + (int64_t)(x_ok ? m0 + lrow : 0) * n_in;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int ksteps = n_in / BK;
  for (int ks = 0; ks < ksteps; ks++) {
    // ---- global -> registers
    const int b = ks >> 2, c = ks & 3;
    uint4 hdr = make_uint4(0, 0, 0, 0), q = make_uint4(0, 0, 0, 0);
    if (w_ok) {
      const uint8_t* p = wrow + 144 * (int64_t)b;
      hdr = load16_a16(p);
      q = load16_a16(p + 16 + 32 * c + 16 * lhalf);
    }
    uint4 xv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      xv[i] = x_ok ? *reinterpret_cast<const uint4*>(xrow + ks * BK + 32 * lhalf + 8 * i)
                   : make_uint4(0, 0, 0, 0);
    }
    // ---- dequantize 16 low-nibble + 16 high-nibble weights
    const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16));
    uint32_t sc1, mn1, sc2, mn2;
    q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c, sc1, mn1);
    q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c + 1, sc2, mn2);
    const float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
    const float d2 = d * (float)sc2, m2 = dmin * (float)mn2;
    const uint32_t qd[4] = {q.x, q.y, q.z, q.w};
    uint32_t lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float fl[4], fh[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const uint32_t byte = (qd[i] >> (8 * k)) & 0xFFu;
        const float tl = d1 * (float)(byte & 0xFu);
        const float th = d2 * (float)(byte >> 4);
        fl[k] = tl - m1;
        fh[k] = th - m2;
      }
      lo[2 * i] = pack_bf16x2(fl[0], fl[1]);
      lo[2 * i + 1] = pack_bf16x2(fl[2], fl[3]);
      hi[2 * i] = pack_bf16x2(fh[0], fh[1]);
      hi[2 * i + 1] = pack_bf16x2(fh[2], fh[3]);
    }
    __syncthreads();  // previous step's fragment reads are done
    {
      uint4* dw = reinterpret_cast<uint4*>(sw + lrow * kLdsStride + 16 * lhalf);
      dw[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
      dw[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
      uint4* dh = reinterpret_cast<uint4*>(sw + lrow * kLdsStride + 32 + 16 * lhalf);
      dh[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
      dh[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
      uint4* dx = reinterpret_cast<uint4*>(sx + lrow * kLdsStride + 32 * lhalf);
#pragma unroll
      for (int i = 0; i < 4; i++) dx[i] = xv[i];
    }
    __syncthreads();
    // ---- MFMA: A = X rows (m), B = W rows (n); lane holds row lane%32, k = 8*(lane/32)..+8
    const int fr = lane & 31, fk = (lane >> 5) * 8;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8_t a[2], bq[2];
#pragma unroll
      for (int i = 0; i < 2; i++) a[i] = lds_frag(sx, wm + 32 * i + fr, kk + fk);
#pragma unroll
      for (int j = 0; j < 2; j++) bq[j] = lds_frag(sw, wn + 32 * j + fr, kk + fk);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], bq[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue: C layout of the 32x32 MFMA: column = lane%32, row = 8*(r/4) + 4*(lane/32) + r%4
  const int cn = lane & 31, rbase = (lane >> 5) * 4;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int n = n0 + wn + 32 * j + cn;
    if (n >= n_out) continue;
    float bv = 0.f;
    if (bias) {
      if (bias_dtype == kF32) bv = static_cast<const float*>(bias)[n];
      else {
        const uint16_t bb = static_cast<const uint16_t*>(bias)[n];
        bv = bias_dtype == kF16 ? f16_bits_to_f32(bb) : bf16_bits_to_f32(bb);
      }
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int mm = m0 + wm + 32 * i + 8 * (r >> 2) + rbase + (r & 3);
        if (mm < m) YElem<YT>::store(y, (int64_t)mm * n_out + n, acc[i][j][r] + bv);
      }
    }
  }
}

hipError_t launch_gemm_q4k(const void* w, const uint16_t* x_bf16, void* y, int y_dtype,
                           const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                           hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  const dim3 grid((unsigned)((n_out + BN - 1) / BN), (unsigned)((m + BM - 1) / BM)), block(kGemmThreads);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  if (y_dtype == kBF16)
    hipLaunchKernelGGL(gemm_q4k_kernel<bf16_tag>, grid, block, 0, s, wb, x_bf16,
                       static_cast<bf16_tag*>(y), bias, bias_dtype, (int)m, (int)n_out, (int)n_in);
  else if (y_dtype == kF32)
    hipLaunchKernelGGL(gemm_q4k_kernel<float>, grid, block, 0, s, wb, x_bf16, static_cast<float*>(y),
                       bias, bias_dtype, (int)m, (int)n_out, (int)n_in);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ttq
