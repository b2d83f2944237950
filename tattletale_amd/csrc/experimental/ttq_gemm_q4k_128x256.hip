// EXPERIMENTAL, not part of the built library (kept as the starting point for the next tiling;
// it passes the GEMM parity tests but runs at 99 us for M = 512, slower than the shipped kernel).
//
// Prefill GEMM for Q4_K weights on gfx950, second tiling:  Y (m, n_out) = X (m, n_in) * W^T.
//
// Same operator as ttq_gemm_q4k.hip (F.linear with a multi-row bf16 activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81), re-tiled around what the hardware
// measures as scarce:
//   * the vector-memory path: a wavefront retires one 16-byte-per-lane load every 64 clk when the
//     lanes cover whole 128-byte lines and every 128 clk otherwise, so X is fetched with
//     full-line loads by all 256 threads into LDS and shared by the four wavefronts;
//   * LDS bandwidth: only the A operand (X) is read from LDS; each wavefront owns 64 columns
//     of W and dequantizes their packed bytes directly into MFMA B-operand registers;
//   * VALU throughput: the dequantization (about 3 instructions per weight) is woven between
//     the MFMAs of the previous k-quarter.
// Tile: 128 rows of X x 256 columns of W per workgroup, four wavefronts of 128 x 64,
// v_mfma_f32_16x16x32_bf16, 128 k per super-step.
//
// k bookkeeping inside a super-step of 128 k (two 32-byte chunks c0, c0+1 of a super-block):
// lane (n = lane%16, g = lane/16) loads, for each of its 4 column blocks j, the 16 bytes
// [16*(g&1), +16) of chunk c0 + (g>>1) of row 16j+n.  Quarter kq of the super-step multiplies
//   kq 0: low nibbles of bytes 0..7     kq 1: low nibbles of bytes 8..15
//   kq 2: high nibbles of bytes 0..7    kq 3: high nibbles of bytes 8..15
// so the 8 k values lane group g contributes to MFMA kq are
//   k = 64*(g>>1) + 32*(kq>>1) + 16*(g&1) + 8*(kq&1) + 0..7        (relative to the super-step)
// and the A fragments are read from the X tile in LDS at exactly those k.
#include "../ttq_device.h"
#include "../ttq_internal.h"

#include <stdlib.h>
#include <type_traits>

namespace ttq {

namespace v3 {

constexpr int kThreads = 256;
constexpr int BM = 128, BN = 256, KS = 128;        // tile and super-step
constexpr int kXStride = KS * 2 + 16;              // bytes per X row in LDS (16 B pad: conflict-free)
constexpr int kXTileBytes = BM * kXStride;
constexpr int kScaleFloats = 4 * 64 * 16;          // per wavefront: 64 rows x (8 d*sc, 8 -dmin*m)

template <typename YT>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_q4k_v3_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                   const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                   int n_tiles, int m_tiles) {
  __shared__ __attribute__((aligned(16))) uint8_t sx[kXTileBytes];
  __shared__ __attribute__((aligned(16))) float ssc[kScaleFloats];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // consecutive workgroups share the W tile and differ in the row tile: W is fetched from HBM once
  const int m_tile = blockIdx.x % m_tiles, n_tile = blockIdx.x / m_tiles;
  if (n_tile >= n_tiles) return;
  const int m0 = m_tile * BM, n0 = n_tile * BN + wave * 64;
  const int64_t row_bytes = (int64_t)(n_in >> 8) * 144;
  const int ln = lane & 15, lg = lane >> 4;

  // ---- W roles
  // quants: row 16j + ln of this wavefront's 64 columns, 16 bytes at 64*pair + 16*lg of the qs area
  // (32-bit byte offsets from the uniform base pointers keep address registers few; the launcher
  // routes buffers of 4 GiB or more to the other kernel)
  uint32_t wq[4];
#pragma unroll
  for (int j = 0; j < 4; j++) wq[j] = (uint32_t)(row_bytes * (int64_t)min(n0 + 16 * j + ln, n_out - 1) + 16 + 16 * lg);
  // header: lane decodes the whole header of row 16*lg + ln once per super-block
  const uint8_t* wh = w + row_bytes * (int64_t)min(n0 + 16 * lg + ln, n_out - 1);
  float* my_sc = ssc + wave * (64 * 16);

  // ---- X staging role: per pass q thread t covers row 16q + t/16, bytes 16*(t%16)
  const int xr0 = tid >> 4, xb = (tid & 15) * 16;
  const uint8_t* xbytes = reinterpret_cast<const uint8_t*>(x);
  uint32_t xg[8];
#pragma unroll
  for (int q = 0; q < 8; q++) xg[q] = (uint32_t)((int64_t)min(m0 + 16 * q + xr0, m - 1) * n_in * 2 + xb);

  f32x4_t acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int nsteps = n_in / KS;      // super-steps; two per super-block
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // plain vector: stays in registers
  u32x4_t xstage[8];
  uint4 hdr;

  auto load_x = [&](int st) {
#pragma unroll
    for (int q = 0; q < 8; q++)
      xstage[q] = *reinterpret_cast<const u32x4_t*>(xbytes + (xg[q] + (uint32_t)st * (KS * 2)));
  };
  auto store_x = [&]() {
#pragma unroll
    for (int q = 0; q < 8; q++) *reinterpret_cast<u32x4_t*>(sx + (16 * q + xr0) * kXStride + xb) = xstage[q];
  };
  auto load_w = [&](uint4 (&dst)[4], int st) {
    const uint32_t off = 144u * (uint32_t)(st >> 1) + 64u * (uint32_t)(st & 1);
#pragma unroll
    for (int j = 0; j < 4; j++) dst[j] = load16_a16(w + (wq[j] + off));
  };
  // decode a header into d*sc_s and -(dmin*m_s), s = 0..7, for this lane's header row
  auto store_scales = [&](const uint4& h) {
    const float d = f16_bits_to_f32((uint16_t)(h.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(h.x >> 16));
    float v[16];
#pragma unroll
    for (int s = 0; s < 8; s++) {
      uint32_t sc, mn;
      q4k_scale_min(h.y, h.z, h.w, s, sc, mn);
      v[s] = d * (float)sc;
      v[8 + s] = -(dmin * (float)mn);
    }
    float4* dst = reinterpret_cast<float4*>(my_sc + (16 * lg + ln) * 16);
#pragma unroll
    for (int q = 0; q < 4; q++) dst[q] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
  };

  // B operands of one k-quarter for the 4 column blocks, from the raw 16 bytes of each
  auto dequant_quarter = [&](auto kqc, const uint4 (&raw)[4], const float (&d1)[4], const float (&nm1)[4],
                             const float (&d2)[4], const float (&nm2)[4], bf16x8_t (&bq)[4]) {
    constexpr int kq = decltype(kqc)::value;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint32_t q0 = (kq & 1) ? raw[j].z : raw[j].x, q1 = (kq & 1) ? raw[j].w : raw[j].y;
      const uint32_t a = (kq & 2) ? ((q0 >> 4) & 0x0F0F0F0Fu) : (q0 & 0x0F0F0F0Fu);
      const uint32_t b = (kq & 2) ? ((q1 >> 4) & 0x0F0F0F0Fu) : (q1 & 0x0F0F0F0Fu);
      const float dd = (kq & 2) ? d2[j] : d1[j], mm = (kq & 2) ? nm2[j] : nm1[j];
      // one fused multiply-add per weight == the canonical two-step form (d*sc*q is exact)
      uint32_t p[4];
      p[0] = pack_bf16x2(fmaf_(dd, (float)(a & 0xFFu), mm), fmaf_(dd, (float)((a >> 8) & 0xFFu), mm));
      p[1] = pack_bf16x2(fmaf_(dd, (float)((a >> 16) & 0xFFu), mm), fmaf_(dd, (float)(a >> 24), mm));
      p[2] = pack_bf16x2(fmaf_(dd, (float)(b & 0xFFu), mm), fmaf_(dd, (float)((b >> 8) & 0xFFu), mm));
      p[3] = pack_bf16x2(fmaf_(dd, (float)((b >> 16) & 0xFFu), mm), fmaf_(dd, (float)(b >> 24), mm));
      __builtin_memcpy(&bq[j], p, 16);
    }
  };
  // scales of this lane's chunk (c0 + (lg>>1)) for the 4 column blocks, from the wavefront's table
  auto fetch_scales = [&](int pair, float (&d1)[4], float (&nm1)[4], float (&d2)[4], float (&nm2)[4]) {
    const int s0 = 2 * (2 * pair + (lg >> 1));   // sub-blocks s0 (low nibbles) and s0+1 (high)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float* t = my_sc + (16 * j + ln) * 16;
      d1[j] = t[s0]; d2[j] = t[s0 + 1];
      nm1[j] = t[8 + s0]; nm2[j] = t[8 + s0 + 1];
    }
  };
  // A fragments of one k-quarter: 8 row blocks
  const int a_base = ln * kXStride + 2 * (64 * (lg >> 1) + 16 * (lg & 1));
  auto mfma_quarter = [&](auto kqc, const bf16x8_t (&bq)[4]) {
    constexpr int kq = decltype(kqc)::value;
    constexpr int kbyte = 2 * (32 * (kq >> 1) + 8 * (kq & 1));
#pragma unroll
    for (int h = 0; h < 2; h++) {
      bf16x8_t a[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint4 v = *reinterpret_cast<const uint4*>(sx + a_base + (16 * (4 * h + i)) * kXStride + kbyte);
        __builtin_memcpy(&a[i], &v, 16);
      }
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          acc[4 * h + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], bq[j], acc[4 * h + i][j], 0, 0, 0);
    }
  };

  // One super-step: the MFMAs of the four k-quarters with the dequantization of quarter kq+1
  // issued ahead of the MFMAs of quarter kq (the scheduler weaves the two streams).
  auto compute = [&](const uint4 (&raw)[4], int pair) {
    float d1[4], nm1[4], d2[4], nm2[4];
    fetch_scales(pair, d1, nm1, d2, nm2);
    bf16x8_t b0[4], b1[4];
    dequant_quarter(std::integral_constant<int, 0>{}, raw, d1, nm1, d2, nm2, b0);
    dequant_quarter(std::integral_constant<int, 1>{}, raw, d1, nm1, d2, nm2, b1);
    mfma_quarter(std::integral_constant<int, 0>{}, b0);
    dequant_quarter(std::integral_constant<int, 2>{}, raw, d1, nm1, d2, nm2, b0);
    mfma_quarter(std::integral_constant<int, 1>{}, b1);
    dequant_quarter(std::integral_constant<int, 3>{}, raw, d1, nm1, d2, nm2, b1);
    mfma_quarter(std::integral_constant<int, 2>{}, b0);
    mfma_quarter(std::integral_constant<int, 3>{}, b1);
  };

  // ---- prologue
  const int nblocks = n_in >> 8;
  uint4 wa[4], wb[4];
  hdr = load16_a16(wh);
  load_x(0);
  load_w(wa, 0);
  store_scales(hdr);
  store_x();
  __syncthreads();

  // ---- main loop: one super-block (two super-steps) per iteration, straight-line body.
  // Loads past the end are clamped to the last step / block (harmless re-reads).
  for (int b = 0; b < nblocks; b++) {
    const int st = 2 * b;
    // first half: chunks 0,1
    load_x(st + 1);
    load_w(wb, st + 1);
    hdr = load16_a16(wh + 144 * (int64_t)min(b + 1, nblocks - 1));
    // the scheduler must not sink these prefetches next to their use (it would, to shorten
    // live ranges, and expose one full memory latency per load)
    __builtin_amdgcn_sched_barrier(0);
    compute(wa, 0);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();                                   // everyone is done reading the X tile
    store_x();
    __syncthreads();
    // second half: chunks 2,3
    load_x(min(st + 2, nsteps - 1));
    load_w(wa, min(st + 2, nsteps - 1));
    __builtin_amdgcn_sched_barrier(0);
    compute(wb, 1);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    store_x();
    store_scales(hdr);                                 // next super-block's scales (wave-private)
    __syncthreads();
  }

  // ---- epilogue: lane holds Y[m0 + 16i + 4*lg + r][n0 + 16j + ln], r = 0..3
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int n = n0 + 16 * j + ln;
    if (n >= n_out) continue;
    const float bv = load_bias(bias, bias_dtype, n);
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int mm = m0 + 16 * i + 4 * lg + r;
        if (mm < m) YElem<YT>::store(y, (int64_t)mm * n_out + n, acc[i][j][r] + bv);
      }
    }
  }
}

}  // namespace v3

hipError_t launch_gemm_q4k_v3(const void* w, const uint16_t* x_bf16, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                              hipStream_t s) {
  using namespace v3;
  if (m == 0 || n_out == 0) return hipSuccess;
  const int n_tiles = (int)((n_out + BN - 1) / BN), m_tiles = (int)((m + BM - 1) / BM);
  const dim3 grid((unsigned)(n_tiles * m_tiles)), block(kThreads);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  if (y_dtype == kBF16)
    hipLaunchKernelGGL(gemm_q4k_v3_kernel<bf16_tag>, grid, block, 0, s, wb, x_bf16, static_cast<bf16_tag*>(y),
                       bias, bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles);
  else if (y_dtype == kF32)
    hipLaunchKernelGGL(gemm_q4k_v3_kernel<float>, grid, block, 0, s, wb, x_bf16, static_cast<float*>(y), bias,
                       bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ttq
