// Q4_K linear layer for a handful of activation rows (up to 64): the regime between the decode
// GEMV and the prefill GEMM (batched decoding, speculative verification, short prompts).
//
// Same operator as ttq_gemm_q4k.hip (F.linear with seq_len > 1,
// workspace/libtorch/src/abi/neural_nets.nim:64-81, reached from
// workspace/transformers/src/layers/linear.nim:45-57).  With so few rows the weights are read
// once and every byte of them is used by one wavefront only, so nothing of W goes through LDS:
//
//   * a workgroup of 8 wavefronts owns 16, 32 or 64 weight rows (output columns; the most that still
//     gives every CU a workgroup); wavefront v owns the super-blocks v, v+8, ... of those rows (a
//     split along K inside the workgroup);
//   * one step of v_mfma_f32_16x16x32_bf16 is one sub-block (32 k): lane (i = lane % 16, g = lane / 16)
//     supplies k = 32*step + 8*g + {0..7}, for weight row 16*rb + i as the A operand and for
//     activation row ("token") 16*tb + i as the B operand.  For the activations that is one
//     16-byte load per step, and the four lanes of a token read 64 consecutive bytes, so a load
//     instruction touches 16 cache lines (what such loads cost is lines looked up, not bytes);
//     the 128 bytes per token block stay in registers for all row blocks of the workgroup;
//   * for the weights it is the 8 bytes 8*g .. 8*g+7 of each of the four 32-byte qs chunks: low
//     nibbles for the even sub-block of the chunk, high nibbles for the odd one, dequantized in
//     registers (canonical arithmetic, one bf16 rounding);
//   * each lane decodes the scale and min of two sub-blocks (2g, 2g+1) of its row and the four
//     lanes of a row exchange them through v_mfma_f32_16x16x4_f32 with a 0/1 selector as the other
//     operand (D[4g'+r][row] = value of lane g = r: an exact all-gather);
//   * the eight wavefronts' partial sums meet in LDS once, at the end; the sums are transposed
//     through LDS so that every thread stores 8 consecutive outputs of one token.
//
// Algorithmic bytes: the packed weights once (n_out * n_in * 0.5625) plus m * n_out outputs; the
// activations (m * n_in * 2 per workgroup) come from L2.  The kernel is bound by the
// dequantization (about 3 vector instructions per weight), not by HBM or the matrix cores.
#include <type_traits>

#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {
namespace {

constexpr int kSkThreads = 512;
constexpr int kSkWaves = kSkThreads / 64;

struct SkRaw { uint4 hdr; uint2 q[4]; };

// RB: blocks of 16 weight rows per workgroup; TB: blocks of 16 tokens (m <= 16 * TB); WD: ring of
// (super-block, row block) items of packed weights per wavefront, WD - 1 of them in flight; XB:
// buffers for a super-block's activations (2: the next super-block's are requested while this one
// is multiplied).
template <int RB, int TB, int WD, int XB>
__global__ void __launch_bounds__(kSkThreads)
gemm_q4k_skinny_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, void* __restrict__ yv,
                       int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in) {
  static_assert((WD == 2 || WD == 4) && (2 * RB) % WD == 0 && (XB == 1 || XB == 2), "ring sizes");
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, kg = lane >> 4;
  const int nsb = n_in >> 8;
  const int n0 = blockIdx.x * (16 * RB);

  // byte offset of (row, super-block 0) and element offset of (token, k = 8*kg)
  uint32_t wofs[RB], xofs[TB];
#pragma unroll
  for (int rb = 0; rb < RB; rb++) wofs[rb] = (uint32_t)min(n0 + 16 * rb + li, n_out - 1) * (uint32_t)(nsb * 144);
#pragma unroll
  for (int tb = 0; tb < TB; tb++) xofs[tb] = (uint32_t)min(16 * tb + li, m - 1) * (uint32_t)n_in + 8u * kg;

  f32x4_t acc[RB][TB];
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int tb = 0; tb < TB; tb++) acc[rb][tb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // selector of the all-gather: as the A operand of the 16x16x4 MFMA (row i = lane % 16, k = lane / 16)
  const float gather_sel = ((li & 3) == kg) ? 1.f : 0.f;
  // Bit positions of the 6-bit scale and min of sub-blocks 2kg and 2kg+1 in the 12 packed bytes:
  // sub-blocks 0..3 have the field whole in bytes 0..7, sub-blocks 4..7 four bits in bytes 8..11 and
  // two on top of bytes 0..7.  Two bit-field extracts each, the second of width 0 in the simple case.
  const bool upper = kg >= 2;
  const uint32_t wl = upper ? 4u : 6u, wh = upper ? 2u : 0u;
  uint32_t sh_sc[2], sh_mn[2], sh_hi[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const uint32_t jj = (2u * kg + h) & 3u;
    sh_sc[h] = 8u * jj;
    sh_mn[h] = upper ? 8u * jj + 4u : 8u * jj;
    sh_hi[h] = 8u * jj + 6u;
  }

  auto fetch = [&](SkRaw& r, int sb, int rb) {
    const uint8_t* p = w + wofs[rb] + (uint32_t)sb * 144u;
    r.hdr = load16_a16(p);
#pragma unroll
    for (int c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const uint2*>(p + 16 + 32 * c + 8 * kg);
  };
  // a super-block's activations: piece i is k = 32*i + 8*kg .. +7 of the lane's token
  auto load_x = [&](uint4 (&xf)[TB][8], int sb) {
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
      for (int i = 0; i < 8; i++)
        xf[tb][i] = *reinterpret_cast<const uint4*>(x + xofs[tb] + 256u * (uint32_t)sb + 32u * i);
  };

  SkRaw raw[WD];
  uint4 xfr[XB][TB][8];

  // The wavefront's items in order: (super-block, row block), row blocks innermost.  Item rb of a
  // super-block of parity XI lives in raw[(XI * RB + rb) % WD]; while it is multiplied, the item
  // WD - 1 places further on is requested.  Requests past the end re-read this super-block (lines
  // already in cache) so that the load counting stays exact.
  auto super_block = [&](auto xi_c, int sb) {
    constexpr int XI = decltype(xi_c)::value;
    constexpr int kAhead = WD - 1;
    const int sb_next = sb + kSkWaves < nsb ? sb + kSkWaves : sb;
    if (XB == 1) load_x(xfr[0], sb);
    else load_x(xfr[XI ^ 1], sb_next);
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
      {
        constexpr int kMaxOff = (RB - 1 + kAhead) / RB;
        const int off = (rb + kAhead) / RB;
        int sb_a = sb + off * kSkWaves;
        if (kMaxOff > 1 || off > 0) sb_a = sb_a < nsb ? sb_a : sb;
        fetch(raw[(XI * RB + rb + kAhead) % WD], sb_a, (rb + kAhead) % RB);
      }
      const SkRaw& r = raw[(XI * RB + rb) % WD];
      // this lane: sub-blocks 2kg and 2kg+1 of its row; then all eight from the row's four lanes
      const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
      const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
      const uint32_t a_sc = upper ? r.hdr.w : r.hdr.y;   // bytes 8-11 or 0-3
      const uint32_t a_mn = upper ? r.hdr.w : r.hdr.z;   // bytes 8-11 or 4-7
      const uint32_t sc1 = __builtin_amdgcn_ubfe(a_sc, sh_sc[0], wl) | (__builtin_amdgcn_ubfe(r.hdr.y, sh_hi[0], wh) << 4);
      const uint32_t sc2 = __builtin_amdgcn_ubfe(a_sc, sh_sc[1], wl) | (__builtin_amdgcn_ubfe(r.hdr.y, sh_hi[1], wh) << 4);
      const uint32_t mn1 = __builtin_amdgcn_ubfe(a_mn, sh_mn[0], wl) | (__builtin_amdgcn_ubfe(r.hdr.z, sh_hi[0], wh) << 4);
      const uint32_t mn2 = __builtin_amdgcn_ubfe(a_mn, sh_mn[1], wl) | (__builtin_amdgcn_ubfe(r.hdr.z, sh_hi[1], wh) << 4);
      const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
      const f32x4_t de = __builtin_amdgcn_mfma_f32_16x16x4f32(gather_sel, d * (float)sc1, zero, 0, 0, 0);
      const f32x4_t dd = __builtin_amdgcn_mfma_f32_16x16x4f32(gather_sel, d * (float)sc2, zero, 0, 0, 0);
      const f32x4_t me = __builtin_amdgcn_mfma_f32_16x16x4f32(gather_sel, -(dmin * (float)mn1), zero, 0, 0, 0);
      const f32x4_t md = __builtin_amdgcn_mfma_f32_16x16x4f32(gather_sel, -(dmin * (float)mn2), zero, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int c = i >> 1;
        const float ds = (i & 1) ? dd[c] : de[c], nm = (i & 1) ? md[c] : me[c];
        uint32_t q0 = ((i & 1) ? (r.q[c].x >> 4) : r.q[c].x) & 0x0F0F0F0Fu;
        uint32_t q1 = ((i & 1) ? (r.q[c].y >> 4) : r.q[c].y) & 0x0F0F0F0Fu;
        // keep the masked words opaque: byte k of them converts with one v_cvt_f32_ubyte<k>
        asm volatile("" : "+v"(q0), "+v"(q1));
        float f[8];
#pragma unroll
        for (int k = 0; k < 4; k++) {
          // fused multiply-add == the canonical two-step form: d is an f16, sc has 6 bits and q 4,
          // so the product is exact in fp32
          f[k] = fmaf_(ds, (float)((q0 >> (8 * k)) & 0xFFu), nm);
          f[4 + k] = fmaf_(ds, (float)((q1 >> (8 * k)) & 0xFFu), nm);
        }
        const uint32_t au[4] = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]),
                                pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        bf16x8_t a;
        __builtin_memcpy(&a, au, 16);
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
          bf16x8_t b;
          __builtin_memcpy(&b, &xfr[XB == 1 ? 0 : XI][tb][i], 16);
          acc[rb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[rb][tb], 0, 0, 0);
        }
      }
    }
  };

  if (wave < nsb) {
#pragma unroll
    for (int q = 0; q < WD - 1; q++) {
      const int sb_q = wave + (q / RB) * kSkWaves;
      fetch(raw[q % WD], sb_q < nsb ? sb_q : wave, q % RB);
    }
    if (XB == 2) load_x(xfr[0], wave);
  }
  for (int sb = wave; sb < nsb; sb += 2 * kSkWaves) {
    super_block(std::integral_constant<int, 0>{}, sb);
    if (sb + kSkWaves < nsb) super_block(std::integral_constant<int, 1>{}, sb + kSkWaves);
  }

  // The wavefronts' partial sums: part[wave][rb][tb][r][lane]; element (rb, tb, r, lane) is weight
  // row 16*rb + 4*(lane/16) + r and token 16*tb + lane%16.
  constexpr int kElems = RB * TB * 4 * 64;
  constexpr int kTileLd = 16 * RB + 1;
  float* part = smem;
  float* tile = smem + kSkWaves * kElems;          // [token][16 * RB + 1]: sums, transposed
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
      for (int r = 0; r < 4; r++) part[wave * kElems + ((rb * TB + tb) * 4 + r) * 64 + lane] = acc[rb][tb][r];
  __syncthreads();
  for (int e = tid; e < kElems; e += kSkThreads) {
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < kSkWaves; v++) s += part[v * kElems + e];
    const int l = e & 63, r = (e >> 6) & 3, q = e >> 8;      // q = rb * TB + tb
    const int rb = q / TB, tb = q - rb * TB;
    const int row = 16 * rb + 4 * (l >> 4) + r, tok = 16 * tb + (l & 15);
    tile[tok * kTileLd + row] = s;
  }
  __syncthreads();
  // 8 consecutive outputs of one token per thread
  for (int t = tid; t < 16 * TB * 2 * RB; t += kSkThreads) {
    const int tok = t / (2 * RB), g = t % (2 * RB);
    const int col = n0 + 8 * g;
    if (tok >= m || col >= n_out) continue;      // n_out is a multiple of 8: a group is all in or all out
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = tile[tok * kTileLd + 8 * g + k] + load_bias(bias, bias_dtype, col + k);
    const int64_t o = (int64_t)tok * n_out + col;
    if (y_dtype == kBF16) {
      *reinterpret_cast<uint4*>(static_cast<uint16_t*>(yv) + o) =
          make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
    } else {
      float4* yo = reinterpret_cast<float4*>(static_cast<float*>(yv) + o);
      yo[0] = make_float4(v[0], v[1], v[2], v[3]);
      yo[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
  }
}

template <int RB, int TB, int WD, int XB>
hipError_t launch_skinny_tb(const uint8_t* w, const uint16_t* x, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  auto kernel = gemm_q4k_skinny_kernel<RB, TB, WD, XB>;
  const size_t lds = (size_t)(kSkWaves * RB * TB * 4 * 64 + 16 * TB * (16 * RB + 1)) * sizeof(float);
  static LargeLds configured;
  if (lds > 64 * 1024) {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
    if (e != hipSuccess) return e;
  }
  const dim3 grid((unsigned)((n_out + 16 * RB - 1) / (16 * RB))), block(kSkThreads);
  hipLaunchKernelGGL(kernel, grid, block, lds, s, w, x, y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in);
  return hipGetLastError();
}

}  // namespace

bool gemm_skinny_supported(int format, int64_t m, int64_t n_out, int64_t n_in) {
  static const int disabled = [] { const char* e = getenv("TTQ_GEMM_NO_SKINNY"); return e ? atoi(e) : 0; }();
  // weight byte offsets and activation element offsets are 32-bit in the kernel; outputs are stored
  // eight at a time
  return !disabled && format == kQ4_K && m >= 1 && m <= 64 && n_out > 0 && n_out % 8 == 0 && n_in > 0 &&
         n_in % 256 == 0 && n_out * (n_in / 256) * 144 < ((int64_t)1 << 32) && m * n_in < ((int64_t)1 << 31);
}

// Cost model (microseconds), fitted to 4096 x 4096, 4096 x 14336 and 14336 x 4096: rounds of workgroups
// over the CUs x (fixed + super-blocks per wavefront x (activation loads + row blocks x weights)).
// The activations of a super-block are re-read from L2 by every workgroup, which is what makes
// more rows per workgroup cheaper per row, as long as every CU still gets a workgroup.
static float skinny_cost_us(int rb, int64_t m, int64_t n_out, int64_t n_in) {
  static const float kX[4] = {1.46f, 2.73f, 4.9f, 6.25f}, kW[4] = {1.13f, 1.14f, 1.28f, 1.6f};
  static const float kF0[4] = {4.5f, 7.8f, 4.2f, 4.7f}, kF1[4] = {1.0f, 0.6f, 0.f, 0.f};
  const int t = (int)((m + 15) / 16) - 1;
  const int64_t wgs = (n_out + 16 * rb - 1) / (16 * rb), cus = device_num_cus();
  const int64_t iters = ((n_in >> 8) + kSkWaves - 1) / kSkWaves;
  return (float)((wgs + cus - 1) / cus) * (kF0[t] + kF1[t] * rb + (float)iters * (kX[t] + rb * kW[t]));
}

static int skinny_choose_rb(int64_t m, int64_t n_out, int64_t n_in, float* cost_us = nullptr) {
  static const int forced_rb = [] { const char* e = getenv("TTQ_SK_RB"); return e ? atoi(e) : 0; }();
  int best = 4;
  float best_cost = 1e30f;
  for (int rb = 4; rb >= 1; rb >>= 1) {
    if (forced_rb > 0 && rb != forced_rb) continue;
    const float c = skinny_cost_us(rb, m, n_out, n_in);
    if (c < best_cost) { best_cost = c; best = rb; }
  }
  if (cost_us) *cost_us = best_cost;
  return best;
}

float gemm_skinny_estimate_us(int64_t m, int64_t n_out, int64_t n_in) {
  float c = 0.f;
  skinny_choose_rb(m, n_out, n_in, &c);
  return c;
}

hipError_t launch_gemm_skinny(const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                              int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (y_dtype != kBF16 && y_dtype != kF32) return hipErrorInvalidValue;
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  // Registers decide how far ahead a wavefront can request: 64 per token block for the activations.
  const int rb = skinny_choose_rb(m, n_out, n_in);
  const int tb = (int)((m + 15) / 16);
#define TTQ_SK_CASE(RBv, TBv, WDv, XBv) \
  if (rb == RBv && tb == TBv)            \
    return launch_skinny_tb<RBv, TBv, WDv, XBv>(wb, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  TTQ_SK_CASE(4, 1, 4, 2) TTQ_SK_CASE(4, 2, 4, 2) TTQ_SK_CASE(4, 3, 2, 1) TTQ_SK_CASE(4, 4, 2, 1)
  TTQ_SK_CASE(2, 1, 4, 2) TTQ_SK_CASE(2, 2, 4, 2) TTQ_SK_CASE(2, 3, 2, 1) TTQ_SK_CASE(2, 4, 2, 1)
  TTQ_SK_CASE(1, 1, 2, 2) TTQ_SK_CASE(1, 2, 2, 2) TTQ_SK_CASE(1, 3, 2, 1) TTQ_SK_CASE(1, 4, 2, 1)
#undef TTQ_SK_CASE
  return hipErrorInvalidValue;
}

}  // namespace ttq
