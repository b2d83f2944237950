// Decode GEMV for Q8_0 weights on gfx950 through the int8 matrix cores.
//
// Same operator as ttq_gemv.hip (F.linear with a single-token activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81).  Q8_0 weights ARE int8, so the 32 quants
// of a block go into v_mfma_i32_16x16x64_i8 as they come from memory: no unpacking at all.
// The activations of a block become block fixed point, split into signed byte planes
// (three for fp32 activations: v = rint(x * 2^(21-E)) = 65536*b2 + 256*b1 + b0, |v| <= 2^22,
// E the exponent of the block's largest |x|; two for 16-bit activations: 2^(13-E), as in the
// Q4_K kernel).  The per-plane sums are exact integers; they are recombined in fp32 (exact for
// two planes, within 2^-24 for three) and multiplied by the block's fp16 scale d.  A
// unit-vector activation reproduces d*q bit for bit.
//
// Shapes.  A step is four blocks (128 weights, 136 bytes) of 16 rows: two MFMAs.  The A operand
// has rows m = 4*b + t (block b of the step, plane t; row 4b+3 is zero), non-zero only where the
// MFMA's k-group belongs to block b, so C[4b+t][n] is the plane-t sum of block b for weight row
// n.  Lane (n = lane%16, g = lane/16) loads the 16 quants of k-group g for both MFMAs and the
// scale of block g, and receives C rows 4g..4g+3: all planes of block g of its own row.
// Work distribution as in ttq_gemv_mfma.hip: 16 wavefronts per CU, a wavefront owns 16 rows and
// one of SL interleaved slices of the steps, one step in flight per wavefront.
#include "ttq_gemv_mfma_common.h"

namespace ttq {

constexpr int64_t kMaxQ8In = 8192;     // plane table: 2 KiB of LDS per 128 activations

template <typename XT> struct Q8X;
template <> struct Q8X<float> {
  static constexpr int kPlanes = 3, kShift = 21;
  typedef float elem_t;
  static __device__ __forceinline__ void load8(const float* p, float (&f)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
};
template <> struct Q8X<bf16_tag> {
  static constexpr int kPlanes = 2, kShift = 13;
  typedef uint16_t elem_t;
  static __device__ __forceinline__ void load8(const uint16_t* p, float (&f)[8]) {
    widen8<bf16_tag>(*reinterpret_cast<const uint4*>(p), f);
  }
};
template <> struct Q8X<f16_tag> {
  static constexpr int kPlanes = 2, kShift = 13;
  typedef uint16_t elem_t;
  static __device__ __forceinline__ void load8(const uint16_t* p, float (&f)[8]) {
    widen8<f16_tag>(*reinterpret_cast<const uint4*>(p), f);
  }
};

// q0/q1: the 16 bytes from the 4-byte aligned address at or below the lane's quants, e0/e1 the
// dword after them (needed when the quants start 2 bytes into q0/q1)
struct Q8Step { uint4 q0, q1; uint32_t e0, e1, d; };

// LDS layout (bytes): plane table [nst][2 MFMAs][64 lanes] x 16 (entry (s, q, la): la = 16*ga + m,
// m = 4b + t; MFMA q covers blocks 2q and 2q+1 of the step, k-group ga the half ga%2 of block
// 2q + ga/2), then the per-block factors [nst][4] floats 2^(E - shift), then the partial row sums
// of the wavefronts [16][16] floats.
// R: steps a wavefront keeps in flight.
template <int R, typename XT, typename YT>
__global__ void __launch_bounds__(kMfmaThreads)
gemv_q8_mfma_kernel(const uint8_t* __restrict__ w, const typename Q8X<XT>::elem_t* __restrict__ x,
                    YT* __restrict__ y, const void* __restrict__ bias, int bias_dtype, int n_out, int nst,
                    int rows_per_wg, int sl_log2) {
  using X = Q8X<XT>;
  constexpr int W = kMfmaWaves, T = X::kPlanes;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  v4i_t* xa = reinterpret_cast<v4i_t*>(smem);
  float* tab = reinterpret_cast<float*>(smem + (size_t)nst * 2048);
  float* part = reinterpret_cast<float*>(smem + (size_t)nst * 2048 + (size_t)nst * 16);

  const int SL = 1 << sl_log2, G = W >> sl_log2;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int gi = wave >> sl_log2, sl = wave & (SL - 1);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nst * 128;
  const typename X::elem_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const uint32_t rb = (uint32_t)nst * 136u;
  const int S = (nst + SL - 1) >> sl_log2;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int rounds = (rows_per_wg + 16 * G - 1) / (16 * G);
  const int t_total = rounds * S;
  const int last = wg_row_end - 1;   // rows past the workgroup's share re-read its last row

  // ---- activations: 8 values per thread, requested before any weights
  const int k0 = 8 * tid;
  float xf[8];
  X::load8(xm + (k0 < n_in ? k0 : 0), xf);
  __builtin_amdgcn_s_barrier();

  // ---- weight stream: loads are unconditional (clamped); quant chunks are only 2-byte aligned
  Q8Step ring[R];
  int ir = 0, isi = 0;
  auto issue = [&](Q8Step& dst) {
    const int st = (isi << sl_log2) + sl;
    const bool ok = ir < rounds && st < nst;
    const int row = min(wg_row0 + (ir * G + gi) * 16 + n, last);
    const uint32_t o = ok ? (uint32_t)row * rb + (uint32_t)st * 136u : 0u;
    // a step's 136 bytes start 8-byte aligned; the quants of blocks 0 and 2 sit 2 bytes past a
    // dword boundary, those of blocks 1 and 3 on one
    const uint32_t oq = o + 34u * (uint32_t)(g >> 1) + 16u * (uint32_t)(g & 1) + (g >= 2 ? 2u : 0u);
    const uint32_t oe = oq + (g >= 2 ? 0u : 16u);
    dst.q0 = load16_a4(w + oq);
    dst.q1 = load16_a4(w + (oq + 68u));
    dst.e0 = load4_a4(w + oe);
    dst.e1 = load4_a4(w + (oe + 68u));
    dst.d = load2(w + (o + 34u * (uint32_t)g));
    if (++isi == S) { isi = 0; ir++; }
  };
#pragma unroll
  for (int i = 0; i < R; i++) issue(ring[i]);

  // ---- zero the plane-table entries that stay zero
  {
    const int la = tid & 63, q = (tid >> 6) & 1;
    const int m = la & 15, ga = la >> 4, b = m >> 2, t = m & 3;
    const bool nonzero = t < T && (b >> 1) == q && (b & 1) == (ga >> 1);
    if (!nonzero) {
      const v4i_t z = {0, 0, 0, 0};
      for (int s = tid >> 7; s < nst; s += kMfmaThreads / 128) xa[(s * 2 + q) * 64 + la] = z;
    }
  }

  // ---- quantize the activations into byte planes
  if (k0 < n_in) {
    uint32_t amax = amax_bits(xf);
    // the four threads of a block are an aligned quad
    amax = umax(amax, dpp_quad_u32<0xB1>(amax));
    amax = umax(amax, dpp_quad_u32<0x4E>(amax));
    const uint32_t eb = amax >> 23;                             // biased exponent of max |x|; 255 for Inf and NaN
    const uint32_t ec = eb < (uint32_t)(X::kShift + 1) ? (uint32_t)(X::kShift + 1) : eb;
    const float mul = __uint_as_float((254u + (uint32_t)X::kShift - ec) << 23);   // 2^(shift-E)
    // non-finite activations poison the block instead of being clipped
    const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - (uint32_t)X::kShift) << 23);
    int pl[3][8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int v = (int)rintf(xf[i] * mul);
      if (T == 3) {
        const int v1 = (v + 128) >> 8;
        pl[2][i] = v;                  // only the low byte is used
        pl[1][i] = v1;
        pl[0][i] = (v1 + 128) >> 8;
      } else {
        pl[1][i] = v;
        pl[0][i] = (v + 128) >> 8;
        pl[2][i] = 0;
      }
    }
    const int s = k0 >> 7, b = (k0 >> 5) & 3, h = (k0 >> 4) & 1, half8 = (k0 >> 3) & 1;
    const int q = b >> 1, ga = 2 * (b & 1) + h;
    uint2* xa8 = reinterpret_cast<uint2*>(smem);
    const int e0 = ((s * 2 + q) * 64 + 16 * ga + 4 * b) * 2 + half8;    // plane 0, in 8-byte units
#pragma unroll
    for (int t = 0; t < T; t++)
      xa8[e0 + 2 * t] = make_uint2(pack_low_bytes(pl[t][0], pl[t][1], pl[t][2], pl[t][3]),
                                   pack_low_bytes(pl[t][4], pl[t][5], pl[t][6], pl[t][7]));
    if ((tid & 3) == 0) tab[s * 4 + b] = f;
  }
  __syncthreads();

  // ---- main loop
  int cr = 0, csi = 0;
  float acc = 0.f;
  auto consume = [&](const Q8Step& s) {
    const int st = (csi << sl_log2) + sl;
    if (cr < rounds && st < nst) {
      const v4i_t* xe = xa + (size_t)st * 128 + lane;
      const v4i_t a0 = xe[0], a1 = xe[64];
      const float f = tab[st * 4 + g];
      v4i_t b0, b1;
      const uint32_t sh = g >= 2 ? 0u : 16u;
      b0[0] = (int)__builtin_amdgcn_alignbit(s.q0.y, s.q0.x, sh);
      b0[1] = (int)__builtin_amdgcn_alignbit(s.q0.z, s.q0.y, sh);
      b0[2] = (int)__builtin_amdgcn_alignbit(s.q0.w, s.q0.z, sh);
      b0[3] = (int)__builtin_amdgcn_alignbit(s.e0, s.q0.w, sh);
      b1[0] = (int)__builtin_amdgcn_alignbit(s.q1.y, s.q1.x, sh);
      b1[1] = (int)__builtin_amdgcn_alignbit(s.q1.z, s.q1.y, sh);
      b1[2] = (int)__builtin_amdgcn_alignbit(s.q1.w, s.q1.z, sh);
      b1[3] = (int)__builtin_amdgcn_alignbit(s.e1, s.q1.w, sh);
      const v4i_t zero = {0, 0, 0, 0};
      // the non-zero rows of the two products are disjoint (blocks 0-1 and 2-3)
      const v4i_t Ca = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, zero, 0, 0, 0);
      const v4i_t Cb = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, zero, 0, 0, 0);
      const v4i_t C = Ca + Cb;
      float sum;
      if (T == 3) sum = ((float)C[0] * 65536.f + (float)C[1] * 256.f) + (float)C[2];
      else sum = (float)(C[0] * 256 + C[1]);
      acc = acc + f16_bits_to_f32((uint16_t)s.d) * (sum * f);
    }
    if (++csi == S) {
      float v = acc;
      v = add_xor16(v);
      v = add_xor32(v);
      if (cr < rounds) {
        if (sl_log2 == 0) {
          const int row = wg_row0 + (cr * G + gi) * 16 + n;
          if (lane < 16 && row < wg_row_end) YElem<YT>::store(ym, row, v + load_bias(bias, bias_dtype, row));
        } else {
          if (lane < 16) part[wave * 16 + n] = v;
        }
      }
      acc = 0.f;
      csi = 0;
      cr++;
    }
  };
  // steady state: every consumed slot is re-requested R steps ahead (past the end: one harmless
  // line); the last R steps drain
  for (int t0 = R; t0 < t_total; t0 += R) {
#pragma unroll
    for (int i = 0; i < R; i++) {
      consume(ring[i]);
      issue(ring[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < R; i++) consume(ring[i]);

  if (sl_log2 != 0) {
    // one round only: add the slices in a fixed order
    __syncthreads();
    if (tid < 16 * G) {
      const int grp = tid >> 4, nn = tid & 15;
      float v = 0.f;
      for (int s2 = 0; s2 < SL; s2++) v += part[(grp * SL + s2) * 16 + nn];
      const int row = wg_row0 + grp * 16 + nn;
      if (row < wg_row_end) YElem<YT>::store(ym, row, v + load_bias(bias, bias_dtype, row));
    }
  }
}

template <typename XT, typename YT>
static hipError_t q8_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                               int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  constexpr int W = kMfmaWaves;
  const int nst = (int)(n_in / 128);
  int num_wg = device_num_cus();
  const int64_t groups = (n_out + 15) / 16;
  if (num_wg > groups) num_wg = (int)groups;
  const int rows_per_wg = (int)((n_out + num_wg - 1) / num_wg);
  num_wg = (int)((n_out + rows_per_wg - 1) / rows_per_wg);
  int sl_log2 = 0;
  while ((2 << sl_log2) <= W && (2 << sl_log2) <= nst && (16 * W >> (sl_log2 + 1)) >= rows_per_wg) sl_log2++;
  const size_t lds = (size_t)nst * 2048 + (size_t)nst * 16 + 1024;
  const auto launch = [&](auto kernel, LargeLds& configured) -> hipError_t {
    {
      const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)num_wg, (unsigned)m), dim3(W * 64), lds, s,
                       static_cast<const uint8_t*>(w), static_cast<const typename Q8X<XT>::elem_t*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, nst, rows_per_wg, sl_log2);
    return hipGetLastError();
  };
  // A workgroup with little to read (a few steps per wavefront) asks for two steps at once:
  // there is nothing to overlap the memory latency with otherwise.  With a long stream one step
  // per wavefront (35 KiB per CU in flight) is better.
  const int S = (nst + (1 << sl_log2) - 1) >> sl_log2;
  const int rounds = (rows_per_wg + (16 * W >> sl_log2) - 1) / (16 * W >> sl_log2);
  static const int forced = mfma_env_int("TTQ_GEMV_Q8_RING", 0);
  const bool two = forced ? forced == 2 : rounds * S <= 2;
  static LargeLds configured1, configured2;
  if (two) return launch(gemv_q8_mfma_kernel<2, XT, YT>, configured2);
  return launch(gemv_q8_mfma_kernel<1, XT, YT>, configured1);
}

template <typename XT>
static hipError_t q8_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                              int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q8_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return q8_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return q8_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

bool gemv_q8_mfma_supported(int format, int64_t n_out, int64_t n_in) {
  static const int disabled = mfma_env_int("TTQ_GEMV_NO_MFMA", 0);
  // byte offsets into the weight buffer are 32-bit in the kernel; with fewer than eight rows per
  // CU the per-workgroup activation set-up outweighs the saving
  return !disabled && format == kQ8_0 && n_out >= 2048 && n_in % 128 == 0 && n_in <= kMaxQ8In &&
         n_out * (n_in / 32) * 34 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_q8_mfma(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                               int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kF32) return q8_launch_x<float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kBF16) return q8_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return q8_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
