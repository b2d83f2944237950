// Decode GEMV for the block formats Q8_0 / Q4_K / Q6_K on gfx950.
//
//   y[n] = sum_k W^[n][k] * x[k] (+ bias[n])        W^ = dequantized weight, never stored
//
// replaces F.linear(x, weight) for a single-token activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81, called from
//  workspace/transformers/src/layers/linear.nim:45-57).
//
// Mapping.  A row of W is cut into "units" of 64 weights; unit u of every row is always
// handled by lane u % 64, so the 64 activations a lane needs never change from row to row.
// A workgroup first stages x in LDS in a lane-major permutation; when a row has at most 64
// units (n_in <= 4096) each lane then pulls its 64 activations into VGPRs once and the row
// loop touches only HBM: per row a wavefront issues 16-byte loads that cover the packed row
// contiguously, unpacks in registers, and finishes with a cross-lane sum.  Rows are dealt
// to wavefronts round-robin, so at any moment the whole chip streams one contiguous span
// of the weight buffer.
//
// Two arithmetic paths:
//   generic : x widened to fp32, fp32 FMA per weight.  Any activation dtype.
//   dot2    : bf16 activations kept as packed pairs, weights turned into bf16 pairs with
//             one AND-OR each (0x4300 | q is the bf16 value 128 + q) and multiplied with
//             v_dot2_f32_bf16; the 128 offset is removed with a per-unit sum of x.
// Both compute sum(q*x) per sub-block first and apply the block scales once per sub-block,
// so for a unit-vector activation the result equals the canonical dequantized weight bit
// for bit.
#include "ttq_device.h"
#include "ttq_internal.h"

#include <stdlib.h>

namespace ttq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;

// LDS slot of activation p (0..63) of unit u, fp32 layout: [u/64][p/4][u%64][p%4]
__device__ __forceinline__ int xslot_f32(int u, int p) {
  return ((((u >> 6) * 16 + (p >> 2)) * 64 + (u & 63)) << 2) + (p & 3);
}

// ------------------------------------------------------------------------------- formats
struct FmtQ8_0 {
  // unit = two consecutive 34-byte blocks (64 weights); the second may be absent at row end
  static __device__ __forceinline__ int units(int n_in) { return (n_in + 63) >> 6; }
  static __device__ __forceinline__ int64_t row_bytes(int n_in) { return (int64_t)(n_in >> 5) * 34; }
  static __device__ __forceinline__ void kmap(int k, int& u, int& p) { u = k >> 6; p = k & 63; }
  // first k of activation slots 16 q .. 16 q + 15 of unit u (consecutive k)
  static __device__ __forceinline__ int64_t kbase(int u, int q) { return 64 * (int64_t)u + 16 * q; }
  struct Raw { uint4 a0, a1, b0, b1; uint32_t d0, d1; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u, int n_in) {
    Raw r;
    const uint8_t* p = row + 68 * (int64_t)u;
    r.d0 = load2(p);
    r.a0 = load16_a2(p + 2);
    r.a1 = load16_a2(p + 18);
    const bool second = (64 * u + 32) < n_in;
    if (second) {
      r.d1 = load2(p + 34);
      r.b0 = load16_a4(p + 36);
      r.b1 = load16_a4(p + 52);
    } else {
      r.d1 = 0;
      r.b0 = make_uint4(0, 0, 0, 0);
      r.b1 = r.b0;
    }
    return r;
  }
  static __device__ __forceinline__ float dot32(const uint4& q0, const uint4& q1, const float* x) {
    const uint32_t dw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int q = (int)(int8_t)((dw[i] >> (8 * k)) & 0xFFu);
        s = fmaf_((float)q, x[4 * i + k], s);
      }
    }
    return s;
  }
  static __device__ __forceinline__ float dot(const Raw& r, const float (&x)[64]) {
    const float s0 = dot32(r.a0, r.a1, &x[0]);
    const float s1 = dot32(r.b0, r.b1, &x[32]);
    const float d0 = f16_bits_to_f32((uint16_t)r.d0), d1 = f16_bits_to_f32((uint16_t)r.d1);
    return d0 * s0 + d1 * s1;
  }
};

struct FmtQ4_K {
  // unit = chunk c of a super-block: 32 qs bytes -> sub-blocks 2c (low nibbles), 2c+1 (high)
  static __device__ __forceinline__ int units(int n_in) { return n_in >> 6; }
  static __device__ __forceinline__ int64_t row_bytes(int n_in) { return (int64_t)(n_in >> 8) * 144; }
  static __device__ __forceinline__ void kmap(int k, int& u, int& p) { u = k >> 6; p = k & 63; }
  static __device__ __forceinline__ int64_t kbase(int u, int q) { return 64 * (int64_t)u + 16 * q; }
  struct Raw { uint4 hdr, q0, q1; int c; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u, int) {
    Raw r;
    const uint8_t* p = row + 144 * (int64_t)(u >> 2);
    r.c = u & 3;
    r.hdr = load16_a16(p);
    r.q0 = load16_a16(p + 16 + 32 * r.c);
    r.q1 = load16_a16(p + 32 + 32 * r.c);
    return r;
  }
  static __device__ __forceinline__ float dot(const Raw& r, const float (&x)[64]) {
    const uint32_t dw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
    float s1 = 0.f, s2 = 0.f, x1 = 0.f, x2 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const uint32_t b = (dw[i] >> (8 * k)) & 0xFFu;
        s1 = fmaf_((float)(b & 0xFu), x[4 * i + k], s1);
        s2 = fmaf_((float)(b >> 4), x[32 + 4 * i + k], s2);
        x1 += x[4 * i + k];
        x2 += x[32 + 4 * i + k];
      }
    }
    const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    uint32_t sc1, mn1, sc2, mn2;
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * r.c, sc1, mn1);
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * r.c + 1, sc2, mn2);
    const float t1 = (d * (float)sc1) * s1 - (dmin * (float)mn1) * x1;
    const float t2 = (d * (float)sc2) * s2 - (dmin * (float)mn2) * x2;
    return t1 + t2;
  }
};

struct FmtQ6_K {
  // unit = (block b, half h, 16-wide l range s): weights 128h + 32j + 16s + i, j=0..3, i=0..15
  // unit index u = 4b + 2h + s; activation slot p = 16j + i
  static __device__ __forceinline__ int units(int n_in) { return n_in >> 6; }
  static __device__ __forceinline__ int64_t row_bytes(int n_in) { return (int64_t)(n_in >> 8) * 210; }
  static __device__ __forceinline__ void kmap(int k, int& u, int& p) {
    const int b = k >> 8, r = k & 255;
    const int h = r >> 7, rr = r & 127;
    const int j = rr >> 5, l = rr & 31;
    u = 4 * b + 2 * h + (l >> 4);
    p = 16 * j + (l & 15);
  }
  // slots 16 j .. 16 j + 15 of unit 4 b + 2 h + s: k = 256 b + 128 h + 32 j + 16 s + i
  static __device__ __forceinline__ int64_t kbase(int u, int q) {
    return 256 * (int64_t)(u >> 2) + 128 * ((u >> 1) & 1) + 32 * q + 16 * (u & 1);
  }
  struct Raw { uint4 a, b, h; uint32_t sc0, sc1; uint32_t d; int s; };
  static __device__ __forceinline__ Raw load(const uint8_t* row, int u, int) {
    Raw r;
    const uint8_t* p = row + 210 * (int64_t)(u >> 2);
    const int h = (u >> 1) & 1;
    r.s = u & 1;
    r.a = load16_a2(p + 64 * h + 16 * r.s);
    r.b = load16_a2(p + 64 * h + 32 + 16 * r.s);
    r.h = load16_a2(p + 128 + 32 * h + 16 * r.s);
    r.sc0 = load4_a2(p + 192 + 8 * h);
    r.sc1 = load4_a2(p + 196 + 8 * h);
    r.d = load2(p + 208);
    return r;
  }
  static __device__ __forceinline__ float dot(const Raw& r, const float (&x)[64]) {
    const uint32_t A[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
    const uint32_t B[4] = {r.b.x, r.b.y, r.b.z, r.b.w};
    const uint32_t H[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const uint32_t a = (A[i] >> (8 * k)) & 0xFFu, b = (B[i] >> (8 * k)) & 0xFFu;
        const uint32_t h = (H[i] >> (8 * k)) & 0xFFu;
        const int q1 = (int)((a & 0xF) | (((h >> 0) & 3) << 4)) - 32;
        const int q2 = (int)((b & 0xF) | (((h >> 2) & 3) << 4)) - 32;
        const int q3 = (int)((a >> 4) | (((h >> 4) & 3) << 4)) - 32;
        const int q4 = (int)((b >> 4) | (((h >> 6) & 3) << 4)) - 32;
        const int l = 4 * i + k;
        s[0] = fmaf_((float)q1, x[l], s[0]);
        s[1] = fmaf_((float)q2, x[16 + l], s[1]);
        s[2] = fmaf_((float)q3, x[32 + l], s[2]);
        s[3] = fmaf_((float)q4, x[48 + l], s[3]);
      }
    }
    const float d = f16_bits_to_f32((uint16_t)r.d);
    // scale bytes of this half: index s + 2j
    const uint32_t lo = r.sc0 >> (8 * r.s), hi = r.sc1 >> (8 * r.s);
    const float c0 = (float)(int8_t)(lo & 0xFF), c1 = (float)(int8_t)((lo >> 16) & 0xFF);
    const float c2 = (float)(int8_t)(hi & 0xFF), c3 = (float)(int8_t)((hi >> 16) & 0xFF);
    return ((d * c0) * s[0] + (d * c1) * s[1]) + ((d * c2) * s[2] + (d * c3) * s[3]);
  }
};

// ------------------------------------------------------------------------- generic kernel
// XREG: a row has at most 64 units, so each lane keeps its activations in registers.
template <class F, typename XT, typename YT, bool XREG>
__global__ void __launch_bounds__(kGemvThreads)
gemv_generic_kernel(const uint8_t* __restrict__ w, const XT* __restrict__ x, YT* __restrict__ y,
                    const void* __restrict__ bias, int bias_dtype, int n_out, int n_in) {
  extern __shared__ float xs[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const XT* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const int units = F::units(n_in);
  const int nit = (units + 63) >> 6;

  // Rows in whole groups of 16 bytes (they then start 16-byte aligned): one load per group.  (Element by element
  // this staging was most of the kernel on small matrices: Q8_0 512x4096 5.8 us, 3.6 with whole groups.)
  constexpr int kVec = 16 / (int)sizeof(XT);
  if (n_in % kVec == 0) {
    for (int k = kVec * tid; k < nit * 4096; k += kVec * kGemvThreads) {
      XT raw[kVec];
      float v[kVec];
      if (k < n_in) {
        const uint4 q = *reinterpret_cast<const uint4*>(__builtin_assume_aligned(xm + k, 16));
        __builtin_memcpy(raw, &q, 16);
#pragma unroll
        for (int i = 0; i < kVec; i++) v[i] = XElem<XT>::load(raw, i);
      } else {
#pragma unroll
        for (int i = 0; i < kVec; i++) v[i] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < kVec; i++) {
        int u, p;
        F::kmap(k + i, u, p);
        xs[xslot_f32(u, p)] = v[i];
      }
    }
  } else {
    for (int k = tid; k < nit * 4096; k += kGemvThreads) {
      const float v = (k < n_in) ? XElem<XT>::load(xm, k) : 0.f;
      int u, p;
      F::kmap(k, u, p);
      xs[xslot_f32(u, p)] = v;
    }
  }
  __syncthreads();

  const int64_t rb = F::row_bytes(n_in);
  const int first = blockIdx.x * kGemvWaves + wave;
  const int stride = gridDim.x * kGemvWaves;
  const float4* xs4 = reinterpret_cast<const float4*>(xs);

  if constexpr (XREG) {
    float xr[64];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float4 v = xs4[r * 64 + lane];
      xr[4 * r] = v.x; xr[4 * r + 1] = v.y; xr[4 * r + 2] = v.z; xr[4 * r + 3] = v.w;
    }
    const bool active = lane < units;
    int row = first;
    // two rows per trip keeps more loads in flight
    for (; row + stride < n_out; row += 2 * stride) {
      float a0 = 0.f, a1 = 0.f;
      if (active) {
        const typename F::Raw r0 = F::load(w + rb * row, lane, n_in);
        const typename F::Raw r1 = F::load(w + rb * (row + stride), lane, n_in);
        a0 = F::dot(r0, xr);
        a1 = F::dot(r1, xr);
      }
      a0 = wave_sum(a0);
      a1 = wave_sum(a1);
      if (lane == 0) {
        YElem<YT>::store(ym, row, a0 + load_bias(bias, bias_dtype, row));
        YElem<YT>::store(ym, row + stride, a1 + load_bias(bias, bias_dtype, row + stride));
      }
    }
    for (; row < n_out; row += stride) {
      float a0 = 0.f;
      if (active) a0 = F::dot(F::load(w + rb * row, lane, n_in), xr);
      a0 = wave_sum(a0);
      if (lane == 0) YElem<YT>::store(ym, row, a0 + load_bias(bias, bias_dtype, row));
    }
  } else {
    for (int row = first; row < n_out; row += stride) {
      float acc = 0.f;
      for (int it = 0; it < nit; it++) {
        const int u = it * 64 + lane;
        if (u < units) {
          const typename F::Raw r = F::load(w + rb * row, u, n_in);
          float xr[64];
#pragma unroll
          for (int q = 0; q < 16; q++) {
            const float4 v = xs4[(it * 16 + q) * 64 + lane];
            xr[4 * q] = v.x; xr[4 * q + 1] = v.y; xr[4 * q + 2] = v.z; xr[4 * q + 3] = v.w;
          }
          acc += F::dot(r, xr);
        }
      }
      acc = wave_sum(acc);
      if (lane == 0) YElem<YT>::store(ym, row, acc + load_bias(bias, bias_dtype, row));
    }
  }
}

// Launch geometry: enough workgroups to give every SIMD several wavefronts, never more
// wavefronts than rows.  TTQ_GEMV_WG_PER_CU overrides the per-CU workgroup count.
static int gemv_grid(int64_t n_out, int default_per_cu) {
  static int per_cu_env = -1;
  if (per_cu_env < 0) {
    per_cu_env = dev_knob("TTQ_GEMV_WG_PER_CU", 0);
  }
  const int per_cu = per_cu_env > 0 ? per_cu_env : default_per_cu;
  const int cus = device_num_cus();
  int64_t g = (int64_t)cus * per_cu;
  const int64_t need = (n_out + kGemvWaves - 1) / kGemvWaves;
  if (g > need) g = need;
  if (g < 1) g = 1;
  return (int)g;
}

template <class F, typename XT, typename YT>
static hipError_t launch_generic(const void* w, const void* x, void* y, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                 hipStream_t s) {
  const int units = (int)((n_in + 63) / 64);
  const int nit = (units + 63) / 64;
  const size_t lds = (size_t)nit * 4096 * sizeof(float);
  const dim3 grid(gemv_grid(n_out, 4), (unsigned)m), block(kGemvThreads);
  if (nit == 1) {
    hipLaunchKernelGGL((gemv_generic_kernel<F, XT, YT, true>), grid, block, lds, s,
                       static_cast<const uint8_t*>(w), static_cast<const XT*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)n_in);
  } else {
    hipLaunchKernelGGL((gemv_generic_kernel<F, XT, YT, false>), grid, block, lds, s,
                       static_cast<const uint8_t*>(w), static_cast<const XT*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)n_in);
  }
  return hipGetLastError();
}

template <class F, typename XT>
static hipError_t launch_generic_y(const void* w, const void* x, void* y, int y_dtype,
                                   const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                                   int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return launch_generic<F, XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_generic<F, XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_generic<F, XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

template <class F>
static hipError_t launch_generic_xy(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                    const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                                    int64_t n_in, hipStream_t s) {
  switch (x_dtype) {
    case kF32: return launch_generic_y<F, float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_generic_y<F, f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_generic_y<F, bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

// ---------------------------------------------------------------------- rows of any length
// Rows longer than the staged kernels hold in LDS (F.linear has no such limit: the down projection of the
// largest dense models has 53248 inputs).  Nothing is staged: a workgroup owns kLongRows consecutive weight rows,
// its 256 threads walk the rows' units 256 apart, and every thread reads the 64 activations of its unit straight
// from memory in four runs of 16 consecutive values, once for all of the rows (the activation row stays in L2, the
// weights are read once); the wavefronts' sums meet in LDS.  (A wavefront per group of rows left most compute
// units idle on matrices of a few thousand rows: Q8_0 3584 x 18944 48 us.)  Same arithmetic as the generic kernel
// (fp32, scales applied once per sub-block).
constexpr int kLongRows = 8;

template <class F, typename XT, typename YT>
__global__ void __launch_bounds__(kGemvThreads)
gemv_long_kernel(const uint8_t* __restrict__ w, const XT* __restrict__ x, YT* __restrict__ y,
                 const void* __restrict__ bias, int bias_dtype, int n_out, int n_in) {
  __shared__ float part[kGemvWaves][kLongRows];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const XT* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const int units = F::units(n_in);
  const int64_t rb = F::row_bytes(n_in);
  constexpr int kVec = 16 / (int)sizeof(XT);           // activations per 16-byte load
  const int groups = (n_out + kLongRows - 1) / kLongRows;
  for (int g = blockIdx.x; g < groups; g += gridDim.x) {
    const int row0 = g * kLongRows;
    float acc[kLongRows];
#pragma unroll
    for (int r = 0; r < kLongRows; r++) acc[r] = 0.f;
    for (int u = tid; u < units; u += kGemvThreads) {
      float xr[64];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int64_t k0 = F::kbase(u, q);
        if (k0 + 16 <= n_in) {
#pragma unroll
          for (int v = 0; v < 16 / kVec; v++) {
            XT raw[kVec];
            const uint4 t = *reinterpret_cast<const uint4*>(__builtin_assume_aligned(xm + k0 + kVec * v, 16));
            __builtin_memcpy(raw, &t, 16);
#pragma unroll
            for (int i = 0; i < kVec; i++) xr[16 * q + kVec * v + i] = XElem<XT>::load(raw, i);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; i++) xr[16 * q + i] = 0.f;      // past the end of a Q8_0 row of an odd number of blocks
        }
      }
      // (rows past the end repeat the last one; their sums are not stored)
#pragma unroll
      for (int r = 0; r < kLongRows; r++)
        acc[r] += F::dot(F::load(w + rb * min(row0 + r, n_out - 1), u, n_in), xr);
    }
#pragma unroll
    for (int r = 0; r < kLongRows; r++) {
      const float sum = wave_sum(acc[r]);
      if (lane == 0) part[wave][r] = sum;
    }
    __syncthreads();
    if (tid < kLongRows && row0 + tid < n_out) {
      float sum = part[0][tid];
#pragma unroll
      for (int v = 1; v < kGemvWaves; v++) sum += part[v][tid];
      YElem<YT>::store(ym, row0 + tid, sum + load_bias(bias, bias_dtype, row0 + tid));
    }
    __syncthreads();      // part is written again in the next round
  }
}

template <class F, typename XT, typename YT>
static hipError_t launch_long(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m,
                              int64_t n_out, int64_t n_in, hipStream_t s) {
  const int64_t need = (n_out + kLongRows - 1) / kLongRows, most = (int64_t)device_num_cus() * 8;
  const dim3 grid((unsigned)(need < most ? need : most), (unsigned)m), block(kGemvThreads);
  hipLaunchKernelGGL((gemv_long_kernel<F, XT, YT>), grid, block, 0, s, static_cast<const uint8_t*>(w),
                     static_cast<const XT*>(x), static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)n_in);
  return hipGetLastError();
}
template <class F, typename XT>
static hipError_t launch_long_y(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                                int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return launch_long<F, XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_long<F, XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_long<F, XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}
template <class F>
static hipError_t launch_long_xy(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (x_dtype) {
    case kF32: return launch_long_y<F, float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_long_y<F, f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_long_y<F, bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

// Longest row the staged decode kernels take: the packed-dot kernel (Q4_K / Q6_K, 16-bit activations) stages 65536
// activations in 128 KiB of LDS, everything else 16384.
bool gemv_row_is_long(int format, int x_dtype, int64_t n_in) {
  const bool dot2 = (format == kQ4_K || format == kQ6_K) && (x_dtype == kF16 || x_dtype == kBF16);
  return n_in > (dot2 ? kMaxGemvIn16 : kMaxGemvInF32);
}

hipError_t launch_gemv(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                       const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                       hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (gemv_row_is_long(format, x_dtype, n_in)) {
    switch (format) {
      case kQ8_0: TTQ_ROUTE(kRouteGemvLong, launch_long_xy<FmtQ8_0>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
      case kQ4_K: TTQ_ROUTE(kRouteGemvLong, launch_long_xy<FmtQ4_K>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
      case kQ6_K: TTQ_ROUTE(kRouteGemvLong, launch_long_xy<FmtQ6_K>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
      default: return hipErrorInvalidValue;
    }
  }
  // a few rows at once: four per pass for up to four rows and for rows too long for the 8- and
  // 16-token tables, else eight or sixteen per pass
  if (gemv_q4k_stream4_supported(format, x_dtype, m, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ4kStream4, launch_gemv_q4k_stream4(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  static const int batch4_max = dev_knob("TTQ_GEMV_BATCH4_MAX_ROWS", 4);
  const bool b4 = gemv_q4k_batch4_supported(format, x_dtype, m, n_out, n_in);
  if (b4 && m <= batch4_max)
    TTQ_ROUTE(kRouteGemvQ4kBatch4, launch_gemv_q4k_batch4(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q4k_batch_supported(format, x_dtype, m, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ4kBatch, launch_gemv_q4k_batch(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (b4) TTQ_ROUTE(kRouteGemvQ4kBatch4, launch_gemv_q4k_batch4(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q6k_stream4_supported(format, x_dtype, m, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ6kStream4, launch_gemv_q6k_stream4(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_dot2_multi_supported(format, x_dtype, m, n_in))
    TTQ_ROUTE(kRouteGemvDot2Multi, launch_gemv_dot2_multi(format, w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q4k_stream_supported(format, x_dtype, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ4kStream, launch_gemv_q4k_stream(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q4k_slice_supported(format, x_dtype, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ4kSlice, launch_gemv_q4k_slice(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q6k_stream_supported(format, x_dtype, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ6kStream, launch_gemv_q6k_stream(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_mfma_supported(format, x_dtype, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ4kMfma, launch_gemv_mfma(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  // Q8_0 with few weights: the fp32 kernel (a wavefront per row, a row's activations in registers) has the shortest
  // prologue; it re-reads the weights per activation row, so the more rows, the smaller the matrix it wins on.
  // Measured against the matrix-core kernels: 1024x4096 3.9 / 4.8 / 6.3 us for 1 / 2 / 4 rows against 5.3 / 6.5 /
  // 8.5, 2048x4096 5.0 / 6.6 / 10.3 against 5.6 / 6.9 / 8.8, 1024x14336 9.3 / 11.8 / 20.4 against 12.3 / 13.9 / 13.5.
  // (Up to 2048 weight rows, two per wavefront: with short rows its lanes are mostly idle, and more rows of them
  // are the matrix-core kernels' again -- 16384x256 9.2 us against 3.8.)
  if (format == kQ8_0 && m <= 4 && n_out <= 2048) {
    const float mb = (float)(n_out * (n_in / 32) * 34) * 1e-6f;
    const float limit = n_in <= 4096 ? (m == 1 ? 12.f : (m == 2 ? 8.5f : 6.f)) : (m <= 2 ? 16.f : 0.f);
    if (mb <= limit) TTQ_ROUTE(kRouteGemvGeneric, launch_generic_xy<FmtQ8_0>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  }
  if (m == 1 && gemv_q8_stream_supported(format, x_dtype, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ8Stream, launch_gemv_q8_stream(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q8_win_supported(format, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ8Win, launch_gemv_q8_win(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_q8_mfma_supported(format, n_out, n_in))
    TTQ_ROUTE(kRouteGemvQ8Mfma, launch_gemv_q8_mfma(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (gemv_dot2_supported(format, x_dtype, n_in))
    TTQ_ROUTE(kRouteGemvDot2, launch_gemv_dot2(format, w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  switch (format) {
    case kQ8_0: TTQ_ROUTE(kRouteGemvGeneric, launch_generic_xy<FmtQ8_0>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
    case kQ4_K: TTQ_ROUTE(kRouteGemvGeneric, launch_generic_xy<FmtQ4_K>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
    case kQ6_K: TTQ_ROUTE(kRouteGemvGeneric, launch_generic_xy<FmtQ6_K>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
    default: return hipErrorInvalidValue;
  }
}


// Rough time (microseconds) of launch_gemv for m >= 2 activation rows, following the dispatch
// above: passes over the weights x (packed megabytes / measured rate of the kernel that runs
// + a fixed cost).  ttq_linear_forward weighs it against the prefill GEMM.
float gemv_estimate_us(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in) {
  const int64_t per = format == kQ8_0 ? 32 : 256, blk = format == kQ8_0 ? 34 : (format == kQ4_K ? 144 : 210);
  const float mb = (float)(n_out * (n_in / per) * blk) * 1e-6f;
  // rows of any length: a pass over the weights per activation row (72 MB in 24.6 us, 155 MB in 51 us, 463 MB in 122 us)
  if (gemv_row_is_long(format, x_dtype, n_in)) return (float)m * (mb / 3.5f + 3.f);
  const bool b4 = gemv_q4k_batch4_supported(format, x_dtype, m, n_out, n_in);
  if (b4 && m <= 4) return mb / 2.75f + 2.f;
  if (gemv_q4k_batch_supported(format, x_dtype, m, n_out, n_in)) {
    const int tok = gemv_q4k_batch_tokens(m, n_in);
    // measured at 2.4, 9.4 and 33 MB of packed weights: 8 tokens 5.3 / 7.9 / 13.9 us, 16 tokens
    // 8.9 / 11.5 / 19.7 us per pass
    return (float)((m + tok - 1) / tok) * (tok == 16 ? mb / 2.7f + 7.5f : mb / 3.9f + 5.5f);
  }
  if (b4) return (float)((m + 3) / 4) * (mb / 2.4f + 2.f);
  if (gemv_q6k_stream4_supported(format, x_dtype, m, n_out, n_in)) {
    // measured at 13.8, 48 and 431 MB: two tokens 5.5 / 11.8 / 68.6 us, four tokens 6.5 / 13.6 / 75.4 us per pass;
    // longer rows: two tokens 13.2 us at 48 MB; four tokens a pass, K streamed in one (up to 8192 values) or two
    // parts, each with its own activation tables: 11.9 us at 27.5 MB, 19.2 at 48, 27.4 at 96
    // rows that are not whole rounds nor 256 / 512 / 1024 values: two tokens a pass (152064x3584: 89.6 us at 447 MB)
    if (n_in % 2048 != 0 && n_in != 1024 && n_in != 512 && n_in != 256) return (float)((m + 1) / 2) * (mb / 5.2f + 4.f);
    if (n_in > 4096) return m == 2 ? mb / 5.f + 3.5f : (float)((m + 3) / 4) * (mb / 5.8f + (n_in > 8192 ? 11.f : 7.2f));
    return m == 2 ? mb / 6.4f + 3.5f : (float)((m + 3) / 4) * (mb / 5.8f + 4.f);
  }
  if (gemv_dot2_multi_supported(format, x_dtype, m, n_in))
    return m <= 2 ? mb / 2.6f + 2.f : (float)((m + 3) / 4) * (mb / 1.7f + 2.f);
  // the register-streamed int8 matrix-core kernel (Q4_K with fp32 activations): a pass per row; measured at 9.4 / 33 /
  // 295 MB: 4.3 / 6.8 / 53 us for one row, 2.4 / 5.0 / 46.5 us for every further one
  if (gemv_mfma_supported(format, x_dtype, n_out, n_in)) return 2.f + (float)m * (mb / 6.8f + 0.8f);
  if (gemv_q8_win_supported(format, n_out, n_in)) {
    const int tok = gemv_q8_win_tokens(x_dtype, m, n_in);
    return (float)((m + tok - 1) / tok) * (mb / (tok == 4 ? 3.1f : 3.6f) + 2.f);
  }
  // the generic kernel, a pass per row (Q6_K with fp32 activations, 3.4 / 13.8 / 48 MB: 4.1 / 7.5 / 16.2 us for one
  // row, 1.2 / 4.5 / 11 us for every further one; rows of 14336 values take twice that)
  return 3.f + (float)m * (mb / 3.3f + 0.3f);
}

}  // namespace ttq
