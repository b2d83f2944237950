// Elementwise / row-wise pieces around the linear layers: silu_and_mul and RMSNorm.
//
// silu_and_mul: out[..., :h] = silu(in[..., :h]) * in[..., h:2h].
//
// Stand-in for workspace/transformers/src/kernels/activations.nim:14-38, which GatedMLP
// applies to the output of the fused gate/up projection
// (workspace/transformers/src/layers/mlp.nim:56-60).  The arithmetic is fp32 with one
// rounding to the output type (the reference rounds silu(gate) to the tensor type first).
// Memory-bound elementwise work: 16-byte loads and stores when the width allows.
#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {

__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.f + expf(-g))) * u; }

template <typename T>
__global__ void __launch_bounds__(256)
silu_and_mul_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t m, int64_t h) {
  const int64_t total = m * h;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / h, c = i - r * h;
    const float g = XElem<T>::load(in, r * 2 * h + c), u = XElem<T>::load(in, r * 2 * h + h + c);
    YElem<T>::store(out, i, silu_mul(g, u));
  }
}

// eight 16-bit elements per thread; h must be a multiple of 8 and the rows 16-byte aligned
template <bool BF16>
__global__ void __launch_bounds__(256)
silu_and_mul16_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int64_t m, int64_t h8) {
  const int64_t total = m * h8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / h8, c = i - r * h8;
    const uint4 gv = *reinterpret_cast<const uint4*>(in + (r * 2 * h8 + c) * 8);
    const uint4 uv = *reinterpret_cast<const uint4*>(in + (r * 2 * h8 + h8 + c) * 8);
    const uint32_t gd[4] = {gv.x, gv.y, gv.z, gv.w}, ud[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t od[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      float g0, g1, u0, u1;
      if (BF16) {
        g0 = bf16_bits_to_f32((uint16_t)gd[k]); g1 = bf16_bits_to_f32((uint16_t)(gd[k] >> 16));
        u0 = bf16_bits_to_f32((uint16_t)ud[k]); u1 = bf16_bits_to_f32((uint16_t)(ud[k] >> 16));
        od[k] = (uint32_t)f32_to_bf16_bits(silu_mul(g0, u0)) | ((uint32_t)f32_to_bf16_bits(silu_mul(g1, u1)) << 16);
      } else {
        g0 = f16_bits_to_f32((uint16_t)gd[k]); g1 = f16_bits_to_f32((uint16_t)(gd[k] >> 16));
        u0 = f16_bits_to_f32((uint16_t)ud[k]); u1 = f16_bits_to_f32((uint16_t)(ud[k] >> 16));
        od[k] = (uint32_t)f32_to_f16_bits(silu_mul(g0, u0)) | ((uint32_t)f32_to_f16_bits(silu_mul(g1, u1)) << 16);
      }
    }
    *reinterpret_cast<uint4*>(out + i * 8) = make_uint4(od[0], od[1], od[2], od[3]);
  }
}

hipError_t launch_silu_and_mul(const void* in, void* out, int dtype, int64_t m, int64_t h, hipStream_t s) {
  if (m == 0 || h == 0) return hipSuccess;
  const auto blocks = [](int64_t work) { return (unsigned)((work + 255) / 256 < 65536 ? (work + 255) / 256 : 65536); };
  if (dtype == kF32) {
    hipLaunchKernelGGL(silu_and_mul_kernel<float>, dim3(blocks(m * h)), dim3(256), 0, s,
                       static_cast<const float*>(in), static_cast<float*>(out), m, h);
  } else if (h % 8 == 0) {
    const uint16_t* i16 = static_cast<const uint16_t*>(in);
    uint16_t* o16 = static_cast<uint16_t*>(out);
    if (dtype == kBF16)
      hipLaunchKernelGGL(silu_and_mul16_kernel<true>, dim3(blocks(m * h / 8)), dim3(256), 0, s, i16, o16, m, h / 8);
    else
      hipLaunchKernelGGL(silu_and_mul16_kernel<false>, dim3(blocks(m * h / 8)), dim3(256), 0, s, i16, o16, m, h / 8);
  } else if (dtype == kBF16) {
    hipLaunchKernelGGL(silu_and_mul_kernel<bf16_tag>, dim3(blocks(m * h)), dim3(256), 0, s,
                       static_cast<const bf16_tag*>(in), static_cast<bf16_tag*>(out), m, h);
  } else {
    hipLaunchKernelGGL(silu_and_mul_kernel<f16_tag>, dim3(blocks(m * h)), dim3(256), 0, s,
                       static_cast<const f16_tag*>(in), static_cast<f16_tag*>(out), m, h);
  }
  return hipGetLastError();
}

// ------------------------------------------------------------------------------ RMSNorm
// One workgroup per row: t = x (+ residual, rounded to the tensor type, as the reference's
// separate add does), normalized = t * rsqrt(mean(t^2) + eps) * gamma in fp32, one rounding.
// Stand-in for RmsNorm.forward / forward_with_residual
// (workspace/transformers/src/layers/norm.nim:23-38).
//
// Two kernels.  rmsnorm_vec_kernel keeps the whole row in registers (16-byte loads, all issued
// before the first use, one pass over memory): rows of up to 1024 * CH vectors whose width and
// addresses are multiples of 16 bytes.  rmsnorm_kernel takes everything else element by element
// in two passes (the second one hits in cache: a row is a few KiB).
template <typename T> __device__ __forceinline__ float round_as(float v);
template <> __device__ __forceinline__ float round_as<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_as<f16_tag>(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
template <> __device__ __forceinline__ float round_as<bf16_tag>(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_kernel(const T* x, const T* residual, const T* __restrict__ gamma, float eps, T* new_residual,
               T* normed, int64_t n) {   // new_residual / normed may be x or residual (same index, same thread)
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.x * n;
  auto value = [&](int64_t k) {
    const float t = XElem<T>::load(x, row + k);
    return residual != nullptr ? round_as<T>(t + XElem<T>::load(residual, row + k)) : t;
  };
  float ss = 0.f;
  for (int64_t k = tid; k < n; k += 256) {
    const float t = value(k);
    ss += t * t;
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  const float total = (red[0] + red[1]) + (red[2] + red[3]);
  const float rs = 1.f / sqrtf(total / (float)n + eps);
  for (int64_t k = tid; k < n; k += 256) {
    const float t = value(k);
    if (new_residual != nullptr) YElem<T>::store(new_residual, row + k, t);
    YElem<T>::store(normed, row + k, (t * rs) * XElem<T>::load(gamma, k));
  }
}

// 16 bytes of a row <-> floats
template <typename T> struct Pack16;
template <> struct Pack16<float> {
  static constexpr int kE = 4;
  static __device__ __forceinline__ void unpack(const uint4& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
  }
};
template <> struct Pack16<bf16_tag> {
  static constexpr int kE = 8;
  static __device__ __forceinline__ void unpack(const uint4& v, float* f) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; k++) { f[2 * k] = __uint_as_float(d[k] << 16); f[2 * k + 1] = __uint_as_float(d[k] & 0xffff0000u); }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    uint32_t d[4];
#pragma unroll
    for (int k = 0; k < 4; k++) d[k] = (uint32_t)f32_to_bf16_bits(f[2 * k]) | ((uint32_t)f32_to_bf16_bits(f[2 * k + 1]) << 16);
    return make_uint4(d[0], d[1], d[2], d[3]);
  }
};
template <> struct Pack16<f16_tag> {
  static constexpr int kE = 8;
  static __device__ __forceinline__ void unpack(const uint4& v, float* f) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; k++) { f[2 * k] = f16_bits_to_f32((uint16_t)d[k]); f[2 * k + 1] = f16_bits_to_f32((uint16_t)(d[k] >> 16)); }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    uint32_t d[4];
#pragma unroll
    for (int k = 0; k < 4; k++) d[k] = (uint32_t)f32_to_f16_bits(f[2 * k]) | ((uint32_t)f32_to_f16_bits(f[2 * k + 1]) << 16);
    return make_uint4(d[0], d[1], d[2], d[3]);
  }
};

// One workgroup of blockDim.x (a multiple of 64, at most 1024) threads per row; thread t owns the
// 16-byte vectors t, t + blockDim.x, ... (CH of them at most) of its row from load to store.
template <typename T, int CH>
__global__ void __launch_bounds__(1024)
rmsnorm_vec_kernel(const T* x, const T* residual, const T* __restrict__ gamma, float eps, T* new_residual,
                   T* normed, int64_t n, int nv) {   // outputs may be x or residual: same index, same thread
  constexpr int kE = Pack16<T>::kE;
  __shared__ float red[16];
  const int tid = threadIdx.x, nt = blockDim.x;
  const int64_t row = (int64_t)blockIdx.x * n;
  const uint4* xr = reinterpret_cast<const uint4*>(x + row);
  const uint4* rr = residual != nullptr ? reinterpret_cast<const uint4*>(residual + row) : nullptr;
  const uint4* gr = reinterpret_cast<const uint4*>(gamma);
  uint4 xv[CH], rv[CH], gv[CH];
#pragma unroll
  for (int c = 0; c < CH; c++) {
    const int i = tid + c * nt;
    if (i < nv) {
      xv[c] = xr[i];
      if (residual != nullptr) rv[c] = rr[i];
      gv[c] = gr[i];
    }
  }
  float t[CH][kE];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; c++) {
    if (tid + c * nt < nv) {
      Pack16<T>::unpack(xv[c], t[c]);
      if (residual != nullptr) {
        float r[kE];
        Pack16<T>::unpack(rv[c], r);
#pragma unroll
        for (int k = 0; k < kE; k++) t[c][k] = round_as<T>(t[c][k] + r[k]);
      }
#pragma unroll
      for (int k = 0; k < kE; k++) ss += t[c][k] * t[c][k];
    }
  }
  ss = wave_sum(ss);
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < (nt >> 6); w++) total += red[w];
  const float rs = 1.f / sqrtf(total / (float)n + eps);
  uint4* nr = new_residual != nullptr ? reinterpret_cast<uint4*>(new_residual + row) : nullptr;
  uint4* no = reinterpret_cast<uint4*>(normed + row);
#pragma unroll
  for (int c = 0; c < CH; c++) {
    const int i = tid + c * nt;
    if (i < nv) {
      if (new_residual != nullptr) nr[i] = Pack16<T>::pack(t[c]);
      float g[kE], o[kE];
      Pack16<T>::unpack(gv[c], g);
#pragma unroll
      for (int k = 0; k < kE; k++) o[k] = (t[c][k] * rs) * g[k];
      no[i] = Pack16<T>::pack(o);
    }
  }
}

template <typename T>
static bool launch_rmsnorm_vec(const void* x, const void* residual, const void* gamma, float eps, void* new_residual_out,
                               void* normed_out, int64_t m, int64_t n, hipStream_t s) {
  constexpr int kE = Pack16<T>::kE;
  const auto misaligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
  if (n % kE != 0 || n / kE > 8 * 1024 || misaligned(x) || misaligned(residual) || misaligned(gamma) ||
      misaligned(new_residual_out) || misaligned(normed_out))
    return false;
  const int nv = (int)(n / kE);
  // the fewest vectors per thread that a workgroup of at most 1024 threads allows
  const int ch = nv <= 1024 ? 1 : nv <= 2048 ? 2 : nv <= 4096 ? 4 : 8;
  const int threads = ((nv + ch - 1) / ch + 63) / 64 * 64;
  const dim3 grid((unsigned)m), block((unsigned)threads);
  const T* xp = static_cast<const T*>(x);
  const T* rp = static_cast<const T*>(residual);
  const T* gp = static_cast<const T*>(gamma);
  T* np = static_cast<T*>(new_residual_out);
  T* op = static_cast<T*>(normed_out);
  switch (ch) {
    case 1: hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 1>), grid, block, 0, s, xp, rp, gp, eps, np, op, n, nv); break;
    case 2: hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 2>), grid, block, 0, s, xp, rp, gp, eps, np, op, n, nv); break;
    case 4: hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 4>), grid, block, 0, s, xp, rp, gp, eps, np, op, n, nv); break;
    default: hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 8>), grid, block, 0, s, xp, rp, gp, eps, np, op, n, nv); break;
  }
  return true;
}

template <typename T>
static void launch_rmsnorm_as(const void* x, const void* residual, const void* gamma, float eps, void* new_residual_out,
                              void* normed_out, int64_t m, int64_t n, hipStream_t s) {
  if (launch_rmsnorm_vec<T>(x, residual, gamma, eps, new_residual_out, normed_out, m, n, s)) return;
  hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3((unsigned)m), dim3(256), 0, s, static_cast<const T*>(x),
                     static_cast<const T*>(residual), static_cast<const T*>(gamma), eps,
                     static_cast<T*>(new_residual_out), static_cast<T*>(normed_out), n);
}

hipError_t launch_rmsnorm(const void* x, const void* residual, const void* gamma, float eps, int dtype,
                          void* new_residual_out, void* normed_out, int64_t m, int64_t n, hipStream_t s) {
  if (m == 0 || n == 0) return hipSuccess;
  if (dtype == kF32)
    launch_rmsnorm_as<float>(x, residual, gamma, eps, new_residual_out, normed_out, m, n, s);
  else if (dtype == kBF16)
    launch_rmsnorm_as<bf16_tag>(x, residual, gamma, eps, new_residual_out, normed_out, m, n, s);
  else
    launch_rmsnorm_as<f16_tag>(x, residual, gamma, eps, new_residual_out, normed_out, m, n, s);
  return hipGetLastError();
}

}  // namespace ttq
