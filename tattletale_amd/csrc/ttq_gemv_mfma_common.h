// Pieces shared by the matrix-core decode GEMV kernels (ttq_gemv_mfma.hip for Q4_K,
// ttq_gemv_q8_mfma.hip for Q8_0): launch shape, activation widening / narrowing, byte packing.
#pragma once

#include "ttq_device.h"
#include "ttq_internal.h"

#include <stdlib.h>

namespace ttq {

typedef int v4i_t __attribute__((ext_vector_type(4)));

constexpr int kMfmaThreads = 1024;
constexpr int kMfmaWaves = kMfmaThreads / kWave;
// Steps in flight per wavefront.  One is best: with 16 wavefronts that is 48 KiB requested per
// CU; asking for more lets the memory system serve the CUs unevenly, and the ones served last
// unpack their whole share after the stream has ended.
constexpr int kMfmaRing = 1;
constexpr int64_t kMaxMfmaIn = 16384;           // the limit of the GEMV entry points
constexpr int kMaxWideSb = 32;                  // up to here the 4 KiB-per-super-block plane table fits LDS

template <int CTRL>
__device__ __forceinline__ float dpp_quad(float v) {
  // (the lane's own value as the "old" operand: every lane has a source, and the compiler need not clear a register)
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false));
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_quad_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}
// lane i of every eight gets lane 7 - i (row_half_mirror): with quads that already agree, the other quad's value
__device__ __forceinline__ uint32_t dpp_other_quad_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, 0x141, 0xF, 0xF, false);
}

// max |f| as the bit pattern of a non-negative float.  Integer compares on purpose: a NaN, which fmaxf would
// drop, counts as larger than infinity, so its exponent field (255) poisons the block as infinity's does.
template <int N>
__device__ __forceinline__ uint32_t amax_bits(const float (&f)[N]) {
  uint32_t a = 0u;
#pragma unroll
  for (int i = 0; i < N; i++) {
    const uint32_t b = __float_as_uint(f[i]) & 0x7FFFFFFFu;
    a = a > b ? a : b;
  }
  return a;
}
__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

template <typename XT> __device__ __forceinline__ void widen8(const uint4& v, float (&f)[8]);
template <> __device__ __forceinline__ void widen8<bf16_tag>(const uint4& v, float (&f)[8]) {
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    f[2 * i] = __uint_as_float(d[i] << 16);
    f[2 * i + 1] = __uint_as_float(d[i] & 0xFFFF0000u);
  }
}
template <> __device__ __forceinline__ void widen8<f16_tag>(const uint4& v, float (&f)[8]) {
  const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    f[2 * i] = f16_bits_to_f32((uint16_t)(d[i] & 0xFFFFu));
    f[2 * i + 1] = f16_bits_to_f32((uint16_t)(d[i] >> 16));
  }
}

// float -> the 16-bit activation type and back (one rounding, nearest-even)
template <typename XT> __device__ __forceinline__ uint16_t narrow1(float v);
template <> __device__ __forceinline__ uint16_t narrow1<bf16_tag>(float v) { return f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ uint16_t narrow1<f16_tag>(float v) { return f32_to_f16_bits(v); }
template <typename XT> __device__ __forceinline__ float widen1(uint16_t b);
template <> __device__ __forceinline__ float widen1<bf16_tag>(uint16_t b) { return bf16_bits_to_f32(b); }
template <> __device__ __forceinline__ float widen1<f16_tag>(uint16_t b) { return f16_bits_to_f32(b); }
// rounds eight floats to the 16-bit type in place and returns their packed bits
template <typename XT> __device__ __forceinline__ uint4 narrow8(float (&f)[8]) {
  uint32_t d[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint16_t lo = narrow1<XT>(f[2 * i]), hi = narrow1<XT>(f[2 * i + 1]);
    f[2 * i] = widen1<XT>(lo);
    f[2 * i + 1] = widen1<XT>(hi);
    d[i] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
  return make_uint4(d[0], d[1], d[2], d[3]);
}

// bytes 0 of a, b, c, d -> one dword (a lowest)
__device__ __forceinline__ uint32_t pack_low_bytes(int a, int b, int c, int d) {
  const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
  return p01 | (p23 << 16);
}

// bytes 1 of a, b, c, d -> one dword (a lowest)
__device__ __forceinline__ uint32_t pack_bytes1(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t p01 = __builtin_amdgcn_perm(b, a, 0x0c0c0501u);
  const uint32_t p23 = __builtin_amdgcn_perm(d, c, 0x0c0c0501u);
  return p01 | (p23 << 16);
}

// 1.5 * 2^23: x + this, rounded to fp32, carries rint(x) in its low mantissa bits for |x| < 2^22
constexpr uint32_t kRoundMagicBits = 0x4B400000u;

// Optional RMSNorm in front of a GEMV: what the kernels that normalize the activation row themselves need.
struct GemvNormArgs {
  const uint16_t* residual;     // (m, n_in) or null
  const uint16_t* gamma;        // (n_in)
  uint16_t* new_residual;       // (m, n_in) or null: x + residual
  uint16_t* normed;             // (m, n_in) or null: the normalized activations the GEMV consumed
  float eps;
};

inline int mfma_env_int(const char* name, int dflt) { return dev_knob(name, dflt); }

}  // namespace ttq
