// Device-side helpers shared by the gfx950 kernels: 16-bit float handling, wavefront
// reductions, unaligned vector loads and the block-format field decoders.
//
// Arithmetic contract: this library is compiled with -ffp-contract=off, so every float
// operator below rounds once, exactly like the canonical CPU dequantizer; fused
// multiply-adds are written explicitly with fmaf_() where they are wanted.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttq {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kWave = 64;

__device__ __forceinline__ float fmaf_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 v = (_Float16)f;  // round-to-nearest-even
  uint16_t h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float((uint32_t)b << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 v = (__bf16)f;  // v_cvt_pk_bf16_f32: round-to-nearest-even
  uint16_t h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t r;
  r[0] = (__bf16)lo;
  r[1] = (__bf16)hi;
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}

// Two floats -> one dword of fp16 halves, one rounding (to nearest even) each.  The values are made opaque first:
// otherwise the compiler folds a fused multiply-add that produced them into the conversion (v_fma_mix*), which rounds
// the exact sum straight to fp16 instead of rounding the fp32 value -- a different result on ties of the fp32 value.
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  asm("" : "+v"(lo));
  asm("" : "+v"(hi));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  const f16x2_t r = __builtin_convertvector(v, f16x2_t);      // one v_cvt_pk_f16_f32
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}

// Activation element -> float, by buffer element type.
template <typename T> struct XElem;
template <> struct XElem<float> {
  static __device__ __forceinline__ float load(const float* p, int64_t i) { return p[i]; }
};
struct f16_tag { uint16_t v; };
struct bf16_tag { uint16_t v; };
template <> struct XElem<f16_tag> {
  static __device__ __forceinline__ float load(const f16_tag* p, int64_t i) { return f16_bits_to_f32(p[i].v); }
};
template <> struct XElem<bf16_tag> {
  static __device__ __forceinline__ float load(const bf16_tag* p, int64_t i) { return bf16_bits_to_f32(p[i].v); }
};

// two floats -> one dword of the 16-bit type XT (bf16_tag / f16_tag), one rounding each
template <class XT> __device__ __forceinline__ uint32_t pack_x2(float lo, float hi) {
  if constexpr (__is_same(XT, f16_tag)) return pack_f16x2(lo, hi);
  else return pack_bf16x2(lo, hi);
}

// Output element <- float.
// store_through: the same store written through to memory (a relaxed store at system scope).  For the last
// instruction of a short kernel: the launch ends when its stores have reached memory, and a line that sits dirty in
// L2 gets there later (0.1 us on a decode GEMV's 56 KiB of outputs).
template <typename T> struct YElem;
template <> struct YElem<float> {
  static __device__ __forceinline__ void store(float* p, int64_t i, float v) { p[i] = v; }
  static __device__ __forceinline__ void store_through(float* p, int64_t i, float v) {
    __hip_atomic_store(p + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
};
template <> struct YElem<f16_tag> {
  static __device__ __forceinline__ void store(f16_tag* p, int64_t i, float v) { p[i].v = f32_to_f16_bits(v); }
  static __device__ __forceinline__ void store_through(f16_tag* p, int64_t i, float v) {
    __hip_atomic_store(&p[i].v, f32_to_f16_bits(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
};
template <> struct YElem<bf16_tag> {
  static __device__ __forceinline__ void store(bf16_tag* p, int64_t i, float v) { p[i].v = f32_to_bf16_bits(v); }
  static __device__ __forceinline__ void store_through(bf16_tag* p, int64_t i, float v) {
    __hip_atomic_store(&p[i].v, f32_to_bf16_bits(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
};

// Optional bias element n as float (dtype codes: 0 = fp32, 1 = fp16, 2 = bf16).
__device__ __forceinline__ float load_bias(const void* bias, int bias_dtype, int64_t n) {
  if (bias == nullptr) return 0.f;
  if (bias_dtype == 0) return static_cast<const float*>(bias)[n];
  const uint16_t b = static_cast<const uint16_t*>(bias)[n];
  return bias_dtype == 1 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}

// 16-byte load from an address that is only 2-byte aligned (Q6_K / Q8_0 blocks).  gfx950
// global loads accept any alignment; the builtin copy keeps the compiler honest about it.
__device__ __forceinline__ uint4 load16_a2(const uint8_t* p) {
  uint4 v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 16);
  return v;
}
__device__ __forceinline__ uint4 load16_a4(const uint8_t* p) {
  uint4 v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 4), 16);
  return v;
}
__device__ __forceinline__ uint4 load16_a16(const uint8_t* p) {
  return *reinterpret_cast<const uint4*>(__builtin_assume_aligned(p, 16));
}
__device__ __forceinline__ uint32_t load4_a2(const uint8_t* p) {
  uint32_t v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 4);
  return v;
}
__device__ __forceinline__ uint32_t load4_a4(const uint8_t* p) {
  return *reinterpret_cast<const uint32_t*>(__builtin_assume_aligned(p, 4));
}
__device__ __forceinline__ uint16_t load2(const uint8_t* p) {
  uint16_t v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 2);
  return v;
}

// v[i] + v[i ^ 16] and v[i] + v[i ^ 32] in every lane i, by gfx950's row swaps (v_permlane16_swap_b32,
// v_permlane32_swap_b32: with the same register on both sides one result holds the even rows' -- the lower
// half's -- values in every row, the other the odd rows' -- the upper half's): two vector-ALU instructions in
// place of a trip through the LDS crossbar (__shfl_xor is ds_bpermute_b32), same sums bit for bit.
__device__ __forceinline__ float add_xor16(float v) {
  const auto s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}
__device__ __forceinline__ float add_xor32(float v) {
  const auto s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}

// The value of lane (lane ^ D), D a power of two up to 32, without the LDS crossbar that __shfl_xor
// (ds_bpermute_b32) goes through: DPP moves inside a row of 16 lanes -- quad permutes for 1 and 2, a reversal
// of eight lanes followed by a reversal of each quad for 4, a rotation by 8 for 8 -- and gfx950's row swaps
// for 16 and 32.  (Each form was checked against __shfl_xor on the GPU.)
template <int D>
__device__ __forceinline__ float lane_xor(float v, int lane) {
  static_assert(D == 1 || D == 2 || D == 4 || D == 8 || D == 16 || D == 32, "a power of two inside the wavefront");
  const int b = __float_as_int(v);
  if constexpr (D == 1) {
    return __int_as_float(__builtin_amdgcn_update_dpp(b, b, 0xB1, 0xF, 0xF, false));      // quad_perm [1, 0, 3, 2]
  } else if constexpr (D == 2) {
    return __int_as_float(__builtin_amdgcn_update_dpp(b, b, 0x4E, 0xF, 0xF, false));      // quad_perm [2, 3, 0, 1]
  } else if constexpr (D == 4) {
    const int t = __builtin_amdgcn_update_dpp(b, b, 0x141, 0xF, 0xF, false);              // row_half_mirror: i -> 7 - i
    return __int_as_float(__builtin_amdgcn_update_dpp(t, t, 0x1B, 0xF, 0xF, false));      // quad_perm [3, 2, 1, 0]
  } else if constexpr (D == 8) {
    return __int_as_float(__builtin_amdgcn_update_dpp(b, b, 0x128, 0xF, 0xF, false));     // row_ror:8
  } else if constexpr (D == 16) {
    const auto s = __builtin_amdgcn_permlane16_swap((unsigned)b, (unsigned)b, false, false);
    return __uint_as_float((lane & 16) ? s[0] : s[1]);
  } else {
    const auto s = __builtin_amdgcn_permlane32_swap((unsigned)b, (unsigned)b, false, false);
    return __uint_as_float((lane & 32) ? s[0] : s[1]);
  }
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
  const int lane = (int)(threadIdx.x & 63u);
  v = add_xor32(v);
  v = add_xor16(v);
  v += lane_xor<8>(v, lane);
  v += lane_xor<4>(v, lane);
  v += lane_xor<2>(v, lane);
  v += lane_xor<1>(v, lane);
  return v;
}

// fp32 activations for the fp16 matrix cores: the power of two that brings a row's largest magnitude to 2^14 (the row
// then fits fp16 with room for sums of its neighbours, and values down to 2^-38 of the largest stay normal numbers).
// Called by all 64 * NW threads of a workgroup with the row (n_in a multiple of 4, 16-byte aligned) and 2 * NW + 1
// floats of LDS; returns the INVERSE of the factor to every thread.  A row with a non-finite value, or of zeros, is not scaled (1):
// its non-finite values convert as they are and poison that row's outputs only.
template <int NW = 4>
__device__ __forceinline__ float block_row_inverse_factor(const float* __restrict__ row, int n_in, float* part) {
  const int t = (int)threadIdx.x, lane = t & 63, wave = t >> 6;
  const float4* src = reinterpret_cast<const float4*>(row);
  float amax = 0.f, bad = 0.f;
  for (int k4 = t; k4 < n_in / 4; k4 += 64 * NW) {
    const float4 v = src[k4];
    const float a = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    // (fmaxf drops NaNs: look at them separately)
    const bool ok = (__float_as_uint(a) < 0x7F800000u) && (v.x == v.x) && (v.y == v.y) && (v.z == v.z) && (v.w == v.w);
    bad = ok ? bad : 1.f;
    amax = fmaxf(amax, a);
  }
  amax = fmaxf(amax, lane_xor<1>(amax, lane)); bad = fmaxf(bad, lane_xor<1>(bad, lane));
  amax = fmaxf(amax, lane_xor<2>(amax, lane)); bad = fmaxf(bad, lane_xor<2>(bad, lane));
  amax = fmaxf(amax, lane_xor<4>(amax, lane)); bad = fmaxf(bad, lane_xor<4>(bad, lane));
  amax = fmaxf(amax, lane_xor<8>(amax, lane)); bad = fmaxf(bad, lane_xor<8>(bad, lane));
  amax = fmaxf(amax, lane_xor<16>(amax, lane)); bad = fmaxf(bad, lane_xor<16>(bad, lane));
  amax = fmaxf(amax, lane_xor<32>(amax, lane)); bad = fmaxf(bad, lane_xor<32>(bad, lane));
  if (lane == 0) { part[wave] = amax; part[NW + wave] = bad; }
  __syncthreads();
  if (t == 0) {
    amax = part[0];
    bad = part[NW];
#pragma unroll
    for (int v = 1; v < NW; v++) { amax = fmaxf(amax, part[v]); bad = fmaxf(bad, part[NW + v]); }
    // factor = 2^(14 - E), E the exponent of the largest magnitude (subnormal maxima count as 2^-126): biased exponent
    // 268 - (E + 127); it stops at 2^126, so that its inverse stays a normal number: rows of tiny values are simply
    // scaled a little less
    const uint32_t eb = __float_as_uint(amax) >> 23, ec = eb < 1u ? 1u : eb;
    float fi = 1.f;
    if (bad == 0.f && amax > 0.f) {
      const uint32_t fe = 268u - ec > 253u ? 253u : 268u - ec;
      fi = __uint_as_float((254u - fe) << 23);
    }
    part[2 * NW] = fi;
  }
  __syncthreads();
  return part[2 * NW];
}
// the factor from its inverse: both are powers of two
__device__ __forceinline__ float row_factor_of_inverse(float inv) {
  return __uint_as_float((254u - (__float_as_uint(inv) >> 23)) << 23);
}

// Q4_K: 6-bit scale and min of sub-block j (0..7) from the 12 packed bytes held as three
// little-endian dwords s0 (bytes 0-3), s1 (4-7), s2 (8-11).
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j,
                                              uint32_t& sc, uint32_t& mn) {
  if (j < 4) {
    sc = (s0 >> (8 * j)) & 63u;
    mn = (s1 >> (8 * j)) & 63u;
  } else {
    const int jj = j - 4;
    sc = ((s2 >> (8 * jj)) & 0xFu) | (((s0 >> (8 * jj + 6)) & 3u) << 4);
    mn = ((s2 >> (8 * jj + 4)) & 0xFu) | (((s1 >> (8 * jj + 6)) & 3u) << 4);
  }
}

}  // namespace ttq
