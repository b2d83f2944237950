// Pieces shared by the trellis kernels: the codebook, the 128-group Hadamard butterfly held in
// registers, and four-element activation loads.
#pragma once

#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {

typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;

// The codebook: a pure function of the 16-bit trellis state (bits 16..31 of `state` are ignored).
// The 32-bit multiply is not what limits the decode here: splitting it into two 16-bit
// multiply-adds was measured slower.
template <int CB>
struct Codebook {
  static constexpr uint32_t kMul = (CB == 0) ? 89226354u : 0xCBAC1FEDu;
  __device__ __forceinline__ void init() {}
  __device__ __forceinline__ _Float16 code(uint32_t state) const {
    uint32_t u = (state & 0xFFFFu) * kMul;
    if (CB == 0) u += 64248484u;
    u = (u & 0x8FFF8FFFu) ^ 0x3B603B60u;
    half2_t h;
    __builtin_memcpy(&h, &u, 4);
    return h[0] + h[1];  // fp16 add, round-to-nearest-even
  }
};

// Unnormalized FWHT of a 128-group held as 4 consecutive values in each of 32 consecutive lanes
// (value index = 4*lane + i): stages 1 and 2 inside the lane, stages 4..64 against the lane
// 1, 2, 4, 8, 16 away.  Same stage order and operand order as the textbook loop
// (lower index gets a+b, upper a-b), so the results do not depend on how it is laid out.
__device__ __forceinline__ void fwht128_quad(float (&v)[4], int lane) {
  float t;
  t = v[0]; v[0] = t + v[1]; v[1] = t - v[1];
  t = v[2]; v[2] = t + v[3]; v[3] = t - v[3];
  t = v[0]; v[0] = t + v[2]; v[2] = t - v[2];
  t = v[1]; v[1] = t + v[3]; v[3] = t - v[3];
#pragma unroll
  for (int d = 1; d < 32; d <<= 1) {
    const bool upper = (lane & d) != 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float o = __shfl_xor(v[i], d, kWave);
      v[i] = upper ? (o - v[i]) : (v[i] + o);
    }
  }
}

// Four consecutive activations (a multiple of four elements from the row start) as floats.
__device__ __forceinline__ void load_x4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(__builtin_assume_aligned(p, 16));
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load_x4(const f16_tag* p, float (&v)[4]) {
  uint2 r;
  __builtin_memcpy(&r, __builtin_assume_aligned(p, 8), 8);
  v[0] = f16_bits_to_f32((uint16_t)r.x); v[1] = f16_bits_to_f32((uint16_t)(r.x >> 16));
  v[2] = f16_bits_to_f32((uint16_t)r.y); v[3] = f16_bits_to_f32((uint16_t)(r.y >> 16));
}
__device__ __forceinline__ void load_x4(const bf16_tag* p, float (&v)[4]) {
  uint2 r;
  __builtin_memcpy(&r, __builtin_assume_aligned(p, 8), 8);
  v[0] = bf16_bits_to_f32((uint16_t)r.x); v[1] = bf16_bits_to_f32((uint16_t)(r.x >> 16));
  v[2] = bf16_bits_to_f32((uint16_t)r.y); v[3] = bf16_bits_to_f32((uint16_t)(r.y >> 16));
}

}  // namespace ttq
