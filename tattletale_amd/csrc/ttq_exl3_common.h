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
template <int D, int N>
__device__ __forceinline__ void fwht_lane_stage(float (&v)[N], int lane) {
  const bool upper = (lane & D) != 0;
#pragma unroll
  for (int i = 0; i < N; i++) {
    const float o = lane_xor<D>(v[i], lane);
    v[i] = upper ? (o - v[i]) : (v[i] + o);
  }
}
__device__ __forceinline__ void fwht128_quad(float (&v)[4], int lane) {
  float t;
  t = v[0]; v[0] = t + v[1]; v[1] = t - v[1];
  t = v[2]; v[2] = t + v[3]; v[3] = t - v[3];
  t = v[0]; v[0] = t + v[2]; v[2] = t - v[2];
  t = v[1]; v[1] = t + v[3]; v[3] = t - v[3];
  fwht_lane_stage<1>(v, lane);
  fwht_lane_stage<2>(v, lane);
  fwht_lane_stage<4>(v, lane);
  fwht_lane_stage<8>(v, lane);
  fwht_lane_stage<16>(v, lane);
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

// ------------------------------------------------------------------------------------------------
// Shared by the matrix-core trellis kernels (decode GEMV and prefill GEMM): workgroup shape, the
// decode of a lane's four weights of a tile into an A fragment, and the LDS layout of a pass of tiles.
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

// 16 wavefronts: a wavefront issues one vector instruction about every five clocks however many others
// share its SIMD, so the decode rate of a compute unit grows with the number of resident wavefronts.
constexpr int kXmThreads = 1024;
constexpr int kXmKSplit = kXmThreads / kWave / 8; // wavefronts per tile column; each takes 8 / kXmKSplit k-tiles of a group
constexpr int kXmTilesPerWave = 8 / kXmKSplit;
constexpr int kXmTok = 8;                         // activation rows per workgroup (two B columns each)
constexpr int kXmChunkTiles = 32;                 // k-tiles per LDS pass
constexpr int kXmChunkK = kXmChunkTiles * 16;
constexpr int kXmColStride = kXmChunkK + 8;       // halfs; 16 bytes of padding: the 16 columns' 8-byte B reads fall on all 64 banks

// Codebook value of the trellis state in bits OFF .. OFF+15 of `w`, written as an fp16 number into half
// HALF of `dst` (the other half is kept when HALF is 1): the sum of the two fp16 numbers that the masked
// hash holds, added by one instruction that picks both halves of its operand itself.
template <int CB, int OFF, int HALF, bool LAST = false>
__device__ __forceinline__ void xm_code(uint32_t w, uint32_t& dst) {
  uint32_t u = __builtin_amdgcn_ubfe(w, OFF, 16) * Codebook<CB>::kMul;
  if constexpr (CB == 0) u += 64248484u;
  u = (u & 0x8FFF8FFFu) ^ 0x3B603B60u;
  if constexpr (HALF == 0)
    asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1" : "=v"(dst) : "v"(u));
  else if constexpr (!LAST)
    asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1"
        : "+v"(dst) : "v"(u));
  else
    // (the wait states keep the matrix-core read that follows clear of the partial register write, which
    // the compiler cannot see inside the statement)
    asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\ts_nop 3"
        : "+v"(dst) : "v"(u));
}

// Four consecutive outputs (idx a multiple of four) in the output buffer's element type.
__device__ __forceinline__ void xm_store4(void* y, int y_dtype, int64_t idx, const float (&o)[4]) {
  if (y_dtype == kF32) {
    *reinterpret_cast<float4*>(static_cast<float*>(y) + idx) = make_float4(o[0], o[1], o[2], o[3]);
  } else {
    uint2 v;
    if (y_dtype == kF16) {
      v.x = (uint32_t)f32_to_f16_bits(o[0]) | ((uint32_t)f32_to_f16_bits(o[1]) << 16);
      v.y = (uint32_t)f32_to_f16_bits(o[2]) | ((uint32_t)f32_to_f16_bits(o[3]) << 16);
    } else {
      v.x = pack_bf16x2(o[0], o[1]);
      v.y = pack_bf16x2(o[2], o[3]);
    }
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + idx) = v;
  }
}

// Four consecutive activations as loaded (converted when they are used, so that the load can stay in flight).
template <typename XT> struct XmRaw;
template <> struct XmRaw<float> {
  float4 r;
  __device__ __forceinline__ void load(const float* p) { r = *reinterpret_cast<const float4*>(__builtin_assume_aligned(p, 16)); }
  __device__ __forceinline__ void get(float (&v)[4]) const { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
};
template <> struct XmRaw<f16_tag> {
  uint2 r;
  __device__ __forceinline__ void load(const f16_tag* p) { __builtin_memcpy(&r, __builtin_assume_aligned(p, 8), 8); }
  __device__ __forceinline__ void get(float (&v)[4]) const {
    v[0] = f16_bits_to_f32((uint16_t)r.x); v[1] = f16_bits_to_f32((uint16_t)(r.x >> 16));
    v[2] = f16_bits_to_f32((uint16_t)r.y); v[3] = f16_bits_to_f32((uint16_t)(r.y >> 16));
  }
};
template <> struct XmRaw<bf16_tag> {
  uint2 r;
  __device__ __forceinline__ void load(const bf16_tag* p) { __builtin_memcpy(&r, __builtin_assume_aligned(p, 8), 8); }
  __device__ __forceinline__ void get(float (&v)[4]) const {
    v[0] = bf16_bits_to_f32((uint16_t)r.x); v[1] = bf16_bits_to_f32((uint16_t)(r.x >> 16));
    v[2] = bf16_bits_to_f32((uint16_t)r.y); v[3] = bf16_bits_to_f32((uint16_t)(r.y >> 16));
  }
};

// Where a lane's windows lie inside a tile's dword string.
template <int BITS>
struct XmLane {
  static constexpr int kWin = BITS <= 5 ? 1 : 2;     // funnel shifts per four weights
  int dw[kWin];                                      // first dword to read, relative to the tile (may be -1)
  uint32_t sh[kWin];                                 // funnel shift
  __device__ __forceinline__ void init(int lane) {
    const int j = lane & 15, q = lane >> 4;
#pragma unroll
    for (int w = 0; w < kWin; w++) {
      const int bit = (16 * j + 4 * q + 2 * w) * BITS;
      const int o = bit & 31, d = bit >> 5;
      // alignbit(hi, lo, s) = low 32 bits of (hi:lo) >> s, s < 32: a window that starts on a dword
      // boundary takes the pair one dword earlier and shifts by nothing
      dw[w] = d - (o == 0);
      sh[w] = (32 - o) & 31;
    }
  }
  // the dwords of one tile that hold this lane's windows
  __device__ __forceinline__ void fetch(const uint32_t* tile, uint32_t (&c)[kWin][2]) const {
#pragma unroll
    for (int w = 0; w < kWin; w++) {
      c[w][0] = tile[dw[w]];
      c[w][1] = tile[dw[w] + 1];
    }
  }
  // the four weights as the matrix cores' A fragment (two registers of two fp16 each)
  template <int CB>
  __device__ __forceinline__ f16x4_t decode(const uint32_t (&c)[kWin][2]) const {
    uint32_t r[2];
    if constexpr (kWin == 1) {
      const uint32_t w = __builtin_amdgcn_alignbit(c[0][0], c[0][1], sh[0]);
      xm_code<CB, 16, 0>(w, r[0]);
      xm_code<CB, 16 - BITS, 1>(w, r[0]);
      xm_code<CB, 16 - 2 * BITS, 0>(w, r[1]);
      xm_code<CB, 16 - 3 * BITS, 1, true>(w, r[1]);
    } else {
#pragma unroll
      for (int p = 0; p < 2; p++) {
        const uint32_t w = __builtin_amdgcn_alignbit(c[p][0], c[p][1], sh[p]);
        xm_code<CB, 16, 0>(w, r[p]);
        if (p == 0) xm_code<CB, 16 - BITS, 1>(w, r[p]);
        else xm_code<CB, 16 - BITS, 1, true>(w, r[p]);
      }
    }
    f16x4_t a;
    __builtin_memcpy(&a, r, 8);
    return a;
  }
};

template <int BITS>
struct XmGeom {
  static constexpr int kTileDw = 8 * BITS;
  static constexpr int kTileStride = kTileDw + 1;                       // + the wrap dword
  static constexpr int kSlabDw = 1 + kXmChunkTiles * 8 * kTileStride;   // one dword in front for dw == -1
  static constexpr int kRunPieces = 16 * BITS;                          // 16-byte pieces of one k-tile's run
  static constexpr int kPieces = kXmChunkTiles * kRunPieces;            // of a full pass
  static constexpr int kSets = (kPieces + kXmThreads - 1) / kXmThreads; // pieces per thread
};

}  // namespace ttq
