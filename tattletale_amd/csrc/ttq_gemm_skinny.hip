// Q4_K / Q6_K / Q8_0 linear layer for a handful of activation rows (up to 64): the regime between
// the decode GEMV and the prefill GEMM (batched decoding, speculative verification, short prompts).
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
//     16-byte piece per step; the 128 bytes per token block stay in registers for all row blocks
//     of the workgroup;
//   * the four pieces of a row (or token) that one request covers are 64 consecutive bytes, but in
//     operand layout they belong to lanes 16 apart, and the memory pipeline merges the accesses of
//     neighbouring lanes only.  So every request is made with lane = 4 * row + piece and the data
//     is exchanged into lane = row + 16 * piece with ds_bpermute when it is used;
//   * for the weights it is the 8 weights at those k of the lane's row, dequantized in registers
//     (canonical arithmetic written as one exact fused multiply-add, one bf16 rounding).  Q4_K: the
//     8 bytes 8*g .. 8*g+7 of each of the four 32-byte qs chunks, low nibbles for the even sub-block
//     of the chunk, high nibbles for the odd one.  Q6_K: 8 bytes of each ql half-row and 8 of qh per
//     128 weights.  Q8_0: half a block (16 bytes) per pair of steps;
//   * Q4_K: each lane decodes the scale and min of two sub-blocks (2g, 2g+1) of its row and the
//     four lanes of a row exchange them through v_mfma_f32_16x16x4_f32 with a 0/1 selector as the
//     other operand (D[4g'+r][row] = value of lane g = r: an exact all-gather).  Q6_K lanes read
//     the row's 16 scale bytes themselves, Q8_0 lanes the scale of the block they hold;
//   * the eight wavefronts' partial sums meet in LDS once, at the end; the sums are transposed
//     through LDS so that every thread stores 8 consecutive outputs of one token.
//
//   * with the fused gate||up weight (FUSE) row blocks alternate between gate rows and up rows of the
//     same outputs and silu(gate) * up is formed where the partial sums meet.
//
// Algorithmic bytes: the packed weights once (n_out * n_in * 0.5625 for Q4_K) plus m * n_out
// outputs; the activations (m * n_in * 2 per workgroup) come from L2.  The kernel is bound by the
// dequantization (about 3 vector instructions per weight) and the activation re-reads, not by HBM
// or the matrix cores.
#include <type_traits>

#include "ttq_device.h"
#include "ttq_internal.h"

namespace ttq {
namespace {

constexpr int kSkThreads = 512;
constexpr int kSkWaves = kSkThreads / 64;
// time per row block relative to Q4_K (cost model)
constexpr float kSkQ6KWeightFactor = 1.2f, kSkQ8WeightFactor = 2.2f;
constexpr float kSkSplitUs = 2.5f;     // a split launch: store, count and add the copies' sums (three trips to the memory side)

__device__ __forceinline__ uint2 load8_a2(const uint8_t* p) {
  uint2 v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 8);
  return v;
}

// Lane exchange: every lane receives `v` of lane `src_lane4 / 4`.
__device__ __forceinline__ uint32_t pull_lane(uint32_t src_lane4, uint32_t v) {
  return (uint32_t)__builtin_amdgcn_ds_bpermute((int)src_lane4, (int)v);
}
__device__ __forceinline__ void pull_lane(uint32_t s4, uint2& v) { v.x = pull_lane(s4, v.x); v.y = pull_lane(s4, v.y); }
__device__ __forceinline__ void pull_lane(uint32_t s4, uint4& v) {
  v.x = pull_lane(s4, v.x); v.y = pull_lane(s4, v.y); v.z = pull_lane(s4, v.z); v.w = pull_lane(s4, v.w);
}

// D[4g'+r][row] = value of the row's lane g = r, for every g': the four lanes of a row exchange a
// float each (v_mfma_f32_16x16x4_f32 against a 0/1 selector, exact).
__device__ __forceinline__ f32x4_t gather_row4(float sel, float v) {
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  return __builtin_amdgcn_mfma_f32_16x16x4f32(sel, v, zero, 0, 0, 0);
}

// 8 weights as scale * u + offset for the bytes u of q0 (weights 0..3) and q1 (4..7).
__device__ __forceinline__ void fma_bytes(uint32_t q0, uint32_t q1, float scale, float offset, float (&f)[8]) {
  // keep the words opaque: byte k of them converts with one v_cvt_f32_ubyte<k>
  asm volatile("" : "+v"(q0), "+v"(q1));
#pragma unroll
  for (int k = 0; k < 4; k++) {
    f[k] = fmaf_(scale, (float)((q0 >> (8 * k)) & 0xFFu), offset);
    f[4 + k] = fmaf_(scale, (float)((q1 >> (8 * k)) & 0xFFu), offset);
  }
}

// The same for nibbles (bytes 0..15).  Read as an 8-bit float (4 exponent, 3 mantissa bits) the codes
// 0..15 are the subnormals and the first binade, all multiples of one step, so the packed
// conversion to fp32 turns two bytes into (byte * step) exactly with one instruction; the step is
// measured on the constant 0x01 and divided out of the scale (a power of two: exact).
__device__ __forceinline__ void fma_nibbles(uint32_t q0, uint32_t q1, float scale, float offset, float (&f)[8]) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const float step = __builtin_amdgcn_cvt_pk_f32_fp8(1, false)[0];
  const float s = scale * (1.f / step);
  const f32x2_t a = __builtin_amdgcn_cvt_pk_f32_fp8((int)q0, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)q0, true);
  const f32x2_t c = __builtin_amdgcn_cvt_pk_f32_fp8((int)q1, false), d = __builtin_amdgcn_cvt_pk_f32_fp8((int)q1, true);
  f[0] = fmaf_(s, a[0], offset); f[1] = fmaf_(s, a[1], offset);
  f[2] = fmaf_(s, b[0], offset); f[3] = fmaf_(s, b[1], offset);
  f[4] = fmaf_(s, c[0], offset); f[5] = fmaf_(s, c[1], offset);
  f[6] = fmaf_(s, d[0], offset); f[7] = fmaf_(s, d[1], offset);
}

// acc += A(16 x 32) * B(32 x 16) with both operands of the activation type
template <class XT>
__device__ __forceinline__ f32x4_t mfma_16x16x32(const uint32_t (&a)[4], const uint4& b, f32x4_t acc) {
  if constexpr (std::is_same<XT, f16_tag>::value) {
    f16x8_t av, bv;
    __builtin_memcpy(&av, a, 16);
    __builtin_memcpy(&bv, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc, 0, 0, 0);
  } else {
    bf16x8_t av, bv;
    __builtin_memcpy(&av, a, 16);
    __builtin_memcpy(&bv, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, acc, 0, 0, 0);
  }
}

// A format supplies: the bytes of 256 weights of a row (kBlockBytes), what lane (row, kg) keeps of
// them (Raw, fetch), the per-super-block preparation of scales (Prep, prepare) and the 8 weights
// of step i as floats (dequant<PK8>, PK8 = nibbles through the packed 8-bit-float conversion where
// the format has nibbles; the kernel rounds them once to the activation type).
struct SkQ4K {
  static constexpr uint32_t kBlockBytes = 144;
  static __device__ __forceinline__ uint32_t x_lane_k(int kg) { return 8u * kg; }
  static __device__ __forceinline__ constexpr uint32_t x_step_k(int i) { return 32u * i; }
  struct Raw { uint4 hdr; uint2 q[4]; };
  struct Prep { f32x4_t de, dd, me, md; };
  // Bit positions of the 6-bit scale and min of sub-blocks 2kg and 2kg+1 in the 12 packed bytes:
  // sub-blocks 0..3 have the field whole in bytes 0..7, sub-blocks 4..7 four bits in bytes 8..11 and
  // two on top of bytes 0..7.  Two bit-field extracts each, the second of width 0 in the simple case.
  struct Lane {
    float sel;
    bool upper;
    uint32_t kg8, wl, wh, sh_sc[2], sh_mn[2], sh_hi[2];
    __device__ __forceinline__ void init(int li, int kg, int load_kg) {
      sel = ((li & 3) == kg) ? 1.f : 0.f;
      kg8 = 8u * load_kg;
      upper = kg >= 2;
      wl = upper ? 4u : 6u;
      wh = upper ? 2u : 0u;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const uint32_t jj = (2u * kg + h) & 3u;
        sh_sc[h] = 8u * jj;
        sh_mn[h] = upper ? 8u * jj + 4u : 8u * jj;
        sh_hi[h] = 8u * jj + 6u;
      }
    }
  };
  static __device__ __forceinline__ void fetch(Raw& r, const uint8_t* p, const Lane& L) {
    r.hdr = load16_a16(p);
#pragma unroll
    for (int c = 0; c < 4; c++) r.q[c] = *reinterpret_cast<const uint2*>(p + 16 + 32 * c + L.kg8);
  }
  static __device__ __forceinline__ void exchange(Raw& r, uint32_t s4) {
    pull_lane(s4, r.hdr);
#pragma unroll
    for (int c = 0; c < 4; c++) pull_lane(s4, r.q[c]);
  }
  // this lane: sub-blocks 2kg and 2kg+1 of its row; then all eight from the row's four lanes
  static __device__ __forceinline__ void prepare(const Raw& r, const Lane& L, Prep& P) {
    const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    const uint32_t a_sc = L.upper ? r.hdr.w : r.hdr.y;   // bytes 8-11 or 0-3
    const uint32_t a_mn = L.upper ? r.hdr.w : r.hdr.z;   // bytes 8-11 or 4-7
    const uint32_t sc1 = __builtin_amdgcn_ubfe(a_sc, L.sh_sc[0], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.y, L.sh_hi[0], L.wh) << 4);
    const uint32_t sc2 = __builtin_amdgcn_ubfe(a_sc, L.sh_sc[1], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.y, L.sh_hi[1], L.wh) << 4);
    const uint32_t mn1 = __builtin_amdgcn_ubfe(a_mn, L.sh_mn[0], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.z, L.sh_hi[0], L.wh) << 4);
    const uint32_t mn2 = __builtin_amdgcn_ubfe(a_mn, L.sh_mn[1], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.z, L.sh_hi[1], L.wh) << 4);
    P.de = gather_row4(L.sel, d * (float)sc1);
    P.dd = gather_row4(L.sel, d * (float)sc2);
    P.me = gather_row4(L.sel, -(dmin * (float)mn1));
    P.md = gather_row4(L.sel, -(dmin * (float)mn2));
  }
  // fused multiply-add == the canonical two-step form: d is an f16, sc has 6 bits and q 4, so the
  // product is exact in fp32
  template <bool PK8>
  static __device__ __forceinline__ void dequant(const Raw& r, const Prep& P, const Lane&, int i, float (&f)[8]) {
    const int c = i >> 1;
    const float ds = (i & 1) ? P.dd[c] : P.de[c], nm = (i & 1) ? P.md[c] : P.me[c];
    const uint32_t q0 = ((i & 1) ? (r.q[c].x >> 4) : r.q[c].x) & 0x0F0F0F0Fu;
    const uint32_t q1 = ((i & 1) ? (r.q[c].y >> 4) : r.q[c].y) & 0x0F0F0F0Fu;
    if constexpr (PK8) fma_nibbles(q0, q1, ds, nm, f);
    else fma_bytes(q0, q1, ds, nm, f);
  }
};

// Q6_K super-block: ql[128] qh[64] scales[16] d; weight 128h + 32j + l (l < 32) is
// (nibble j/2 of ql[64h + 32(j%2) + l]) | (bits 2j, 2j+1 of qh[32h + l]) << 4, minus 32, times
// d * scales[8h + 2j + l/16].  Step i = 4h + j, l = 8kg .. 8kg+7.
struct SkQ6K {
  static constexpr uint32_t kBlockBytes = 210;
  static __device__ __forceinline__ uint32_t x_lane_k(int kg) { return 8u * kg; }
  static __device__ __forceinline__ constexpr uint32_t x_step_k(int i) { return 32u * i; }
  struct Raw { uint2 qa[2], qb[2], qh[2]; uint4 sc; uint32_t d; };
  struct Prep { float ds[8], off[8]; };
  struct Lane {
    uint32_t kg8, sbit;
    __device__ __forceinline__ void init(int, int kg, int load_kg) {
      kg8 = 8u * load_kg;
      sbit = 8u * (uint32_t)(kg >> 1);      // scale byte l/16 inside each pair of scale bytes
    }
  };
  static __device__ __forceinline__ void exchange(Raw& r, uint32_t s4) {
#pragma unroll
    for (int h = 0; h < 2; h++) { pull_lane(s4, r.qa[h]); pull_lane(s4, r.qb[h]); pull_lane(s4, r.qh[h]); }
    pull_lane(s4, r.sc);
    r.d = pull_lane(s4, r.d);
  }
  static __device__ __forceinline__ void fetch(Raw& r, const uint8_t* p, const Lane& L) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      r.qa[h] = load8_a2(p + 64 * h + L.kg8);
      r.qb[h] = load8_a2(p + 64 * h + 32 + L.kg8);
      r.qh[h] = load8_a2(p + 128 + 32 * h + L.kg8);
    }
    r.sc = load16_a2(p + 192);
    r.d = load2(p + 208);
  }
  static __device__ __forceinline__ void prepare(const Raw& r, const Lane& L, Prep& P) {
    const float d = f16_bits_to_f32((uint16_t)r.d);
    const uint32_t w[4] = {r.sc.x, r.sc.y, r.sc.z, r.sc.w};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      // scale byte 8h + 2j + l/16 = dword 2h + j/2, byte 2(j%2) + l/16
      const int h = i >> 2, j = i & 3;
      const float sc = (float)(int)__builtin_amdgcn_sbfe((int)w[2 * h + (j >> 1)], 16u * (j & 1) + L.sbit, 8);
      P.ds[i] = d * sc;
      P.off[i] = -32.f * P.ds[i];
    }
  }
  // (d * sc) * (q - 32) as one fused multiply-add on the unsigned q: the same exact product
  template <bool PK8>
  static __device__ __forceinline__ void dequant(const Raw& r, const Prep& P, const Lane&, int i, float (&f)[8]) {
    const int h = i >> 2, j = i & 3;
    const uint2 ql = (j & 1) ? r.qb[h] : r.qa[h];
    const uint32_t n0 = ((j >> 1) ? (ql.x >> 4) : ql.x) & 0x0F0F0F0Fu;
    const uint32_t n1 = ((j >> 1) ? (ql.y >> 4) : ql.y) & 0x0F0F0F0Fu;
    const uint32_t h0 = (r.qh[h].x >> (2 * j)) & 0x03030303u;
    const uint32_t h1 = (r.qh[h].y >> (2 * j)) & 0x03030303u;
    fma_bytes((h0 << 4) | n0, (h1 << 4) | n1, P.ds[i], P.off[i], f);
  }
};

// Q8_0: eight blocks of {fp16 d, 32 int8} per 256 weights.  Lane kg keeps half a block per pair of
// steps -- bytes 16(kg%2) .. +15 of block 2p + kg/2 for steps 2p, 2p+1 -- and that block's scale, so
// a pair costs one 16-byte and one 2-byte load.  Step 2p + s then multiplies
// k = 32(2p + kg/2) + 16(kg%2) + 8s .. +7, and the activations are read at the same k.
struct SkQ8_0 {
  static constexpr uint32_t kBlockBytes = 8 * 34;
  static __device__ __forceinline__ uint32_t x_lane_k(int kg) { return 32u * (kg >> 1) + 16u * (kg & 1); }
  static __device__ __forceinline__ constexpr uint32_t x_step_k(int i) { return 64u * (i >> 1) + 8u * (i & 1); }
  struct Raw { uint4 q[4]; uint32_t d[4]; };
  struct Prep { float d[4], off[4]; };
  struct Lane {
    uint32_t bofs;     // byte offset of the lane's block of pair 0
    uint32_t qofs;     // of its 16 quant bytes in it
    __device__ __forceinline__ void init(int, int, int load_kg) {
      bofs = 34u * (uint32_t)(load_kg >> 1);
      qofs = bofs + 2u + 16u * (uint32_t)(load_kg & 1);
    }
  };
  static __device__ __forceinline__ void exchange(Raw& r, uint32_t s4) {
#pragma unroll
    for (int pr = 0; pr < 4; pr++) { pull_lane(s4, r.q[pr]); r.d[pr] = pull_lane(s4, r.d[pr]); }
  }
  static __device__ __forceinline__ void fetch(Raw& r, const uint8_t* p, const Lane& L) {
#pragma unroll
    for (int pr = 0; pr < 4; pr++) {
      r.q[pr] = load16_a2(p + 68 * pr + L.qofs);
      r.d[pr] = load2(p + 68 * pr + L.bofs);
    }
  }
  static __device__ __forceinline__ void prepare(const Raw& r, const Lane&, Prep& P) {
#pragma unroll
    for (int pr = 0; pr < 4; pr++) {
      P.d[pr] = f16_bits_to_f32((uint16_t)r.d[pr]);
      P.off[pr] = -128.f * P.d[pr];
    }
  }
  // d * q as one fused multiply-add on u = q + 128 (the sign bit flipped): d * u - 128 d
  template <bool PK8>
  static __device__ __forceinline__ void dequant(const Raw& r, const Prep& P, const Lane&, int i, float (&f)[8]) {
    const int pr = i >> 1;
    const uint32_t q0 = (i & 1) ? r.q[pr].z : r.q[pr].x, q1 = (i & 1) ? r.q[pr].w : r.q[pr].y;
    fma_bytes(q0 ^ 0x80808080u, q1 ^ 0x80808080u, P.d[pr], P.off[pr], f);
  }
};

// Split along K: the grid holds `splits` copies of the row tiles, copy c works on super-blocks
// [c, c + 1) * nsb / splits, and the copies of a tile add up through a workspace (see the epilogue).
struct SkSplit {
  int splits;          // 1: none
  int tiles;           // workgroups of one copy
  float* partials;
  uint32_t* counters;  // one per tile, zero between launches
  const float* row_scale;   // or null: a factor per token on the sums, before the bias (activations that were scaled row by row)
};
constexpr int kSkMaxCounters = 16384;

// RB: blocks of 16 weight rows per workgroup; TB: blocks of 16 tokens (m <= 16 * TB); WD: ring of
// (super-block, row block) items of packed weights per wavefront, WD - 1 of them in flight; XB:
// buffers for a super-block's activations (2: the next super-block's are requested while this one
// is multiplied).
template <class WF, class XT, int RB, int TB, int WD, int XB, bool FUSE>
__global__ void __launch_bounds__(kSkThreads)
gemm_skinny_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, void* __restrict__ yv,
                       int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                       SkSplit sp) {
  static_assert((WD == 2 || WD == 4) && (2 * RB) % WD == 0 && (XB == 1 || XB == 2), "ring sizes");
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, kg = lane >> 4;
  const int nsb = n_in >> 8;
  // FUSE: the weight holds gate rows [0, n_out) then up rows [n_out, 2 * n_out) (the fused
  // gate||up projection of workspace/transformers/src/layers/mlp.nim:39) and the kernel writes
  // silu(gate . x) * (up . x) for its 8 * RB outputs: row blocks alternate between the gate rows
  // and the up rows of the same 16 outputs.
  static_assert(!FUSE || RB % 2 == 0, "a fused workgroup needs gate and up row blocks in pairs");
  constexpr int kOutPerWg = FUSE ? 8 * RB : 16 * RB;
  const int ksplit = sp.splits > 1 ? (int)blockIdx.x / sp.tiles : 0;
  const int tile_id = (int)blockIdx.x - ksplit * sp.tiles;
  const int n0 = tile_id * kOutPerWg;
  // this workgroup's super-blocks
  const int sb_lo = ksplit * (nsb / sp.splits), sb_hi = sb_lo + nsb / sp.splits;

  // byte offset of (row, super-block 0) and element offset of (token, k = 8*kg)
  uint32_t wofs[RB], xofs[TB];
  // Weights and activations are requested with the four pieces of a row (token) in adjacent lanes
  // (lane = 4 * row + piece: one 64-byte run per row and quad of lanes) and exchanged into the MFMA
  // operand layout (lane = row + 16 * piece) when they are used: the memory pipeline merges the
  // accesses of neighbouring lanes only.
  const int load_row = lane >> 2, load_kg = lane & 3;
  const uint32_t from_lane4 = 4u * (uint32_t)(4 * li + kg);
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
    wofs[rb] = (uint32_t)(FUSE ? min(n0 + 16 * (rb >> 1) + load_row, n_out - 1) + (rb & 1) * n_out
                               : min(n0 + 16 * rb + load_row, n_out - 1)) *
               ((uint32_t)nsb * WF::kBlockBytes);
#pragma unroll
  for (int tb = 0; tb < TB; tb++)
    xofs[tb] = (uint32_t)min(16 * tb + load_row, m - 1) * (uint32_t)n_in + WF::x_lane_k(load_kg);

  f32x4_t acc[RB][TB];
#pragma unroll
  for (int rb = 0; rb < RB; rb++)
#pragma unroll
    for (int tb = 0; tb < TB; tb++) acc[rb][tb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  typename WF::Lane L;
  L.init(li, kg, load_kg);
  auto fetch = [&](typename WF::Raw& r, int sb, int rb) {
    WF::fetch(r, w + wofs[rb] + (uint32_t)sb * WF::kBlockBytes, L);
  };
  // a super-block's activations: piece i is the lane's token at the eight k of step i (for Q4_K and
  // Q6_K k = 32*i + 8*kg .. +7; any assignment of k to (step, kg) works as long as weights and
  // activations agree, and Q8_0 uses one that makes its loads 16 bytes long)
  auto load_x = [&](uint4 (&xf)[TB][8], int sb) {
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
      for (int i = 0; i < 8; i++)
        xf[tb][i] = *reinterpret_cast<const uint4*>(x + xofs[tb] + 256u * (uint32_t)sb + WF::x_step_k(i));
  };

  typename WF::Raw raw[WD];
  uint4 xfr[XB][TB][8];

  // The wavefront's items in order: (super-block, row block), row blocks innermost.  Item rb of a
  // super-block of parity XI lives in raw[(XI * RB + rb) % WD]; while it is multiplied, the item
  // WD - 1 places further on is requested.  Requests past the end re-read this super-block (lines
  // already in cache) so that the load counting stays exact.
  auto super_block = [&](auto xi_c, int sb) {
    constexpr int XI = decltype(xi_c)::value;
    constexpr int kAhead = WD - 1;
    const int sb_next = sb + kSkWaves < sb_hi ? sb + kSkWaves : sb;
    if constexpr (XB == 1) load_x(xfr[0], sb);
    // this super-block's activations into the operand layout (they were requested one super-block
    // ago when there are two buffers)
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
      for (int i = 0; i < 8; i++) pull_lane(from_lane4, xfr[XB == 1 ? 0 : XI][tb][i]);
    if constexpr (XB == 2) load_x(xfr[XI ^ 1], sb_next);
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
      {
        constexpr int kMaxOff = (RB - 1 + kAhead) / RB;
        const int off = (rb + kAhead) / RB;
        int sb_a = sb + off * kSkWaves;
        if (kMaxOff > 1 || off > 0) sb_a = sb_a < sb_hi ? sb_a : sb;
        fetch(raw[(XI * RB + rb + kAhead) % WD], sb_a, (rb + kAhead) % RB);
      }
      typename WF::Raw& r = raw[(XI * RB + rb) % WD];
      WF::exchange(r, from_lane4);
      typename WF::Prep P;
      WF::prepare(r, L, P);
#pragma unroll
      for (int i = 0; i < 8; i++) {
        float f[8];
        // (with three token blocks the compiler schedules the packed conversion badly: 4096 x 14336,
        // 48 rows 36.7 us against 28.0 us with one conversion per byte)
        WF::template dequant<TB != 3>(r, P, L, i, f);
        const uint32_t au[4] = {pack_x2<XT>(f[0], f[1]), pack_x2<XT>(f[2], f[3]), pack_x2<XT>(f[4], f[5]),
                                pack_x2<XT>(f[6], f[7])};
#pragma unroll
        for (int tb = 0; tb < TB; tb++)
          acc[rb][tb] = mfma_16x16x32<XT>(au, xfr[XB == 1 ? 0 : XI][tb][i], acc[rb][tb]);
      }
    }
  };

  if (sb_lo + wave < sb_hi) {
#pragma unroll
    for (int q = 0; q < WD - 1; q++) {
      const int sb_q = sb_lo + wave + (q / RB) * kSkWaves;
      fetch(raw[q % WD], sb_q < sb_hi ? sb_q : sb_lo + wave, q % RB);
    }
    if (XB == 2) load_x(xfr[0], sb_lo + wave);
  }
  for (int sb = sb_lo + wave; sb < sb_hi; sb += 2 * kSkWaves) {
    super_block(std::integral_constant<int, 0>{}, sb);
    if (sb + kSkWaves < sb_hi) super_block(std::integral_constant<int, 1>{}, sb + kSkWaves);
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
  // ---- split along K: the tile of sums goes to the workspace, a counter per tile says how many copies have
  // arrived, and the workgroup that arrives last adds all copies in copy order -- the same sum whichever
  // arrives last -- and writes the outputs.  Nobody waits for anybody.  Sums and counter move as device-scope
  // relaxed atomics (the L2 caches of the dies are not coherent with each other; these accesses go through to
  // the memory side), the stores are complete before the count, the loads are issued after it.
  if constexpr (!FUSE) {
    if (sp.splits > 1) {
      constexpr int kTileFloats = 16 * TB * kTileLd;
      float* all = sp.partials + (size_t)tile_id * (size_t)(sp.splits * kTileFloats);
      float* mine = all + ksplit * kTileFloats;
      for (int e = tid; e < kTileFloats; e += kSkThreads)
        __hip_atomic_store(mine + e, tile[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      uint32_t* flag = reinterpret_cast<uint32_t*>(part);          // the wavefronts' partial sums are done with
      if (tid == 0)
        flag[0] = __hip_atomic_fetch_add(sp.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (flag[0] != (uint32_t)(sp.splits - 1)) return;
      if (tid == 0) __hip_atomic_store(sp.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      for (int e = tid; e < kTileFloats; e += kSkThreads) {
        float v = __hip_atomic_load(all + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int c = 1; c < sp.splits; c++)
          v += __hip_atomic_load(all + c * kTileFloats + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        tile[e] = v;
      }
      __syncthreads();
    }
  }
  // 8 consecutive outputs of one token per thread
  constexpr int kGroups = kOutPerWg / 8;
  for (int t = tid; t < 16 * TB * kGroups; t += kSkThreads) {
    const int tok = t / kGroups, g = t % kGroups;
    const int col = n0 + 8 * g;
    if (tok >= m || col >= n_out) continue;      // n_out is a multiple of 8: a group is all in or all out
    float v[8];
    const float rs = !FUSE && sp.row_scale ? sp.row_scale[tok] : 1.f;
    if constexpr (FUSE) {
      // outputs 8g .. 8g+7 of the workgroup: gate in row block 2 * (g / 2), up in the next one
      const int lr = 32 * (g >> 1) + 8 * (g & 1);
#pragma unroll
      for (int k = 0; k < 8; k++) {
        const float gt = tile[tok * kTileLd + lr + k] + load_bias(bias, bias_dtype, col + k);
        const float up = tile[tok * kTileLd + lr + 16 + k] + load_bias(bias, bias_dtype, (int64_t)n_out + col + k);
        // silu with the hardware exp2 / reciprocal, as the tiled kernel's epilogue forms it
        v[k] = (gt * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(gt * -1.4426950408889634f))) * up;
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; k++) v[k] = tile[tok * kTileLd + 8 * g + k] * rs + load_bias(bias, bias_dtype, col + k);
    }
    const int64_t o = (int64_t)tok * n_out + col;
    if (y_dtype == kBF16) {
      *reinterpret_cast<uint4*>(static_cast<uint16_t*>(yv) + o) =
          make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
    } else if (y_dtype == kF16) {
      *reinterpret_cast<uint4*>(static_cast<uint16_t*>(yv) + o) =
          make_uint4(pack_f16x2(v[0], v[1]), pack_f16x2(v[2], v[3]), pack_f16x2(v[4], v[5]), pack_f16x2(v[6], v[7]));
    } else {
      float4* yo = reinterpret_cast<float4*>(static_cast<float*>(yv) + o);
      yo[0] = make_float4(v[0], v[1], v[2], v[3]);
      yo[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
  }
}

// n_out counts outputs: weight rows, or gate/up pairs when fused.
template <int RB, int TB, bool FUSE, class K>
hipError_t launch_skinny_k(K kernel, const uint8_t* w, const uint16_t* x, void* y, int y_dtype, const void* bias,
                           int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int splits, hipStream_t s,
                           const float* row_scale) {
  const size_t lds = (size_t)(kSkWaves * RB * TB * 4 * 64 + 16 * TB * (16 * RB + 1)) * sizeof(float);
  static LargeLds configured;          // one per kernel instantiation: K is part of this function's type
  if (lds > 64 * 1024) {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
    if (e != hipSuccess) return e;
  }
  constexpr int kOutPerWg = FUSE ? 8 * RB : 16 * RB;
  const int tiles = (int)((n_out + kOutPerWg - 1) / kOutPerWg);
  SkSplit sp{1, tiles, nullptr, nullptr, row_scale};
  if (!FUSE && splits > 1) {
    // (the chooser has checked that the super-blocks divide evenly and that the counters suffice)
    void* part = nullptr;
    void* cnt = nullptr;
    hipError_t e = stream_workspace(kWsGemmPartials, s, (size_t)tiles * splits * (16 * TB * (16 * RB + 1)) * sizeof(float), &part);
    if (e == hipSuccess) e = stream_workspace(kWsGemmCounters, s, (size_t)kSkMaxCounters * 4, &cnt, true);
    if (e != hipSuccess) return e;
    sp.splits = splits;
    sp.partials = static_cast<float*>(part);
    sp.counters = static_cast<uint32_t*>(cnt);
  }
  const dim3 grid((unsigned)(tiles * sp.splits)), block(kSkThreads);
  hipLaunchKernelGGL(kernel, grid, block, lds, s, w, x, y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, sp);
  return hipGetLastError();
}

template <class WF, class XT, int RB, int TB, int WD, int XB, bool FUSE>
hipError_t launch_skinny_tb(const uint8_t* w, const uint16_t* x, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int splits, hipStream_t s,
                            const float* row_scale) {
  return launch_skinny_k<RB, TB, FUSE>(gemm_skinny_kernel<WF, XT, RB, TB, WD, XB, FUSE>, w, x, y, y_dtype, bias,
                                       bias_dtype, m, n_out, n_in, splits, s, row_scale);
}

// Cost model (microseconds), a least-squares fit to 4096 x 4096, 4096 x 14336 and 14336 x 4096 with
// Q4_K weights, 16 and 64 weight rows per workgroup: rounds of workgroups over the CUs x (fixed +
// super-blocks per wavefront x (activation loads + row blocks x weights)) + packed megabytes x
// 0.2 (the stream itself, about 5 TB/s).  The activations of a super-block are re-read from L2 by
// every workgroup, which is what makes more rows per workgroup cheaper per row, as long as every
// CU still gets a workgroup.  The weight term is scaled for the other formats.
float skinny_cost_us(int format, int rb, int splits, int64_t m, int64_t n_out, int64_t n_in) {
  static const float kF0[4] = {1.95f, 2.78f, 2.11f, 2.51f}, kX[4] = {0.44f, 1.30f, 1.87f, 2.36f};
  static const float kW[4] = {0.97f, 0.88f, 1.10f, 1.31f};
  const float wf = format == kQ6_K ? kSkQ6KWeightFactor : (format == kQ8_0 ? kSkQ8WeightFactor : 1.f);
  const int64_t block_bytes = format == kQ4_K ? 144 : (format == kQ6_K ? 210 : 272);
  const float mb = (float)(n_out * (n_in >> 8) * block_bytes) * 1e-6f;
  const int t = (int)((m + 15) / 16) - 1;
  const int64_t wgs = splits * ((n_out + 16 * rb - 1) / (16 * rb)), cus = device_num_cus();
  const int64_t iters = ((n_in >> 8) / splits + kSkWaves - 1) / kSkWaves;
  return (float)((wgs + cus - 1) / cus) * (kF0[t] + (float)iters * (kX[t] + rb * wf * kW[t])) + 0.2f * mb +
         (splits > 1 ? kSkSplitUs : 0.f);
}

// rows = weight rows (twice the outputs when fused, which also rules out single row blocks).  Few row tiles and a
// long K: every workgroup re-reads all activations of its tokens, so more rows per workgroup are cheaper per
// row, and a second copy of the grid along K gives the compute units those bigger tiles would leave idle
// something to do (4096 x 14336, 64 rows: 16 rows per workgroup 35.6 us, 32 rows in two copies 27.2 us).  The
// kernel takes any number of copies that divides the super-blocks; a sweep over 1 / 2 / 4 / 7 / 8 copies x 16 / 32
// / 64 rows per workgroup on five shapes found nothing that beats two by more than the noise, and the cost
// model above, fitted to full grids, misjudges the deeper splits, so two is what the chooser offers.
struct SkChoice { int rb, splits; float cost_us; };
SkChoice skinny_choose(int format, int64_t m, int64_t rows, int64_t n_in, bool fuse) {
  static const int forced_rb = dev_knob("TTQ_SK_RB", 0);
  static const int forced_splits = dev_knob("TTQ_SK_SPLITS", 0);
  static const int kSplits[] = {1, 2};
  const int64_t nsb = n_in >> 8, cus = device_num_cus();
  SkChoice best{4, 1, 1e30f};
  for (int pass = 0; pass < 2 && best.cost_us > 1e29f; pass++) {
    for (int rb = 4; rb >= (fuse ? 2 : 1); rb >>= 1) {
      if (forced_rb > 0 && rb != forced_rb && !(fuse && forced_rb == 1)) continue;
      const int64_t tiles = (rows + 16 * rb - 1) / (16 * rb);
      for (int sp : kSplits) {
        if (pass == 0 && forced_splits > 0 && sp != forced_splits) continue;
        if (pass == 1 && sp != 1) continue;
        if (sp > 1 && (fuse || nsb % sp != 0 || tiles * sp > cus || tiles > kSkMaxCounters)) continue;
        const float c = skinny_cost_us(format, rb, sp, m, rows, n_in);
        if (c < best.cost_us) best = SkChoice{rb, sp, c};
      }
    }
  }
  return best;
}

// Registers decide how far ahead a wavefront can request: 64 per token block for the activations.
template <class WF, class XT, bool FUSE>
hipError_t launch_skinny_fmt(int format, const uint8_t* wb, const uint16_t* x_bf16, void* y, int y_dtype,
                             const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                             hipStream_t s, const float* row_scale = nullptr) {
  const SkChoice ch = skinny_choose(format, m, FUSE ? 2 * n_out : n_out, n_in, FUSE);
  const int rb = ch.rb;
  const int tb = (int)((m + 15) / 16);
#define TTQ_SK_CASE(RBv, TBv, WDv, XBv) \
  if (rb == RBv && tb == TBv)            \
    return launch_skinny_tb<WF, XT, RBv, TBv, WDv, XBv, FUSE>(wb, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, ch.splits, s, row_scale);
  TTQ_SK_CASE(4, 1, 4, 2) TTQ_SK_CASE(4, 2, 4, 2) TTQ_SK_CASE(4, 3, 2, 1) TTQ_SK_CASE(4, 4, 2, 1)
  TTQ_SK_CASE(2, 1, 4, 2) TTQ_SK_CASE(2, 2, 4, 2) TTQ_SK_CASE(2, 3, 2, 1) TTQ_SK_CASE(2, 4, 2, 1)
  if constexpr (!FUSE) {
    TTQ_SK_CASE(1, 1, 2, 2) TTQ_SK_CASE(1, 2, 2, 2) TTQ_SK_CASE(1, 3, 2, 1) TTQ_SK_CASE(1, 4, 2, 1)
  }
#undef TTQ_SK_CASE
  return hipErrorInvalidValue;
}

}  // namespace

bool gemm_skinny_supported(int format, int64_t m, int64_t n_out, int64_t n_in) {
  static const int disabled = dev_knob("TTQ_GEMM_NO_SKINNY", 0);
  const int64_t block_bytes = format == kQ4_K ? 144 : (format == kQ6_K ? 210 : 272);
  // weight byte offsets and activation element offsets are 32-bit in the kernel; outputs are stored
  // eight at a time
  return !disabled && (format == kQ4_K || format == kQ6_K || format == kQ8_0) && m >= 1 && m <= 64 && n_out > 0 &&
         n_out % 8 == 0 && n_in > 0 && n_in % 256 == 0 && n_out * (n_in / 256) * block_bytes < ((int64_t)1 << 32) &&
         m * n_in < ((int64_t)1 << 31);
}

float gemm_skinny_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in) {
  return skinny_choose(format, m, n_out, n_in, false).cost_us;
}

// The fused gate||up + silu_and_mul form: n_ff outputs from 2 * n_ff weight rows (Q4_K).
bool gemm_skinny_silu_mul_supported(int64_t m, int64_t n_ff, int64_t n_in) {
  return gemm_skinny_supported(kQ4_K, m, 2 * n_ff, n_in) && n_ff % 8 == 0;
}

float gemm_skinny_silu_mul_estimate_us(int64_t m, int64_t n_ff, int64_t n_in) {
  return skinny_choose(kQ4_K, m, 2 * n_ff, n_in, true).cost_us;
}

hipError_t launch_gemm_skinny_silu_mul(const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                                       int bias_dtype, int64_t m, int64_t n_ff, int64_t n_in, hipStream_t s) {
  if (m == 0 || n_ff == 0) return hipSuccess;
  if (y_dtype != kBF16 && y_dtype != kF32) return hipErrorInvalidValue;
  return launch_skinny_fmt<SkQ4K, bf16_tag, true>(kQ4_K, static_cast<const uint8_t*>(w), x_bf16, y, y_dtype, bias, bias_dtype, m,
                                        n_ff, n_in, s);
}

hipError_t launch_gemm_skinny(int format, const void* w, const uint16_t* x, int x_dtype, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                              hipStream_t s, const float* row_scale) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (y_dtype != kBF16 && y_dtype != kF32 && y_dtype != kF16) return hipErrorInvalidValue;
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  if (x_dtype == kBF16) {
    if (row_scale) return hipErrorInvalidValue;      // (row factors come with the scaled fp16 copy of fp32 activations)
    switch (format) {
      case kQ4_K: return launch_skinny_fmt<SkQ4K, bf16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
      case kQ6_K: return launch_skinny_fmt<SkQ6K, bf16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
      case kQ8_0: return launch_skinny_fmt<SkQ8_0, bf16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
      default: return hipErrorInvalidValue;
    }
  }
  if (x_dtype == kF16) {
    switch (format) {
      case kQ4_K: return launch_skinny_fmt<SkQ4K, f16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s, row_scale);
      case kQ6_K: return launch_skinny_fmt<SkQ6K, f16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s, row_scale);
      case kQ8_0: return launch_skinny_fmt<SkQ8_0, f16_tag, false>(format, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s, row_scale);
      default: return hipErrorInvalidValue;
    }
  }
  return hipErrorInvalidValue;
}

// More than 64 rows: one launch per 64 rows.
hipError_t launch_gemm_skinny_chunked(int format, const void* w, const uint16_t* x, int x_dtype, void* y, int y_dtype,
                                      const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                      hipStream_t s, const float* row_scale) {
  const int64_t ysize = y_dtype == kF32 ? 4 : 2;
  for (int64_t r0 = 0; r0 < m; r0 += 64) {
    const int64_t rows = m - r0 < 64 ? m - r0 : 64;
    const hipError_t e = launch_gemm_skinny(format, w, x + r0 * n_in, x_dtype,
                                            static_cast<uint8_t*>(y) + r0 * n_out * ysize, y_dtype, bias, bias_dtype,
                                            rows, n_out, n_in, s, row_scale ? row_scale + r0 : nullptr);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// fp32 activations: every row scaled by a power of two (its largest magnitude to 2^14) and rounded to fp16, row-major,
// with the inverse factors behind the copy; the fp16 kernel multiplies its sums by them.  One workgroup per row.
constexpr int kScaleWaves = 16;      // a row of 14336 values is 3.5 loads per thread: the pass is two trips to memory
static __global__ void __launch_bounds__(64 * kScaleWaves) scale_rows_f16_kernel(const float* __restrict__ x,
                                                                                 uint16_t* __restrict__ xs,
                                                                                 float* __restrict__ inv, int n_in) {
  __shared__ float part[2 * kScaleWaves + 1];
  const float* row = x + (int64_t)blockIdx.x * n_in;
  const float fi = block_row_inverse_factor<kScaleWaves>(row, n_in, part);
  const float f = row_factor_of_inverse(fi);
  const float4* src = reinterpret_cast<const float4*>(row);
  uint2* dst = reinterpret_cast<uint2*>(xs + (int64_t)blockIdx.x * n_in);
  for (int k4 = (int)threadIdx.x; k4 < n_in / 4; k4 += 64 * kScaleWaves) {
    const float4 v = src[k4];
    dst[k4] = make_uint2(pack_f16x2(v.x * f, v.y * f), pack_f16x2(v.z * f, v.w * f));
  }
  if (threadIdx.x == 0) inv[blockIdx.x] = fi;
}

hipError_t launch_gemm_skinny_f32(int format, const void* w, const float* x, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  void* ws = nullptr;
  const size_t copy_bytes = ((size_t)m * (size_t)n_in * 2 + 255) & ~(size_t)255;
  hipError_t e = stream_workspace(kWsPackedActivations, s, copy_bytes + (size_t)m * 4, &ws);
  if (e != hipSuccess) return e;
  uint16_t* xs = static_cast<uint16_t*>(ws);
  float* inv = reinterpret_cast<float*>(static_cast<char*>(ws) + copy_bytes);
  hipLaunchKernelGGL(scale_rows_f16_kernel, dim3((unsigned)m), dim3(64 * kScaleWaves), 0, s, x, xs, inv, (int)n_in);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  return launch_gemm_skinny_chunked(format, w, xs, kF16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s, inv);
}

}  // namespace ttq
