// Prefill GEMM for Q4_K, Q6_K and Q8_0 weights on gfx950, producer/consumer form:
// Y (m, n_out) = X (m, n_in) * W^T.
//
// Replaces F.linear(x, weight) for a multi-row bf16 activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81; the prefill case of
//  workspace/transformers/src/layers/attn.nim:154-156).
//
// A wavefront issues its instructions in order, so one that loads, dequantizes AND multiplies
// leaves the matrix pipe idle whenever it is busy with the other two.  Here a workgroup of
// twelve wavefronts (three per SIMD) owns a 256 x BN tile of Y and splits the roles:
//   consumers (wavefronts 0-3, 64 rows of the tile each): nothing but LDS fragment reads and
//       v_mfma_f32_16x16x32_bf16.  Their 64 rows x 64 k of X per step lie in a private pair of LDS stages,
//       the 16-byte chunks of a row XOR-swizzled so that the fragment reads (16 rows x one chunk) hit 16
//       different bank groups.
//   producers (wavefronts 4-7): load the tile's packed blocks once per 256 k, dequantize
//       64 k per step with the format's canonical arithmetic (Q4_K: d*sc*q - dmin*m, where one
//       fused multiply-add reproduces it exactly because d*sc*q has at most 21 significant bits;
//       Q6_K: (d*sc)*(q-32); Q8_0: d*q), round to bf16 nearest-even and write the B fragments to
//       a double-buffered LDS tile.  Only this role knows the weight format.
//   movers (wavefronts 8-11, one per consumer): buffer loads of whole 128-byte lines of X into three rotating
//       register sets, three steps ahead, and ds_write_b128 into the consumer's stage that has just been freed.
// The hardware interleaves the three kinds of wavefront on each SIMD: the vector ALU and memory
// work runs in the shadow of the consumers' MFMAs.  One barrier per 64-k step.
//
// Why X goes through registers and not through global_load_lds: all bytes written to LDS pass one port of about
// 85 bytes per cycle and compute unit, whoever writes.  Reads flow freely past global_load_lds traffic, but a
// ds_write that waits for the port holds up the LDS reads queued behind it, and with the X stream hogging the
// port the W producers' ds_writes waited most of the time: consumers + movers + producers ran half again as long
// as any two of them (measured; the ladder's ABL 2048 rung keeps that form).
//
// This header holds the kernel and its launcher; ttq_gemm_pc.hip chooses the tile and owns the split-K workspace.
// ABL (a bit mask, 0 in the product) switches stages of the kernel off for the measurement ladder of
// ttq_ladder_gemm.hip: 1 the consumers' fragment reads and MFMAs, 2 the movers' requests, 4 the W producers' LDS
// stores, 8 their dequantization arithmetic, 16 their global loads (every role keeps its barriers); 512 reads the
// wavefronts' clocks around the barriers, 1024 drops the barriers, 2048 moves X by global_load_lds into rings of
// four stages, 4096 puts real activation values into every LDS buffer at the start.
#pragma once

#include "ttq_device.h"
#include "ttq_internal.h"

#include <stdlib.h>
#include <type_traits>

namespace ttq {

constexpr int kPcThreads = 768;          // 4 consumers, 4 W producers, 4 X movers
// MB = blocks of 16 rows per consumer wavefront: 4 (a 256-row tile of X per workgroup) for prefill,
// 1 (64 rows) when the whole activation has no more rows than that.
constexpr int kXStages = 4;
constexpr int pc_bm(int mb) { return 64 * mb; }            // rows of X per workgroup
constexpr int pc_xstage(int mb) { return 16 * mb * 128; }  // bytes: one consumer's rows x 64 k of bf16

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}

// The barrier of this kernel.  __syncthreads() would also wait for every outstanding
// global_load_lds (they write LDS, so a release fence drains them), which is exactly the
// prefetch this kernel lives on; all that is needed is that the wavefront's own LDS accesses
// are done and that the compiler moves no LDS access across.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16-byte LDS store the compiler does not see as one.  It cannot tell a store to the W tile
// from the asynchronous global_load_lds writes into the X ring and would wait for ALL
// outstanding requests before every visible LDS store; the barrier protocol below already
// orders the two.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_store16(uint32_t lds_addr, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const u32x4_t v = {a, b, c, d};
  asm volatile("ds_write_b128 %0, %1" : : "v"(lds_addr), "v"(v) : "memory");
}

// ---- what the W producers know about a format.  A producer thread owns one row of the tile
// and, of every 64-k step, the weights k = 16*whalf + e and k = 32 + 16*whalf + e (e = 0..15):
// `lo` and `hi` below, 8 bf16 pairs each (kWholeKsub formats: k = 32*whalf + e, e = 0..31 instead).
// Raw holds the thread's share of 256 k of its row.
template <int FMT> struct WFmt;

template <> struct WFmt<kQ4_K> {
  static constexpr int kUnitBytes = 144;               // one super-block
  static constexpr bool kWholeKsub = false;
  struct Raw { uint4 hdr, q[4]; };
  static __device__ __forceinline__ void load(Raw& dst, const uint8_t* p, int whalf) {
    dst.hdr = load16_a16(p);
#pragma unroll
    for (int c = 0; c < 4; c++) dst.q[c] = load16_a16(p + 16 + 32 * c + 16 * whalf);
  }
  template <int C, class XT = bf16_tag>
  static __device__ __forceinline__ void dequant(const Raw& r, int, uint32_t (&lo)[8], uint32_t (&hi)[8]) {
    const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    uint32_t sc1, mn1, sc2, mn2;
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * C, sc1, mn1);
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * C + 1, sc2, mn2);
    const float d1 = d * (float)sc1, nm1 = -(dmin * (float)mn1);
    const float d2 = d * (float)sc2, nm2 = -(dmin * (float)mn2);
    // Nibble bytes (0..15) read as 8-bit floats (4 exponent, 3 mantissa bits) are the subnormals and
    // the first binade: multiples of one step, so the packed conversion to fp32 gives byte * step
    // exactly, two bytes per instruction; the step (a power of two) is divided out of the scale.
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const float inv_step = 1.f / __builtin_amdgcn_cvt_pk_f32_fp8(1, false)[0];
    const float e1 = d1 * inv_step, e2 = d2 * inv_step;
    const uint32_t qd[4] = {r.q[C].x, r.q[C].y, r.q[C].z, r.q[C].w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // low nibbles are sub-block 2C (the first 32 k of the step), high nibbles sub-block 2C+1
      const uint32_t l4 = qd[i] & 0x0F0F0F0Fu, h4 = (qd[i] >> 4) & 0x0F0F0F0Fu;
      const f32x2_t la = __builtin_amdgcn_cvt_pk_f32_fp8((int)l4, false), lb = __builtin_amdgcn_cvt_pk_f32_fp8((int)l4, true);
      const f32x2_t ha = __builtin_amdgcn_cvt_pk_f32_fp8((int)h4, false), hb = __builtin_amdgcn_cvt_pk_f32_fp8((int)h4, true);
      // fused multiply-add == canonical two-step form here (the product is exact)
      const float fl[4] = {fmaf_(e1, la[0], nm1), fmaf_(e1, la[1], nm1), fmaf_(e1, lb[0], nm1), fmaf_(e1, lb[1], nm1)};
      const float fh[4] = {fmaf_(e2, ha[0], nm2), fmaf_(e2, ha[1], nm2), fmaf_(e2, hb[0], nm2), fmaf_(e2, hb[1], nm2)};
      lo[2 * i] = pack_x2<XT>(fl[0], fl[1]);
      lo[2 * i + 1] = pack_x2<XT>(fl[2], fl[3]);
      hi[2 * i] = pack_x2<XT>(fh[0], fh[1]);
      hi[2 * i + 1] = pack_x2<XT>(fh[2], fh[3]);
    }
  }
};

// Q6_K super-block: ql[128] qh[64] scales[16] d.  Of each 128-weight half, weight l (< 32) is
// the low nibble of ql[l], weight 32+l the low nibble of ql[32+l], weights 64+l and 96+l the
// high nibbles of the same two bytes; qh[l] holds their four 2-bit tops.  Step C of the
// super-block is weights 64*(C&1) .. +63 of half C/2, so the thread needs ql[l], ql[32+l] and
// qh[l] for its l = 16*whalf + e; the scale of weight group t (32 weights) and this l is
// scales[8*half + 2*t + whalf].
template <> struct WFmt<kQ6_K> {
  static constexpr int kUnitBytes = 210;
  static constexpr bool kWholeKsub = false;
  struct Raw { uint4 ql[4], qh[2], sc; uint32_t d; };
  static __device__ __forceinline__ void load(Raw& dst, const uint8_t* p, int whalf) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      dst.ql[2 * h] = load16_a2(p + 64 * h + 16 * whalf);
      dst.ql[2 * h + 1] = load16_a2(p + 64 * h + 32 + 16 * whalf);
      dst.qh[h] = load16_a2(p + 128 + 32 * h + 16 * whalf);
    }
    dst.sc = load16_a2(p + 192);
    dst.d = load2(p + 208);
  }
  template <int C, class XT = bf16_tag>
  static __device__ __forceinline__ void dequant(const Raw& r, int whalf, uint32_t (&lo)[8], uint32_t (&hi)[8]) {
    constexpr int H = C >> 1, ODD = C & 1;
    const float d = f16_bits_to_f32((uint16_t)r.d);
    const uint32_t scw[4] = {r.sc.x, r.sc.y, r.sc.z, r.sc.w};
    const uint32_t sw4 = scw[2 * H + ODD] >> (8 * whalf);       // scales 8H + 4*ODD + whalf (+2)
    const float s1 = d * (float)(int)(int8_t)(sw4 & 0xFFu);
    const float s2 = d * (float)(int)(int8_t)((sw4 >> 16) & 0xFFu);
    const float m1 = -32.f * s1, m2 = -32.f * s2;
    const uint32_t a4[4] = {r.ql[2 * H].x, r.ql[2 * H].y, r.ql[2 * H].z, r.ql[2 * H].w};
    const uint32_t b4[4] = {r.ql[2 * H + 1].x, r.ql[2 * H + 1].y, r.ql[2 * H + 1].z, r.ql[2 * H + 1].w};
    const uint32_t h4[4] = {r.qh[H].x, r.qh[H].y, r.qh[H].z, r.qh[H].w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t qa = ((a4[i] >> (4 * ODD)) & 0x0F0F0F0Fu) | (((h4[i] >> (4 * ODD)) & 0x03030303u) << 4);
      const uint32_t qb = ((b4[i] >> (4 * ODD)) & 0x0F0F0F0Fu) | (((h4[i] >> (4 * ODD + 2)) & 0x03030303u) << 4);
      float fl[4], fh[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        // s * (u - 32) in one fused multiply-add: -32 * s is exact, so the single rounding is
        // that of the canonical product s * (float)(u - 32)
        fl[k] = fmaf_(s1, (float)((qa >> (8 * k)) & 0xFFu), m1);
        fh[k] = fmaf_(s2, (float)((qb >> (8 * k)) & 0xFFu), m2);
      }
      lo[2 * i] = pack_x2<XT>(fl[0], fl[1]);
      lo[2 * i + 1] = pack_x2<XT>(fl[2], fl[3]);
      hi[2 * i] = pack_x2<XT>(fh[0], fh[1]);
      hi[2 * i + 1] = pack_x2<XT>(fh[2], fh[3]);
    }
  }
};

// Q8_0: eight 34-byte blocks { d, q[32] } per 256 k; step C is blocks 2C and 2C+1.  Here a thread
// takes the whole block 2C + whalf of every step (kWholeKsub: its 32 weights are k = 32*whalf + e,
// `lo` the first 16, `hi` the last 16): one scale per block.  Block i starts 34 i = 32 i + 2 i bytes into the
// 272-byte unit, i.e. 2 i bytes into an aligned 16-byte chunk: the thread loads the three aligned chunks that
// hold its block (loads at 2-byte alignment are served several times slower: the Q8_0 GEMM spent twice the
// cycles of the Q4_K one waiting, with the same instruction counts) and shifts the bytes into place when it
// dequantizes.
template <> struct WFmt<kQ8_0> {
  static constexpr int kUnitBytes = 8 * 34;
  static constexpr bool kWholeKsub = true;
  struct Raw { uint4 ch[4][3]; };
  static __device__ __forceinline__ void load(Raw& dst, const uint8_t* p, int whalf) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const uint8_t* a = p + 32 * (2 * c + whalf);
      dst.ch[c][0] = load16_a16(a);
      dst.ch[c][1] = load16_a16(a + 16);
      dst.ch[c][2] = load16_a16(a + 32);
    }
  }
  template <int C, class XT = bf16_tag>
  static __device__ __forceinline__ void dequant(const Raw& r, int whalf, uint32_t (&lo)[8], uint32_t (&hi)[8]) {
    // the block starts 4 C + 2 whalf bytes into the three chunks
    const uint32_t D[12] = {r.ch[C][0].x, r.ch[C][0].y, r.ch[C][0].z, r.ch[C][0].w, r.ch[C][1].x, r.ch[C][1].y,
                            r.ch[C][1].z, r.ch[C][1].w, r.ch[C][2].x, r.ch[C][2].y, r.ch[C][2].z, r.ch[C][2].w};
    const bool odd = whalf != 0;
    const float d = f16_bits_to_f32((uint16_t)(odd ? D[C] >> 16 : D[C] & 0xFFFFu));
    const float md = -128.f * d;
    uint32_t a4[4], b4[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      a4[j] = odd ? D[C + 1 + j] : __builtin_amdgcn_alignbyte(D[C + 1 + j], D[C + j], 2);
      b4[j] = odd ? D[C + 5 + j] : __builtin_amdgcn_alignbyte(D[C + 5 + j], D[C + 4 + j], 2);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // q + 128 as an unsigned byte converts in one instruction; d * (u - 128) as one fused
      // multiply-add rounds once, like the canonical d * q (128 * d is exact)
      const uint32_t ua = a4[i] ^ 0x80808080u, ub = b4[i] ^ 0x80808080u;
      float fl[4], fh[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        fl[k] = fmaf_(d, (float)((ua >> (8 * k)) & 0xFFu), md);
        fh[k] = fmaf_(d, (float)((ub >> (8 * k)) & 0xFFu), md);
      }
      lo[2 * i] = pack_x2<XT>(fl[0], fl[1]);
      lo[2 * i + 1] = pack_x2<XT>(fl[2], fl[3]);
      hi[2 * i] = pack_x2<XT>(fh[0], fh[1]);
      hi[2 * i + 1] = pack_x2<XT>(fh[2], fh[3]);
    }
  }
};

// Split along K: copies of the tile grid, where the copies of a tile leave their partial sums, and the arrival
// counters (zero between launches).

// The same GEMM over a copy of the activations in fragment order (ttq_gemm_pcd.h, instantiated in ttq_gemm_pcd.hip):
// tile = index into launch_gemm_pc's table of tile shapes.
hipError_t launch_gemm_packed(int format, bool fuse, int tile, const uint8_t* wb, const uint16_t* xp, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp,
                              hipStream_t s, bool x_f16 = false, const float* row_scale = nullptr);
size_t gemm_packed_activation_bytes(int64_t m, int64_t n_in);
hipError_t launch_gemm_pack_activations(const void* x, int x_dtype, uint16_t* xp, int64_t m, int64_t n_in, hipStream_t s,
                                        bool keep_f16 = false);
// fp32 activations -> fp16 in fragment order, every row scaled by a power of two that brings its largest magnitude to
// 2^14; row_scale[row] receives the inverse factor
hipError_t launch_gemm_pack_activations_scaled(const float* x, uint16_t* xp, float* row_scale, int64_t m, int64_t n_in,
                                               hipStream_t s);

// What a consumer wavefront does with its finished accumulators (shared by the kernels of this file and of
// ttq_gemm_pcd.h): the meeting of the K copies, bias, silu_and_mul, rounding, and the store of Y.
struct PcEpi {
  PcSplit sp;
  int ksplit, m_tile, n_tile, n_tiles, wave, lane;
  uint8_t* stg;            // this wavefront's LDS staging area: 16 * MB rows of (BN or BO) * 2 + 16 bytes
  void* yv;
  int y_dtype;
  const void* bias;
  int bias_dtype, m, n_out, n0, m0;
  const uint16_t* col_scale = nullptr;   // (ROT) fp16 scale per output column, applied after the rotation
  const float* row_scale = nullptr;      // a factor per row of Y (the activations were scaled row by row), or none
  bool f16_rows = false;                 // fp16 outputs leave through the staged 16-byte row stores too (the fp16 kernels)
};

// ROT (tiles of 128 columns = one Hadamard group of output channels; the trellis layer): the 128 sums of every row
// are rotated (Walsh-Hadamard butterfly, 1/sqrt(128)) and scaled per column before bias and store.
template <int NJ, int MB, bool FUSE, int NC = 4, bool ROT = false>    // NC = consumer wavefronts per workgroup
__device__ __forceinline__ void pc_epilogue(f32x4_t (&acc)[MB][NJ], const PcEpi& e) {
  constexpr int BN = NJ * 16;
  constexpr int BO = FUSE ? BN / 2 : BN;     // outputs per tile
  const PcSplit sp = e.sp;
  const int ksplit = e.ksplit, m_tile = e.m_tile, n_tile = e.n_tile, n_tiles = e.n_tiles, wave = e.wave, lane = e.lane;
  void* yv = e.yv;
  const int y_dtype = e.y_dtype, bias_dtype = e.bias_dtype, m = e.m, n_out = e.n_out, n0 = e.n0, m0 = e.m0;
  const void* bias = e.bias;
  // rows whose activations were scaled before they were rounded (fp32 activations as scaled fp16): undo it on the
  // sums, before the copies along K meet and before the bias
  if (e.row_scale != nullptr) {
    const int rs4 = (lane >> 4) * 4;
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float f = e.row_scale[min(m0 + 16 * i + rs4 + r, m - 1)];
#pragma unroll
        for (int j = 0; j < NJ; j++) acc[i][j][r] *= f;
      }
  }
  // ---- split along K: this wavefront's 64 x BN partial sums go to the workspace (whole kilobytes per store
  // instruction), a counter per (tile, consumer) says how many copies have arrived, and the wavefront that
  // arrives last adds all copies in copy order -- the same sum whichever arrives last -- and carries on to the
  // epilogue.  Nobody waits for anybody.  The eight L2 caches of the device are not coherent with each other:
  // partial sums and counter are written and read as device-scope atomics (relaxed: they go through to the
  // memory side and come from there), the stores are complete before the count, the loads are issued after
  // it.  A release / acquire pair would do the same by writing back and invalidating a whole L2, under every
  // other workgroup still running: 34 -> 88 us on 4096 x 4096 at 512 rows.
  if constexpr (!FUSE) {
    if (sp.splits > 1) {
      constexpr int kPartFloats = MB * NJ * 256;
      const int unit = (m_tile * n_tiles + n_tile) * NC + wave;
      float* all = sp.partials + (size_t)unit * (size_t)(sp.splits * kPartFloats);
      uint64_t* mine = reinterpret_cast<uint64_t*>(all + ksplit * kPartFloats);
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          uint64_t lo, hi;
          const f32x4_t v = acc[i][j];
          lo = (uint64_t)__float_as_uint(v[0]) | ((uint64_t)__float_as_uint(v[1]) << 32);
          hi = (uint64_t)__float_as_uint(v[2]) | ((uint64_t)__float_as_uint(v[3]) << 32);
          uint64_t* q = mine + ((i * NJ + j) * 64 + lane) * 2;
          __hip_atomic_store(q, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(q + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      uint32_t arrived = 0;
      if (lane == 0)
        arrived = __hip_atomic_fetch_add(sp.counters + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      arrived = (uint32_t)__builtin_amdgcn_readfirstlane((int)arrived);
      if (arrived != (uint32_t)(sp.splits - 1)) return;
      asm volatile("" ::: "memory");
      // ready for the next launch on the stream
      if (lane == 0) __hip_atomic_store(sp.counters + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // two copies: the other one is added to the registers (a + b = b + a); more: all in copy order
      const bool two = sp.splits == 2;
      for (int c = two ? 1 - ksplit : 0; c < (two ? 2 - ksplit : sp.splits); c++) {
        const uint64_t* other = reinterpret_cast<const uint64_t*>(all + c * kPartFloats);
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
          for (int j = 0; j < NJ; j++) {
            const uint64_t* q = other + ((i * NJ + j) * 64 + lane) * 2;
            const uint64_t lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint64_t hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const f32x4_t v = {__uint_as_float((uint32_t)lo), __uint_as_float((uint32_t)(lo >> 32)),
                               __uint_as_float((uint32_t)hi), __uint_as_float((uint32_t)(hi >> 32))};
            if (c == 0 && !two) acc[i][j] = v;
            else acc[i][j] += v;
          }
      }
    }
  }

  // ---- epilogue: lane holds Y[m0 + 16i + 4*(lane/16) + r][n0 + 16j + lane%16], r = 0..3
  const int cn = lane & 15, rb4 = (lane >> 4) * 4;
  if constexpr (ROT) {
    static_assert(NJ == 8 && !FUSE, "one Hadamard group of 128 columns per tile");
    // column 16 j + cn: bits 0-3 of the column index live in the lane (DPP moves inside a row of 16 lanes), bits 4-6
    // in the register index j
    float cs[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) cs[j] = 0.08838834764831845f * f16_bits_to_f32(e.col_scale[n0 + 16 * j + cn]);
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        float v[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) v[j] = acc[i][j][r];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          float o;
          o = lane_xor<1>(v[j], lane); v[j] = (cn & 1) ? o - v[j] : v[j] + o;
          o = lane_xor<2>(v[j], lane); v[j] = (cn & 2) ? o - v[j] : v[j] + o;
          o = lane_xor<4>(v[j], lane); v[j] = (cn & 4) ? o - v[j] : v[j] + o;
          o = lane_xor<8>(v[j], lane); v[j] = (cn & 8) ? o - v[j] : v[j] + o;
        }
#pragma unroll
        for (int d = 1; d < NJ; d <<= 1)
#pragma unroll
          for (int j = 0; j < NJ; j++)
            if ((j & d) == 0) {
              const float a = v[j], b = v[j | d];
              v[j] = a + b;
              v[j | d] = a - b;
            }
#pragma unroll
        for (int j = 0; j < NJ; j++) acc[i][j][r] = v[j] * cs[j];
      }
  }
  if constexpr (FUSE) {
    // gate in lanes cn < 8, the matching up eight lanes further; silu(g) * u in fp32, one rounding.
    const bool full = y_dtype == kBF16 && n0 + BO <= n_out && (n_out & 7) == 0;
    constexpr int kRowBytes = BO * 2 + 16;
    uint8_t* stg = e.stg;
    // Column blocks are taken in pairs: lanes cn < 8 finish block j (own gate, up from eight lanes
    // further), lanes cn >= 8 block j+1 (own up, gate from eight lanes back), so that the exp2 and
    // reciprocal -- quarter-rate instructions -- run once per output and not twice.  Both halves
    // write output column n0 + 8j + cn.
#pragma unroll
    for (int j = 0; j < NJ; j += 2) {
      const bool pair = j + 1 < NJ;
      const bool lowhalf = cn < 8;
      const int o = n0 + 8 * j + cn;
      const bool live = lowhalf || pair;
      const int oc = min(o, n_out - 1);
      const float bg = load_bias(bias, bias_dtype, (int64_t)oc);
      const float bu = load_bias(bias, bias_dtype, (int64_t)oc + (int64_t)n_out);
#pragma unroll
      for (int i = 0; i < MB; i++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float a0 = acc[i][j][r];
          const float a1 = pair ? acc[i][j + 1 < NJ ? j + 1 : j][r] : 0.f;
          const float up0 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(a0), 0x108, 0xF, 0xF, false));
          const float gt1 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(a1), 0x118, 0xF, 0xF, false));
          const float g = (lowhalf ? a0 : gt1) + bg;
          const float u = (lowhalf ? up0 : a1) + bu;
          // silu with the hardware exp2 / reciprocal (1 ulp each): the result is rounded to bf16 or
          // is one term of a 2e-2 comparison, and the library versions cost five times as much
          const float res = (g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f))) * u;
          if (live) {
            const int row = 16 * i + rb4 + r;
            if (full) {
              *reinterpret_cast<uint16_t*>(stg + row * kRowBytes + (8 * j + cn) * 2) = f32_to_bf16_bits(res);
            } else if (o < n_out && m0 + row < m) {
              if (y_dtype == kBF16) YElem<bf16_tag>::store(static_cast<bf16_tag*>(yv), (int64_t)(m0 + row) * n_out + o, res);
              else if (y_dtype == kF16) YElem<f16_tag>::store(static_cast<f16_tag*>(yv), (int64_t)(m0 + row) * n_out + o, res);
              else YElem<float>::store(static_cast<float*>(yv), (int64_t)(m0 + row) * n_out + o, res);
            }
          }
        }
      }
    }
    if (full) {
      uint8_t* yb = static_cast<uint8_t*>(yv);
      constexpr int kChunks = BO / 8;      // 16-byte chunks per row
      constexpr int kSlots = 16 * MB * kChunks;
#pragma unroll
      for (int t = 0; t < (kSlots + 63) / 64; t++) {
        const int c = t * 64 + lane;
        const int row = c / kChunks, ch = c - row * kChunks;
        if (c >= kSlots) break;
        const uint4 v = *reinterpret_cast<const uint4*>(stg + row * kRowBytes + ch * 16);
        if (m0 + row < m)
          *reinterpret_cast<uint4*>(yb + ((int64_t)(m0 + row) * n_out + n0 + ch * 8) * 2) = v;
      }
    }
    return;
  }
  if ((y_dtype == kBF16 || ((ROT || e.f16_rows) && y_dtype == kF16)) && n0 + BN <= n_out && (n_out & 7) == 0) {
    // Full tile of bf16: transpose through the wavefront's own (now idle) X ring, so that global
    // memory sees 16-byte stores along the rows instead of 2-byte ones.  Row stride 240 bytes.
    constexpr int kRowBytes = BN * 2 + 16;
    uint8_t* stg = e.stg;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      const float bv = load_bias(bias, bias_dtype, n0 + 16 * j + cn);
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          *reinterpret_cast<uint16_t*>(stg + (16 * i + rb4 + r) * kRowBytes + (16 * j + cn) * 2) =
              ((ROT || e.f16_rows) && y_dtype == kF16) ? f32_to_f16_bits(acc[i][j][r] + bv) : f32_to_bf16_bits(acc[i][j][r] + bv);
    }
    // same wavefront wrote and reads: LDS keeps program order, no barrier needed
    uint8_t* yb = static_cast<uint8_t*>(yv);
    constexpr int kChunks = BN / 8;      // 16-byte chunks per row
    constexpr int kSlots = 16 * MB * kChunks;
#pragma unroll
    for (int t = 0; t < (kSlots + 63) / 64; t++) {
      const int c = t * 64 + lane;
      const int row = c / kChunks, ch = c - row * kChunks;
      if (c >= kSlots) break;
      const uint4 v = *reinterpret_cast<const uint4*>(stg + row * kRowBytes + ch * 16);
      if (m0 + row < m)
        *reinterpret_cast<uint4*>(yb + ((int64_t)(m0 + row) * n_out + n0 + ch * 8) * 2) = v;
    }
    return;
  }
  if constexpr (ROT) {
    if (y_dtype == kF32 && n0 + BN <= n_out && (n_out & 3) == 0) {
      // Full tile of fp32: the same transpose, half of the columns at a time (64 floats and the padding are the 272
      // bytes of a staged row), so that global memory sees 16-byte stores along the rows.
      static_assert(NJ % 2 == 0, "two halves of whole column blocks");
      constexpr int kRowBytes = BN * 2 + 16;
      uint8_t* stg = e.stg;
      uint8_t* yb = static_cast<uint8_t*>(yv);
      constexpr int kChunks = BN / 8;      // 16-byte chunks per half row
      constexpr int kSlots = 16 * MB * kChunks;
#pragma unroll
      for (int p = 0; p < 2; p++) {
#pragma unroll
        for (int jj = 0; jj < NJ / 2; jj++) {
          const int j = p * (NJ / 2) + jj;
          const float bv = load_bias(bias, bias_dtype, n0 + 16 * j + cn);
#pragma unroll
          for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 4; r++)
              *reinterpret_cast<float*>(stg + (16 * i + rb4 + r) * kRowBytes + (16 * jj + cn) * 4) = acc[i][j][r] + bv;
        }
#pragma unroll
        for (int t = 0; t < (kSlots + 63) / 64; t++) {
          const int c = t * 64 + lane;
          const int row = c / kChunks, ch = c - row * kChunks;
          if (c >= kSlots) break;
          const uint4 v = *reinterpret_cast<const uint4*>(stg + row * kRowBytes + ch * 16);
          if (m0 + row < m)
            *reinterpret_cast<uint4*>(yb + ((int64_t)(m0 + row) * n_out + n0 + p * (BN / 2) + ch * 4) * 4) = v;
        }
      }
      return;
    }
  }
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int n = n0 + 16 * j + cn;
    if (n >= n_out) continue;
    const float bv = load_bias(bias, bias_dtype, n);
#pragma unroll
    for (int i = 0; i < MB; i++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int mm = m0 + 16 * i + rb4 + r;
        if (mm < m) {
          const float v = acc[i][j][r] + bv;
          if (y_dtype == kBF16) YElem<bf16_tag>::store(static_cast<bf16_tag*>(yv), (int64_t)mm * n_out + n, v);
          else if (y_dtype == kF16) YElem<f16_tag>::store(static_cast<f16_tag*>(yv), (int64_t)mm * n_out + n, v);
          else YElem<float>::store(static_cast<float*>(yv), (int64_t)mm * n_out + n, v);
        }
      }
    }
  }
}

// 64 k of a producer thread's row (chunk C of the 256 k in `r`), dequantized, rounded to bf16 and stored as B
// fragments into W stage `buf` of the tile at LDS address sw_addr.  whalf / wj / wn: the thread's half of every
// 32-byte chunk, its column block and its column inside the block.
template <int NJ, int FMT, int ABL, int C, class XT = bf16_tag>
__device__ __forceinline__ void pc_dequant_to_lds(const typename WFmt<FMT>::Raw& r, int buf, int whalf, int wj, int wn,
                                                  uint32_t sw_addr) {
  using WF = WFmt<FMT>;
  using WRaw = typename WF::Raw;
  constexpr int kWUnits = 2 * NJ * 64;
  constexpr int c = C;
  uint32_t lo[8], hi[8];
  if constexpr ((ABL & 8) != 0) {
    // ladder: the raw words instead of the dequantized ones
    const uint32_t* raw = reinterpret_cast<const uint32_t*>(&r);
#pragma unroll
    for (int i = 0; i < 8; i++) { lo[i] = raw[(4 * c + i) % (sizeof(WRaw) / 4)]; hi[i] = raw[(4 * c + i + 4) % (sizeof(WRaw) / 4)]; }
  } else {
    WF::template dequant<c, XT>(r, whalf, lo, hi);
  }
  if constexpr ((ABL & 4) != 0) {
    // ladder: no LDS stores; keep the values alive
    uint32_t keep = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) keep ^= lo[i] ^ hi[i];
    asm volatile("" : : "v"(keep));
  } else if constexpr (WF::kWholeKsub) {
    // k = 32*half + e -> ksub `half`, groups 0..3
    const uint32_t base = sw_addr + (uint32_t)(buf * kWUnits + whalf * (NJ * 64) + wj * 64 + wn) * 16u;
    lds_store16(base, lo[0], lo[1], lo[2], lo[3]);
    lds_store16(base + 256u, lo[4], lo[5], lo[6], lo[7]);
    lds_store16(base + 512u, hi[0], hi[1], hi[2], hi[3]);
    lds_store16(base + 768u, hi[4], hi[5], hi[6], hi[7]);
  } else {
    // k = 16*half + e  -> ksub 0, groups 2*half and 2*half+1; k = 32 + 16*half + e: ksub 1
    const uint32_t base = sw_addr + (uint32_t)(buf * kWUnits + (wj * 4 + 2 * whalf) * 16 + wn) * 16u;
    lds_store16(base, lo[0], lo[1], lo[2], lo[3]);
    lds_store16(base + 256u, lo[4], lo[5], lo[6], lo[7]);
    lds_store16(base + NJ * 1024u, hi[0], hi[1], hi[2], hi[3]);
    lds_store16(base + NJ * 1024u + 256u, hi[4], hi[5], hi[6], hi[7]);
  }
}

// The W producer role (wavefronts 4-7 of either kernel): thread pt (0..255) owns one row of the tile and half of
// every 32-byte chunk; it loads the packed blocks, dequantizes 64 k per step and writes the B fragments into the
// double-buffered W tile at LDS address sw_addr, keeping the step barrier `bar`.
template <int NJ, int FMT, bool FUSE, int ABL, class XT = bf16_tag, typename Bar>
__device__ __forceinline__ void pc_produce_w(const uint8_t* __restrict__ w, int pt, int n0, int n_out, int row_blocks,
                                             int block0, int nblocks, uint32_t sw_addr, Bar&& bar) {
  constexpr int BN = NJ * 16;
  constexpr int kWUnits = 2 * NJ * 64;
  // thread -> (tile row, 16-byte half of every 32-byte chunk); with BN = 112 the last 32
  // threads mirror threads 0..31 (same loads, same LDS writes of the same values)
  // (a 64-column tile needs only half of the producer threads: the others just keep the barriers)
  constexpr bool kSpare = 4 * BN <= 256;
  const bool widle = kSpare && pt >= 2 * BN;
  const int wt = pt < 2 * BN ? pt : (kSpare ? pt % (2 * BN) : pt - 2 * BN);
  // the two halves of a row in adjacent lanes: a 64-lane load then touches 32 rows, not 64
  const int wr = wt >> 1, whalf = wt & 1;
  // clamped: rows past the end are never stored
  const int wrow = FUSE ? min(n0 + 8 * (wr >> 4) + (wr & 7), n_out - 1) + ((wr >> 3) & 1) * n_out
                        : min(n0 + wr, n_out - 1);
  using WF = WFmt<FMT>;
  using WRaw = typename WF::Raw;
  const uint8_t* wptr = w + (int64_t)row_blocks * WF::kUnitBytes * (int64_t)wrow + (int64_t)block0 * WF::kUnitBytes;
  const int wj = wr >> 4, wn = wr & 15;
  auto load_w = [&](WRaw& dst, int b) {
    if (widle || (ABL & 16) != 0) return;
    // past the end: a harmless re-read
    WF::load(dst, wptr + WF::kUnitBytes * (int64_t)min(b, nblocks - 1), whalf);
  };
  auto dequant_to_lds = [&](const WRaw& r, auto cc, int buf) {
    if (widle) return;
    pc_dequant_to_lds<NJ, FMT, ABL, decltype(cc)::value, XT>(r, buf, whalf, wj, wn, sw_addr);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // The packed blocks come from HBM (about 2 us away): block b+2 is requested at the
  // start of block b, into the register set block b-1 used.  Three sets rotate by name, so no
  // copy ever forces a request to complete early.  These wavefronts issue no other global
  // loads, so the compiler's own counting of outstanding requests is exact.
  // Iteration s prepares step s+1: chunks 1..3 of block b, then chunk 0 of block b+1.
  auto do_block = [&](const WRaw& cur, const WRaw& nxt, WRaw& into, int b) {
    load_w(into, b + 2);
    dequant_to_lds(cur, I1{}, 1);
    bar();
    dequant_to_lds(cur, I2{}, 0);
    bar();
    dequant_to_lds(cur, I3{}, 1);
    bar();
    dequant_to_lds(nxt, I0{}, 0);      // the chunk written in the very last iteration is never read
    bar();
  };
  WRaw wa{}, wb{}, wc{};
  load_w(wa, 0);
  load_w(wb, 1);
  dequant_to_lds(wa, I0{}, 0);
  bar();                       // barrier -1
  for (int b = 0; b < nblocks; b += 3) {
    do_block(wa, wb, wc, b);
    if (b + 1 < nblocks) do_block(wb, wc, wa, b + 1);
    if (b + 2 < nblocks) do_block(wc, wa, wb, b + 2);
  }
}

// W tile in LDS: [ksub 2][j NJ][g 4][n 16] units of 16 bytes (8 consecutive k of one column),
// i.e. exactly the B operand of lane g*16+n for column block j.
// FUSE: the weight holds gate rows [0, n_out) followed by up rows [n_out, 2*n_out), as GatedMLP
// builds it (workspace/transformers/src/layers/mlp.nim:39), and the kernel writes
// silu(gate . x) * (up . x), the silu_and_mul of
// workspace/transformers/src/kernels/activations.nim:14-38, for n_out outputs.  A tile then covers
// BN / 2 outputs: column 16j + c of the tile is output n0 + 8j + c%8, its gate row for c < 8 and
// its up row for c >= 8, so that a gate value and its up value meet eight lanes apart in the same
// accumulator register.
template <int NJ, int FMT, int MB, bool FUSE, int ABL = 0>
__global__ void __launch_bounds__(kPcThreads)
gemm_pc_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, void* __restrict__ yv,
                   int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                   int n_tiles, int m_tiles, int xcds_per_mtile, PcSplit sp) {
  constexpr int BN = NJ * 16;
  constexpr int kWUnits = 2 * NJ * 64;
  // X reaches LDS through the movers' registers (two LDS stages per consumer; the registers are the lookahead).
  // ABL & 2048 (ladder only): the earlier form, global_load_lds straight into a ring of four stages.
  constexpr bool kXDma = (ABL & 2048) != 0;
  constexpr int kXS = kXDma ? kXStages : 2;
  constexpr int kPcBM = pc_bm(MB), kXStage = pc_xstage(MB), kXRingBytes = 4 * kXS * kXStage;
  constexpr int kDma = 2 * MB;           // 8-row requests per consumer and step
  // two separate arrays, so that the compiler can tell LDS writes to the W tile from the
  // asynchronous global_load_lds writes into the X ring (otherwise it drains every outstanding
  // request before each W write)
  __shared__ __attribute__((aligned(16))) uint8_t smem[kXRingBytes];
  __shared__ uint4 sw[2 * kWUnits];
  __shared__ uint32_t pf_sink[kXDma ? 4 * 64 : 1];   // (DMA form) where the movers' L2 prefetch requests land

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // ladder (ABL & 512): cycles this wavefront spends in all, at the step barrier and (movers) waiting for its
  // requests to land; written to sp.counters[(workgroup * 12 + wavefront) * 4 ...] when the K loop is over
  [[maybe_unused]] uint32_t t_bar = 0, t_vm = 0;
  [[maybe_unused]] const uint64_t t_begin = (ABL & 512) ? __builtin_readcyclecounter() : 0;
  [[maybe_unused]] const uint64_t rt_begin = (ABL & 512) ? __builtin_amdgcn_s_memrealtime() : 0;
  auto bar = [&]() {
    if constexpr ((ABL & 1024) != 0) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // ladder: every role at its own pace (results are garbage)
    } else if constexpr ((ABL & 512) != 0) {
      const uint64_t t0 = __builtin_readcyclecounter();
      lds_barrier();
      t_bar += (uint32_t)(__builtin_readcyclecounter() - t0);
    } else {
      lds_barrier();
    }
  };
  auto trace_out = [&]() {
    if constexpr ((ABL & 512) != 0) {
      if (lane == 0) {
        uint32_t* t = sp.counters + ((size_t)blockIdx.x * 12 + wave) * 4;
        t[0] = (uint32_t)(__builtin_readcyclecounter() - t_begin);
        t[1] = t_bar;
        t[2] = t_vm;
        t[3] = (uint32_t)(__builtin_amdgcn_s_memrealtime() - rt_begin);     // 100 MHz ticks
      }
    }
  };
  // Tile assignment.  Workgroups are dealt to the 8 XCDs round-robin (XCD = id % 8) and every XCD
  // has its own L2.  All workgroups of one row tile read the same 256 x n_in slab of X, so when
  // the row tiles divide the XCDs evenly each XCD is given workgroups of ONE row tile only.
  // Split along K (sp.splits > 1): the grid holds sp.splits copies of the tile grid, copy c works on blocks
  // [c, c + 1) * nblocks of every row and the copies of a tile add up in the epilogue.
  const int ksplit = sp.splits > 1 ? (int)blockIdx.x / sp.tile_wgs : 0;
  const int bid = (int)blockIdx.x - ksplit * sp.tile_wgs;
  int n_tile, m_tile;
  if (xcds_per_mtile > 0) {
    const int xcd = bid & 7, slot = bid >> 3;
    m_tile = xcd / xcds_per_mtile;
    n_tile = slot * xcds_per_mtile + xcd % xcds_per_mtile;
  } else {
    m_tile = bid % m_tiles;
    n_tile = bid / m_tiles;
  }
  if (n_tile >= n_tiles) return;
  constexpr int BO = FUSE ? BN / 2 : BN;     // outputs per tile
  const int n0 = n_tile * BO;
  const int row_blocks = n_in >> 8;                                  // super-blocks (256 k) in a row of W
  const int nblocks = sp.splits > 1 ? row_blocks / sp.splits : row_blocks;   // this workgroup's share of them
  const int block0 = ksplit * nblocks;
  const int ksteps = nblocks * 4;

  if constexpr ((ABL & 4096) != 0) {
    // ladder: real activation values in every LDS stage and W tile, so that a rung whose movers or producers
    // are switched off still multiplies operands that toggle the matrix cores like the real ones do
    const uint4* src = reinterpret_cast<const uint4*>(x);
    uint4* xs = reinterpret_cast<uint4*>(smem);
    const int lim = min(m, 256) * n_in / 8;
    for (int i = tid; i < kXRingBytes / 16; i += kPcThreads) xs[i] = src[(i * 7 + (int)blockIdx.x * 64) % lim];
    for (int i = tid; i < 2 * kWUnits; i += kPcThreads) sw[i] = src[(i * 5 + (int)blockIdx.x * 32 + 4096) % lim];
    __syncthreads();
  }

  // One barrier per 64-k step, numbered s = -1 .. ksteps-1.  Barrier s means: the data of step
  // s+1 is complete in LDS (W buffer (s+1)%2, X stage (s+1)%3) and every LDS read of step s has
  // finished.  The consumers pass it in the MIDDLE of step s (between the MFMAs of the two 32-k
  // halves), the producers after preparing step s+1.

  if (wave >= 8) {
    // ------------------------------------------------------------------ X mover
    const int pc = wave - 8;
    const uint8_t* xb = reinterpret_cast<const uint8_t*>(x);
    uint8_t* ring = smem + pc * (kXS * kXStage);
    if constexpr (!kXDma) {
      // Mover p feeds consumer p.  Request i covers rows 8i .. 8i+7 of the consumer's 16 * MB, lane l the LDS slot
      // (row 8i + l/8, position l%8) and the chunk stored there is position ^ (row & 7): eight consecutive rows
      // then hold a given chunk in eight different 16-byte bank groups.  The rows of step s+3 are requested into
      // one of three register sets while step s+1 moves from its set to LDS stage (s+1) & 1, which the consumer
      // finished reading before barrier s-1.  (Writes to LDS by global_load_lds and by ds_write do not mix:
      // whenever both kinds are in flight on a compute unit the LDS reads of every wavefront stall behind them.)
      uint32_t xoff[kDma];
#pragma unroll
      for (int i = 0; i < kDma; i++) {
        const int rl = 8 * i + (lane >> 3);
        const int row = min(m_tile * kPcBM + pc * (16 * MB) + rl, m - 1);   // clamped: never stored to Y
        xoff[i] = (uint32_t)row * (uint32_t)(n_in * 2) + (uint32_t)(((lane & 7) ^ (rl & 7)) * 16);
      }
      const uint32_t ring_addr = (uint32_t)(size_t)(lptr_t)ring + (uint32_t)lane * 16u;
      // (the activation is smaller than 4 GiB: the launcher checks)
      const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(xb), 0, (int)((uint32_t)m * (uint32_t)(n_in * 2)), 0x00020000);
      struct XSet { uint4 v[kDma]; };
      auto request = [&](XSet& dst, int ks) {
        if constexpr ((ABL & 2) != 0) return;
        // buffer loads: resource + per-lane offset (loop-invariant) + uniform offset of the step, so that a request
        // needs no address arithmetic and no temporary register
        const int koff = (4 * block0 + min(ks, ksteps - 1)) * 128;   // past the end: a harmless re-read
#pragma unroll
        for (int i = 0; i < kDma; i++) {
          const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (int)xoff[i], koff, 0);
          dst.v[i] = make_uint4(v[0], v[1], v[2], v[3]);
        }
      };
      auto to_lds = [&](const XSet& src, int ks) {
        if constexpr ((ABL & 2) != 0) return;
        if (ks >= ksteps) return;           // the consumers reuse their rings in the epilogue
        const uint32_t a = ring_addr + (uint32_t)(ks & 1) * (uint32_t)kXStage;
#pragma unroll
        for (int i = 0; i < kDma; i++) lds_store16(a + i * 1024u, src.v[i].x, src.v[i].y, src.v[i].z, src.v[i].w);
      };
      XSet xa{}, xb_{}, xc{};
      request(xa, 0);
      request(xb_, 1);
      request(xc, 2);
      to_lds(xa, 0);
      bar();                             // barrier -1
      // iteration s: request step s+3 into the set step s used, move step s+1 to LDS
      for (int s3 = 0; s3 < ksteps; s3 += 3) {
        request(xa, s3 + 3);
        to_lds(xb_, s3 + 1);
        bar();                           // barrier s3
        if (s3 + 1 < ksteps) {
          request(xb_, s3 + 4);
          to_lds(xc, s3 + 2);
          bar();
        }
        if (s3 + 2 < ksteps) {
          request(xc, s3 + 5);
          to_lds(xa, s3 + 3);
          bar();
        }
      }
      trace_out();
      return;
    }
    // (ladder only, ABL & 2048) The earlier form: global_load_lds straight into a ring of four stages.  DMA
    // instruction i covers rows 8i .. 8i+7 of the consumer's rows, lane l the LDS slot (row 8i + l/8, position l%8).
    uint32_t xoff[kDma];
#pragma unroll
    for (int i = 0; i < kDma; i++) {
      const int rl = 8 * i + (lane >> 3);
      const int key = rl & 7;
      const int row = min(m_tile * kPcBM + pc * (16 * MB) + rl, m - 1);   // clamped: never stored
      xoff[i] = (uint32_t)row * (uint32_t)(n_in * 2) + (uint32_t)(((lane & 7) ^ key) * 16);
    }
    // L2 prefetch.  All workgroups of an XCD walk the same slab of X in step, so a line that is
    // not in their L2 yet is missed by all of them at once and every one waits out the HBM
    // latency, which is longer than the three stages of lookahead.  Each mover therefore also
    // touches the line (64 k of one row = 128 bytes) of its consumer's 64 rows kPf steps ahead,
    // as one 4-byte request per lane into a scratch LDS word: no register, nothing to wait for.
    constexpr int kPf = 8;
    constexpr int kPfReq = 1;                    // prefetch requests per step
    const uint8_t* pf_row =
        xb + (size_t)min(m_tile * kPcBM + pc * (16 * MB) + (lane & (16 * MB - 1)), m - 1) * (size_t)(n_in * 2);
    auto dma_step = [&](int ks, int stage) {
      if constexpr ((ABL & 2) != 0) return;
      const uint32_t koff = (uint32_t)(4 * block0 + ks) * 128u;
#pragma unroll
      for (int i = 0; i < kDma; i++)
        __builtin_amdgcn_global_load_lds((gptr_t)(xb + (size_t)(xoff[i] + koff)),
                                         (lptr_t)(ring + stage * kXStage + i * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(pf_row + (size_t)(4 * block0 + min(ks + kPf, ksteps - 1)) * 128),
                                         (lptr_t)(pf_sink + pc * 64), 4, 0, 0);
    };
    // Requests complete in order, so "all but the youngest N have landed" is the only wait there
    // is.  A step is kDma data requests and one prefetch.  Iteration s requests step s+3
    // into the stage that barrier s-1 freed and then makes sure step s+1 has landed: the
    // prefetch that followed it and steps s+2, s+3 (2 * (kDma + 1) + 1 requests) may stay in flight.
    // Nothing is requested past the last step: the consumers reuse their rings in the epilogue.
    dma_step(0, 0);
    dma_step(1, 1);
    dma_step(2, 2);
    wait_vmcnt<2 * (kDma + kPfReq) + kPfReq>();
    bar();                       // barrier -1
    int st = 3;
    for (int s2 = 0; s2 < ksteps - 3; s2++) {
      dma_step(s2 + 3, st);
      st = (st + 1) & (kXStages - 1);
      if constexpr ((ABL & 512) != 0) {
        const uint64_t t0 = __builtin_readcyclecounter();
        wait_vmcnt<2 * (kDma + kPfReq) + kPfReq>();
        t_vm += (uint32_t)(__builtin_readcyclecounter() - t0);
      } else {
        wait_vmcnt<2 * (kDma + kPfReq) + kPfReq>();
      }
      bar();                     // barrier s
    }
    wait_vmcnt<kDma + 2 * kPfReq>();
    bar();                       // barrier ksteps-3: step ksteps-2 has landed
    wait_vmcnt<0>();
    bar();                       // barrier ksteps-2: the last step has landed
    bar();                       // barrier ksteps-1
    trace_out();
    return;
  }

  if (wave >= 4) {
    // ------------------------------------------------------------------ W producer
    pc_produce_w<NJ, FMT, FUSE, ABL>(w, tid - 256, n0, n_out, row_blocks, block0, nblocks,
                                     (uint32_t)(size_t)(lptr_t)(&sw[0]), bar);
    trace_out();
    return;
  }

  // -------------------------------------------------------------------- consumer
  const int m0 = m_tile * kPcBM + wave * (16 * MB);
  const uint8_t* myx = smem + wave * (kXS * kXStage);
  const int fr = lane & 15, fg = lane >> 4;
  // A fragments: row 16*ib + fr, chunk 4*half + fg, stored at position chunk ^ key(row)
  const int akey = fr & 7;
  const int apos[2] = {(fr * 8 + (fg ^ akey)) * 16, (fr * 8 + ((4 + fg) ^ akey)) * 16};
  // A step is 2*NJ groups of four MFMAs: group g uses the A fragments of half g/NJ (four row
  // blocks) and the B fragment of column block g%NJ.  B fragments are read two groups ahead
  // into a ring of four, A fragments half a step ahead, and __builtin_amdgcn_sched_barrier
  // pins that order: left alone the compiler sinks every read to just before its use and the
  // wavefront then waits out the LDS latency fourteen times per step.
  constexpr int G = 2 * NJ;
  uint4 afr[2][MB];                     // A fragments of half 0 / half 1
  bf16x8_t bring[4];
  auto read_a = [&](uint4 (&dst)[MB], int stage, int half) {
    const uint8_t* xbase = myx + stage * kXStage + apos[half];
#pragma unroll
    for (int ib = 0; ib < MB; ib++) dst[ib] = *reinterpret_cast<const uint4*>(xbase + ib * 2048);
  };
  auto read_b = [&](bf16x8_t& dst, int buf, int g) {   // g = half * NJ + j
    const uint4 v = sw[buf * kWUnits + g * 64 + lane];
    __builtin_memcpy(&dst, &v, 16);
  };

  f32x4_t acc[MB][NJ];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // one step; everything that selects a buffer is a compile-time constant, so that every LDS
  // address is one register plus an immediate.  SO = ring slot of the step's group 0: 2*NJ is
  // not always a multiple of four, and the first two groups of the next step are read while
  // the last two of this one still hold their slots.
  auto step = [&](auto so, auto stage, auto bufc) {
    constexpr int SO = decltype(so)::value, ST = decltype(stage)::value, BUF = decltype(bufc)::value;
    constexpr int STN = (ST + 1) & (kXS - 1);
    if constexpr ((ABL & 1) != 0) { bar(); return; }
#pragma unroll
    for (int g = 0; g < G; g++) {
      if (g == G - 2) bar();     // barrier ks: step ks+1 is in LDS, reads of step ks done
      if (g + 2 < G) read_b(bring[(g + 2 + SO) & 3], BUF, g + 2);
      else read_b(bring[(g + 2 + SO) & 3], BUF ^ 1, g + 2 - G);
      if (g == (NJ > 3 ? NJ - 3 : 0)) read_a(afr[1], ST, 1);
      if (g == G - 2) read_a(afr[0], STN, 0);
      __builtin_amdgcn_sched_barrier(0);
      const int half = g / NJ, j = g % NJ;
#pragma unroll
      for (int i = 0; i < MB; i++) {
        bf16x8_t a;
        __builtin_memcpy(&a, &afr[half][i], 16);
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bring[(g + SO) & 3], acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  bar();                         // barrier -1: step 0 is in LDS
  read_a(afr[0], 0, 0);
  read_b(bring[0], 0, 0);
  read_b(bring[1], 0, 1);
  static_assert(kXStages == 4, "the step loop is unrolled over the four X stages");
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  for (int ks = 0; ks < ksteps; ks += 4) {   // ksteps is a multiple of four
    step(std::integral_constant<int, 0>{}, C0{}, C0{});
    step(std::integral_constant<int, (G & 3)>{}, C1{}, C1{});
    step(std::integral_constant<int, ((2 * G) & 3)>{}, std::integral_constant<int, (2 & (kXS - 1))>{}, C0{});
    step(std::integral_constant<int, ((3 * G) & 3)>{}, std::integral_constant<int, (3 & (kXS - 1))>{}, C1{});   // after the last step: stale reads, never used
  }
  trace_out();

  pc_epilogue<NJ, MB, FUSE>(acc, PcEpi{sp, ksplit, m_tile, n_tile, n_tiles, wave, lane,
                                       smem + wave * (kXS * kXStage), yv, y_dtype, bias, bias_dtype, m, n_out, n0, m0});
}

// The caller owns the split-K workspace: sp.splits == 1 (no partials, no counters) or a prepared PcSplit whose
// tile_wgs this function fills in.
template <int FMT, int MB, int NJ, bool FUSE, int ABL = 0>
static hipError_t launch_pc_grid(const uint8_t* wb, const uint16_t* x, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp, hipStream_t s) {
  constexpr int BO = FUSE ? NJ * 8 : NJ * 16, BM = pc_bm(MB);
  const int n_tiles = (int)((n_out + BO - 1) / BO), m_tiles = (int)((m + BM - 1) / BM);
  int xcds_per_mtile = 0;
  unsigned nwg = (unsigned)(n_tiles * m_tiles);
  if (m_tiles >= 2 && m_tiles <= 8 && 8 % m_tiles == 0) {
    xcds_per_mtile = 8 / m_tiles;
    nwg = (unsigned)(((n_tiles + xcds_per_mtile - 1) / xcds_per_mtile) * 8);
  }
  sp.tile_wgs = (int)nwg;
  hipLaunchKernelGGL((gemm_pc_kernel<NJ, FMT, MB, FUSE, ABL>), dim3(nwg * (unsigned)sp.splits), dim3(kPcThreads), 0, s, wb,
                     x, y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles, xcds_per_mtile, sp);
  return hipGetLastError();
}

}  // namespace ttq
