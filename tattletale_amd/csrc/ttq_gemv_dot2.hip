// Decode GEMV fast path for 16-bit activations (bf16 / fp16) on gfx950: packed dot products.
//
// Same operator as ttq_gemv.hip (F.linear with a single-token activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81), different arithmetic:
// the activations stay 16-bit, packed two to a register, and the quantized integers are
// turned into 16-bit floats with ONE and-or each, using the fact that OR-ing a small
// integer q into the mantissa of a suitable power of two gives an exact float:
//       bf16:  0x4300 | q  ==  128 + q      (q < 128)
//       fp16:  0x6400 | q  ==  1024 + q     (q < 1024)
// v_dot2_f32_{bf16,f16} then multiplies two weights by two activations per instruction
// and accumulates in fp32; the constant offset is removed with a per-lane sum of the
// activations (computed once, the activations never change from row to row):
//       sum (OFF + q) x  -  OFF * sum x  =  sum q x.
// Scales are applied once per sub-block, so a unit-vector activation still reproduces
// the canonical dequantized weight exactly.
//
// Work distribution.  Lane l always owns unit l (mod 64) of a row (a unit = 64 weights),
// so when a row has at most 64 units the lane's 32 activation registers are loaded once.
// Each wavefront owns a contiguous range of rows and walks it in batches of four rows,
// double-buffered: the 16-byte loads of the next batch are in flight while the current
// batch is unpacked, so HBM never waits for the ALUs.  The first batch is requested
// before the activations are staged, hiding that latency too.
#include "ttq_device.h"
#include "ttq_internal.h"

#include <stdlib.h>

namespace ttq {

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

struct OpsBF16 {
  static constexpr uint32_t kMagic = 0x43004300u;   // (128.0, 128.0)
  static constexpr float kOffset = 128.f;
  static constexpr uint32_t kOnes = 0x3F803F80u;    // (1.0, 1.0)
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    bf16x2_t x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(x, y, c, false);
  }
};
struct OpsF16 {
  static constexpr uint32_t kMagic = 0x64006400u;   // (1024.0, 1024.0)
  static constexpr float kOffset = 1024.f;
  static constexpr uint32_t kOnes = 0x3C003C00u;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    f16x2_t x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_fdot2(x, y, c, false);
  }
};

// (v & mask) | magic is a single v_and_or_b32 when `magic` lives in a VGPR (the instruction
// takes no literal and only one scalar operand; with two literals the compiler falls back to
// v_and + v_or).  opaque_vgpr() pins a constant into a VGPR without emitting anything.
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t magic_vgpr) {
  return (v & mask) | magic_vgpr;
}

// Sum over the 64 lanes with DPP adds; the total lands in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
  return v + __int_as_float(moved);
}
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v = dpp_add<0xB1, 0xF>(v);    // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);    // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xF>(v);   // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);   // row_mirror: every lane holds its row's sum
  v = dpp_add<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

// Developer timeline instrumentation, compiled in only with -DTTQ_PHASE_TRACE: lane 0 of every
// wavefront stores the 100 MHz real-time counter at a few phase boundaries.
#ifdef TTQ_PHASE_TRACE
__device__ unsigned long long* g_phase_trace = nullptr;
#define TTQ_TRACE_POINT(wave_id, slot)                                                          \
  do {                                                                                          \
    if (g_phase_trace != nullptr && (threadIdx.x & 63) == 0)                                    \
      g_phase_trace[(size_t)(wave_id) * 8 + (slot)] = __builtin_amdgcn_s_memrealtime();         \
  } while (0)
#else
#define TTQ_TRACE_POINT(wave_id, slot) do { } while (0)
#endif

constexpr int kFastThreads = 512;
constexpr int kStageChunk = kFastThreads * 8;   // activations staged per pass of the workgroup
constexpr int kFastWaves = kFastThreads / kWave;
constexpr int kBatch = 4;     // rows per pass when activations are re-read from LDS
constexpr int kRing = 4;      // row buffers per wavefront when activations sit in registers
constexpr int kEarlyRows = 1; // rows requested before the activations are staged
constexpr int kLongRing = 6;  // unit-group buffers per wavefront on the long-row path
constexpr int kLongEarly = 2; // of them requested before the activations are staged

// LDS slot (dword) of activation-pair register `reg` of unit u: [u/64][reg/4][u%64][reg%4]
__device__ __forceinline__ int xpair_slot(int u, int reg) {
  return ((((u >> 6) * 8 + (reg >> 2)) * 64 + (u & 63)) << 2) + (reg & 3);
}

// Pairs (x0,x2), (x1,x3), (x4,x6), (x5,x7) of eight consecutive 16-bit activations
__device__ __forceinline__ void make_pairs(const uint4& v, uint2& p0, uint2& p1) {
  p0.x = (v.x & 0xFFFFu) | (v.y << 16);
  p0.y = (v.x >> 16) | (v.y & 0xFFFF0000u);
  p1.x = (v.z & 0xFFFFu) | (v.w << 16);
  p1.y = (v.z >> 16) | (v.w & 0xFFFF0000u);
}

// -------------------------------------------------------------------------------- Q4_K
// unit u = (super-block u/4, chunk c = u%4): 32 qs bytes; low nibbles -> sub-block 2c,
// high nibbles -> sub-block 2c+1.  Activation pairs of a unit, register 4i+kind for qs dword
// i: kind 0 = (x[4i], x[4i+2]), 1 = (x[4i+1], x[4i+3]), 2/3 = the same 32 positions further.
struct DotQ4K {
  static constexpr int kSums = 2;
  static __device__ __forceinline__ int64_t row_bytes(int n_in) { return (int64_t)(n_in >> 8) * 144; }
  static constexpr uint32_t kGroupBytes = 16 * 144;   // 64 units
  struct Raw { uint4 hdr, q0, q1; };

  // Per-lane constants.  A lane always decodes chunk c = lane % 4, so the bit positions of its
  // two 6-bit scales and mins inside the 12 packed bytes never change: sub-blocks 0..3 keep
  // the whole field in bytes 0..7, sub-blocks 4..7 keep 4 bits in bytes 8..11 and 2 bits on top
  // of bytes 0..7.  Written as two bit-field extracts (the second with width 0 for the simple
  // case) so that no branch is needed.
  struct Lane {
    uint32_t off_hdr, off_q;        // byte offsets of the header and the 32 qs bytes in the row
    bool upper;                     // sub-blocks 4..7
    uint32_t wl, wh;                // widths of the low and the high part
    uint32_t sc_lo[2], mn_lo[2], hi[2];  // bit offsets, for sub-blocks 2c and 2c+1
    __device__ __forceinline__ void init(int u) {
      const int c = u & 3;
      off_hdr = 144u * (uint32_t)(u >> 2);
      off_q = off_hdr + 16u + 32u * (uint32_t)c;
      upper = c >= 2;
      wl = upper ? 4u : 6u;
      wh = upper ? 2u : 0u;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const uint32_t j = 2u * c + h, jj = j & 3u;
        sc_lo[h] = 8u * jj;
        mn_lo[h] = upper ? 8u * jj + 4u : 8u * jj;
        hi[h] = 8u * jj + 6u;
      }
    }
  };

  // `keep` is all ones for a real row and zero for a row past the end (every lane then reads
  // the first bytes of a valid row: one harmless cache line)
  static __device__ __forceinline__ void fetch(Raw& r, const uint8_t* rp, const Lane& L, uint32_t keep) {
    r.hdr = load16_a16(rp + (L.off_hdr & keep));
    r.q0 = load16_a16(rp + (L.off_q & keep));
    r.q1 = load16_a16(rp + ((L.off_q + 16) & keep));
  }

  // thread holds x[k0 .. k0+8): unit k0/64, qs dwords i0 = (k0 % 32) / 4 and i0 + 1
  static __device__ __forceinline__ void stage(uint32_t* xs, int k0, const uint4& v) {
    const int u = k0 >> 6, o = k0 & 63;
    const int kbase = (o >> 5) << 1;          // kinds 0/1 for the low half, 2/3 for the high
    const int i0 = (o & 31) >> 2;
    uint2 p0, p1;
    make_pairs(v, p0, p1);
    *reinterpret_cast<uint2*>(&xs[xpair_slot(u, 4 * i0 + kbase)]) = p0;
    *reinterpret_cast<uint2*>(&xs[xpair_slot(u, 4 * (i0 + 1) + kbase)]) = p1;
  }

  template <class Ops>
  static __device__ __forceinline__ void sums(const uint32_t (&xr)[32], float (&sx)[kSums]) {
    float a = 0.f, b = 0.f, c = 0.f, d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      a = Ops::dot2(xr[4 * i + 0], Ops::kOnes, a);
      b = Ops::dot2(xr[4 * i + 1], Ops::kOnes, b);
      c = Ops::dot2(xr[4 * i + 2], Ops::kOnes, c);
      d = Ops::dot2(xr[4 * i + 3], Ops::kOnes, d);
    }
    sx[0] = a + b;
    sx[1] = c + d;
  }

  // Dot product of one unit (64 weights) with the lane's activations; off = kOffset * sx.
  template <class Ops>
  static __device__ __forceinline__ float unit_dot(const Raw& r, const Lane& L, const uint32_t (&xr)[32],
                                                   const float (&sx)[kSums], const float (&off)[kSums],
                                                   uint32_t magic) {
    const uint32_t dw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
    constexpr uint32_t M = 0x000F000Fu;
    float s1a = 0.f, s1b = 0.f, s2a = 0.f, s2b = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t q = dw[i];
      s1a = Ops::dot2(and_or(q, M, magic), xr[4 * i + 0], s1a);
      s1b = Ops::dot2(and_or(q >> 8, M, magic), xr[4 * i + 1], s1b);
      s2a = Ops::dot2(and_or(q >> 4, M, magic), xr[4 * i + 2], s2a);
      s2b = Ops::dot2(and_or(q >> 12, M, magic), xr[4 * i + 3], s2b);
    }
    const float q1 = (s1a + s1b) - off[0];   // sum q*x over sub-block 2c
    const float q2 = (s2a + s2b) - off[1];   // sub-block 2c+1
    const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    const uint32_t a_sc = L.upper ? r.hdr.w : r.hdr.y;   // bytes 8-11 or 0-3
    const uint32_t a_mn = L.upper ? r.hdr.w : r.hdr.z;   // bytes 8-11 or 4-7
    const uint32_t sc1 = __builtin_amdgcn_ubfe(a_sc, L.sc_lo[0], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.y, L.hi[0], L.wh) << 4);
    const uint32_t sc2 = __builtin_amdgcn_ubfe(a_sc, L.sc_lo[1], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.y, L.hi[1], L.wh) << 4);
    const uint32_t mn1 = __builtin_amdgcn_ubfe(a_mn, L.mn_lo[0], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.z, L.hi[0], L.wh) << 4);
    const uint32_t mn2 = __builtin_amdgcn_ubfe(a_mn, L.mn_lo[1], L.wl) | (__builtin_amdgcn_ubfe(r.hdr.z, L.hi[1], L.wh) << 4);
    const float t1 = (d * (float)sc1) * q1 - (dmin * (float)mn1) * sx[0];
    const float t2 = (d * (float)sc2) * q2 - (dmin * (float)mn2) * sx[1];
    return t1 + t2;
  }
};

// -------------------------------------------------------------------------------- Q6_K
// unit u = 4b + 2h + s of block b: the 64 weights 128h + 32j + 16s + i (j = 0..3, i = 0..15).
// They come from 16 bytes of ql (low nibbles: j = 0, high: j = 2), the 16 bytes 32 further
// (j = 1, 3) and 16 bytes of qh (2 bits per j).  Four bytes of each give one dword of four
// 6-bit values per j; (Q & 0x00FF00FF) | magic and ((Q >> 8) & 0x00FF00FF) | magic turn it into
// two float pairs.  Register 8j + 2d + parity holds (x[16j+4d+parity], x[16j+4d+parity+2]).
// The weights are q - 32 and the magic adds 128 (bf16) or 1024 (fp16): the offset removed per j
// is (kOffset + 32) * sum(x).
struct DotQ6K {
  static constexpr int kSums = 4;
  static __device__ __forceinline__ int64_t row_bytes(int n_in) { return (int64_t)(n_in >> 8) * 210; }
  static constexpr uint32_t kGroupBytes = 16 * 210;   // 64 units
  struct Raw { uint4 a, b, h; uint2 sc; uint32_t d; };
  struct Lane {
    uint32_t off_a, off_h, off_sc, off_d;
    uint32_t sbit;   // 8*s: bit offset of the lane's first scale byte inside each scale dword
    __device__ __forceinline__ void init(int u) {
      const uint32_t blk = 210u * (uint32_t)(u >> 2);
      const uint32_t h = (u >> 1) & 1, s = u & 1;
      off_a = blk + 64u * h + 16u * s;
      off_h = blk + 128u + 32u * h + 16u * s;
      off_sc = blk + 192u + 8u * h;
      off_d = blk + 208u;
      sbit = 8u * s;
    }
  };
  static __device__ __forceinline__ void fetch(Raw& r, const uint8_t* rp, const Lane& L, uint32_t keep) {
    r.a = load16_a2(rp + (L.off_a & keep));
    r.b = load16_a2(rp + ((L.off_a + 32) & keep));
    r.h = load16_a2(rp + (L.off_h & keep));
    uint2 sc;
    __builtin_memcpy(&sc, __builtin_assume_aligned(rp + (L.off_sc & keep), 2), 8);
    r.sc = sc;
    r.d = load2(rp + (L.off_d & keep));
  }
  // thread holds x[k0 .. k0+8): block, half, j, s and the dwords d0 = (k0 % 16) / 4, d0 + 1
  static __device__ __forceinline__ void stage(uint32_t* xs, int k0, const uint4& v) {
    const int b = k0 >> 8, r = k0 & 255;
    const int h = r >> 7, j = (r >> 5) & 3, s = (r >> 4) & 1, d0 = (r & 15) >> 2;
    const int u = 4 * b + 2 * h + s;
    uint2 p0, p1;
    make_pairs(v, p0, p1);
    *reinterpret_cast<uint4*>(&xs[xpair_slot(u, 8 * j + 2 * d0)]) = make_uint4(p0.x, p0.y, p1.x, p1.y);
  }
  template <class Ops>
  static __device__ __forceinline__ void sums(const uint32_t (&xr)[32], float (&sx)[kSums]) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        a = Ops::dot2(xr[8 * j + 2 * i], Ops::kOnes, a);
        b = Ops::dot2(xr[8 * j + 2 * i + 1], Ops::kOnes, b);
      }
      sx[j] = a + b;
    }
  }
  template <class Ops>
  static __device__ __forceinline__ float unit_dot(const Raw& r, const Lane& L, const uint32_t (&xr)[32],
                                                   const float (&sx)[kSums], const float (&off)[kSums],
                                                   uint32_t magic) {
    const uint32_t A[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
    const uint32_t B[4] = {r.b.x, r.b.y, r.b.z, r.b.w};
    const uint32_t H[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
    constexpr uint32_t N4 = 0x0F0F0F0Fu, H2 = 0x30303030u, M = 0x00FF00FFu;
    float acc[4][2];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j][0] = acc[j][1] = 0.f;
#pragma unroll
    for (int d = 0; d < 4; d++) {
      uint32_t Q[4];
      Q[0] = (A[d] & N4) | ((H[d] << 4) & H2);
      Q[1] = (B[d] & N4) | ((H[d] << 2) & H2);
      Q[2] = ((A[d] >> 4) & N4) | (H[d] & H2);
      Q[3] = ((B[d] >> 4) & N4) | ((H[d] >> 2) & H2);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        acc[j][0] = Ops::dot2(and_or(Q[j], M, magic), xr[8 * j + 2 * d], acc[j][0]);
        acc[j][1] = Ops::dot2(and_or(Q[j] >> 8, M, magic), xr[8 * j + 2 * d + 1], acc[j][1]);
      }
    }
    const float dd = f16_bits_to_f32((uint16_t)r.d);
    // scale bytes s, s+2 of the low dword (j = 0, 1) and of the high dword (j = 2, 3)
    const float c0 = (float)(int)__builtin_amdgcn_sbfe((int)r.sc.x, L.sbit, 8);
    const float c1 = (float)(int)__builtin_amdgcn_sbfe((int)r.sc.x, L.sbit + 16, 8);
    const float c2 = (float)(int)__builtin_amdgcn_sbfe((int)r.sc.y, L.sbit, 8);
    const float c3 = (float)(int)__builtin_amdgcn_sbfe((int)r.sc.y, L.sbit + 16, 8);
    const float t0 = (dd * c0) * ((acc[0][0] + acc[0][1]) - off[0]);
    const float t1 = (dd * c1) * ((acc[1][0] + acc[1][1]) - off[1]);
    const float t2 = (dd * c2) * ((acc[2][0] + acc[2][1]) - off[2]);
    const float t3 = (dd * c3) * ((acc[3][0] + acc[3][1]) - off[3]);
    return (t0 + t1) + (t2 + t3);
  }
  static constexpr float kExtraOffset = 32.f;
};

template <class F> struct ExtraOffset { static constexpr float value = 0.f; };
template <> struct ExtraOffset<DotQ6K> { static constexpr float value = 32.f; };

__device__ __forceinline__ void load_x_regs(const uint32_t* xs, int it, int lane, uint32_t (&xr)[32]) {
  const uint4* xs4 = reinterpret_cast<const uint4*>(xs);
#pragma unroll
  for (int r = 0; r < 8; r++) {
    const uint4 v = xs4[(it * 8 + r) * 64 + lane];
    xr[4 * r] = v.x; xr[4 * r + 1] = v.y; xr[4 * r + 2] = v.z; xr[4 * r + 3] = v.w;
  }
}

// BIG: rows of more than 32768 values (16 staging passes instead of 8; shorter rows keep the form with half the
// staging registers).
template <class F, class Ops, typename YT, bool XREG, bool BIG = false>
__global__ void __launch_bounds__(kFastThreads)
gemv_dot2_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                 const void* __restrict__ bias, int bias_dtype, int n_out, int n_in, int rows_per_wave,
                 int flat) {
  extern __shared__ uint32_t xs[];
  const int tid = threadIdx.x, lane = tid & 63;
  // the wave index is the same in all 64 lanes: keep it (and every row address) scalar
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint16_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const int units = n_in >> 6;
  const int nit = (units + 63) >> 6;
  const int64_t rb = F::row_bytes(n_in);

  const int gw = blockIdx.x * kFastWaves + wave;
  TTQ_TRACE_POINT(gw, 0);
  const int row0 = gw * rows_per_wave;
  const int row_end = min(row0 + rows_per_wave, n_out);
  const int last = n_out - 1;

  // lanes beyond the last unit of a short row read unit 0 and are given zero activations
  const bool active = lane < units;
  typename F::Lane L;
  L.init(active ? lane : 0);

  typename F::Raw ring[XREG ? kRing : kLongRing];

  // Long rows, flat order: the wavefront's work is the sequence of items (row, group of 64 units),
  // row by row.  next_item() requests the next one (items past the end fetch one harmless line,
  // so that the compiler's load counting stays exact).  A lane whose unit lies beyond the row's
  // last one reads its unit of group 0 instead (valid packed bytes; its activations are zero).
  int f_row = row0, f_it = 0;
  auto next_item = [&](typename F::Raw& dst) {
    const bool valid = f_row < row_end;
    const uint32_t group = (f_it * 64 + lane < units) ? (uint32_t)f_it * F::kGroupBytes : 0u;
    F::fetch(dst, w + rb * (valid ? f_row : min(row0, last)) + (valid ? group : 0u), L, valid ? 0xFFFFFFFFu : 0u);
    if (++f_it == nit) { f_it = 0; f_row++; }
  };

  // stage x as permuted pairs: one 16-byte load (8 activations) per thread and pass,
  // all passes requested before the first is consumed
  {
    constexpr int kMaxChunks = XREG ? 1 : (int)((BIG ? kMaxGemvIn16 : kMaxGemvIn16 / 2) / kStageChunk);
    uint4 xv[kMaxChunks];
#pragma unroll
    for (int ch = 0; ch < kMaxChunks; ch++) {
      // unconditional loads from a clamped address keep the control flow straight, so the
      // compiler can wait for exactly these loads and not for the weight loads behind them
      const int k0 = ch * kStageChunk + 8 * tid;
      const bool ok = k0 < n_in;
      const uint4 v = *reinterpret_cast<const uint4*>(xm + (ok ? k0 : 0));
      xv[ch] = ok ? v : make_uint4(0, 0, 0, 0);
    }
    // XREG: request the first kEarlyRows rows right behind the activations and the rest of the
    // ring only once x is staged.  Under a full-rate weight stream every request waits in
    // queues as deep as the bytes already asked for, so x must not be asked for behind a
    // whole batch; a bare s_barrier (no memory wait) also makes sure every wavefront's x request
    // is queued before any weight request of this workgroup.  The weight loads are
    // unconditional and clamped to the last row, to keep the control flow straight.
    if constexpr (XREG) {
      __builtin_amdgcn_s_barrier();
#pragma unroll
      for (int r = 0; r < kEarlyRows; r++) F::fetch(ring[r], w + rb * min(row0 + r, last), L, 0xFFFFFFFFu);
    } else if (flat) {
      __builtin_amdgcn_s_barrier();
#pragma unroll
      for (int r = 0; r < kLongEarly; r++) next_item(ring[r]);
    }
#pragma unroll
    for (int ch = 0; ch < kMaxChunks; ch++) {
      const int k0 = ch * kStageChunk + 8 * tid;
      if (k0 < nit * 4096) F::stage(xs, k0, xv[ch]);
    }
  }
  __syncthreads();
  TTQ_TRACE_POINT(gw, 1);
  // wavefronts without rows fall through: their loads are clamped and their stores masked

  const uint32_t magic = opaque_vgpr(Ops::kMagic);
  constexpr float kOff = Ops::kOffset + ExtraOffset<F>::value;
  auto store_rows = [&](auto& acc, int base) {
    constexpr int kN = (int)(sizeof(acc) / sizeof(float));
#pragma unroll
    for (int r = 0; r < kN; r++) acc[r] = wave_sum_to_lane63(acc[r]);
    if (lane == 63) {
#pragma unroll
      for (int r = 0; r < kN; r++) {
        const int row = base + r;
        if (row < row_end) YElem<YT>::store_through(ym, row, acc[r] + load_bias(bias, bias_dtype, row));
      }
    }
  };

  if constexpr (XREG) {
    uint32_t xr[32];
    float sx[F::kSums], off[F::kSums];
    load_x_regs(xs, 0, lane, xr);
    F::template sums<Ops>(xr, sx);
#pragma unroll
    for (int i = 0; i < F::kSums; i++) off[i] = kOff * sx[i];
    TTQ_TRACE_POINT(gw, 2);

    // Row-granular software pipeline over a ring of kRing row buffers: while row r is unpacked,
    // rows r+1 .. r+kRing-1 are in flight (loads return in request order).  Keeping only a few
    // rows in flight per wavefront matters: asking for everything at once fills the memory
    // queues so deeply that issuing the requests itself stalls the wavefront for microseconds.
    // Loads are always issued (rows past the end fetch one harmless line) so that the
    // compiler's load counting stays exact; only the arithmetic is skipped.
    auto fetch = [&](typename F::Raw& dst, int row) {
      const bool valid = row < row_end;
      F::fetch(dst, w + rb * (valid ? row : min(row0, last)), L, valid ? 0xFFFFFFFFu : 0u);
    };
#pragma unroll
    for (int r = kEarlyRows; r < kRing - 1; r++) fetch(ring[r], row0 + r);
    for (int base = row0; base < row_end; base += kRing) {
      float acc[kRing];
#pragma unroll
      for (int i = 0; i < kRing; i++) {
        fetch(ring[(i + kRing - 1) % kRing], base + i + kRing - 1);
        acc[i] = 0.f;
        if (base + i < row_end) acc[i] = F::template unit_dot<Ops>(ring[i], L, xr, sx, off, magic);
      }
      store_rows(acc, base);
    }
    TTQ_TRACE_POINT(gw, 5);
  } else {
    // long rows: activations come from LDS for every unit
    if (flat) {
      // The per-group activation sums do not depend on the row: each wavefront works out a share
      // of them once, into LDS behind the staged pairs ([group][sum][lane]).
      float* xsum = reinterpret_cast<float*>(xs + nit * 2048);
      for (int it = wave; it < nit; it += kFastWaves) {
        uint32_t xr[32];
        float sx[F::kSums];
        load_x_regs(xs, it, lane, xr);
        F::template sums<Ops>(xr, sx);
#pragma unroll
        for (int i = 0; i < F::kSums; i++) xsum[(it * F::kSums + i) * 64 + lane] = sx[i];
      }
      __syncthreads();
      // Ring of kLongRing items: while one is unpacked the next kLongRing-1 are in flight.
#pragma unroll
      for (int r = kLongEarly; r < kLongRing - 1; r++) next_item(ring[r]);
      int c_row = row0, c_it = 0;
      float acc1[1] = {0.f};
      while (c_row < row_end) {
#pragma unroll
        for (int i = 0; i < kLongRing; i++) {
          next_item(ring[(i + kLongRing - 1) % kLongRing]);
          if (c_row < row_end) {
            uint32_t xr[32];
            float sx[F::kSums], off[F::kSums];
            load_x_regs(xs, c_it, lane, xr);
#pragma unroll
            for (int k = 0; k < F::kSums; k++) {
              sx[k] = xsum[(c_it * F::kSums + k) * 64 + lane];
              off[k] = kOff * sx[k];
            }
            acc1[0] += F::template unit_dot<Ops>(ring[i], L, xr, sx, off, magic);
            if (++c_it == nit) {
              store_rows(acc1, c_row);
              acc1[0] = 0.f;
              c_it = 0;
              c_row++;
            }
          }
        }
      }
      return;
    }
    if (row_end - row0 < kBatch) {
      // fewer rows than a batch (many CUs, few rows each): the batch runs along the row instead,
      // kBatch groups of 64 units requested together
      for (int row = row0; row < row_end; row++) {
        float acc1[1] = {0.f};
        for (int it0 = 0; it0 < nit; it0 += kBatch) {
          typename F::Raw buf[kBatch];
          typename F::Lane Ls[kBatch];
#pragma unroll
          for (int j = 0; j < kBatch; j++) {
            const int u = min(it0 + j, nit - 1) * 64 + lane;
            Ls[j].init(u < units ? u : 0);
            F::fetch(buf[j], w + rb * row, Ls[j], 0xFFFFFFFFu);
          }
#pragma unroll
          for (int j = 0; j < kBatch; j++) {
            if (it0 + j < nit) {
              uint32_t xr[32];
              float sx[F::kSums], off[F::kSums];
              load_x_regs(xs, it0 + j, lane, xr);
              F::template sums<Ops>(xr, sx);
#pragma unroll
              for (int i = 0; i < F::kSums; i++) off[i] = kOff * sx[i];
              acc1[0] += F::template unit_dot<Ops>(buf[j], Ls[j], xr, sx, off, magic);
            }
          }
        }
        store_rows(acc1, row);
      }
      return;
    }
    for (int base = row0; base < row_end; base += kBatch) {
      float acc[kBatch];
#pragma unroll
      for (int r = 0; r < kBatch; r++) acc[r] = 0.f;
      for (int it = 0; it < nit; it++) {
        const int u = it * 64 + lane;
        typename F::Lane Lu;
        Lu.init(u < units ? u : 0);
        typename F::Raw buf[kBatch];
#pragma unroll
        for (int r = 0; r < kBatch; r++)      // rows past the wavefront's share: its own last row again (cache hits)
          F::fetch(buf[r], w + rb * min(base + r, row_end - 1), Lu, 0xFFFFFFFFu);
        uint32_t xr[32];
        float sx[F::kSums], off[F::kSums];
        load_x_regs(xs, it, lane, xr);
        F::template sums<Ops>(xr, sx);
#pragma unroll
        for (int i = 0; i < F::kSums; i++) off[i] = kOff * sx[i];
#pragma unroll
        for (int r = 0; r < kBatch; r++)
          if (base + r < row_end) acc[r] += F::template unit_dot<Ops>(buf[r], Lu, xr, sx, off, magic);
      }
      store_rows(acc, base);
    }
  }
}

// ------------------------------------------------------------------------------ a few rows at once
// The same arithmetic for TOK activation rows ("tokens") per pass over the weights: the activations
// of all tokens are staged in LDS as permuted pairs, a unit's packed bytes are loaded and unpacked
// once (the unpacking of unit_dot is common to the TOK calls and is shared by the compiler), and
// only the dot products and the per-token offsets repeat.  A pass costs about 1.4 times a
// single-row pass for two tokens and 2.2 times for four.  blockIdx.y walks the groups of TOK
// tokens; tokens past the end re-read the last one and are not stored.
template <class F, class Ops, typename YT, int TOK>
__global__ void __launch_bounds__(kFastThreads)
gemv_dot2_multi_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                       const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                       int rows_per_wave) {
  extern __shared__ uint32_t xs[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int t0 = blockIdx.y * TOK;
  const int units = n_in >> 6;
  const int nit = (units + 63) >> 6;
  const int tok_dwords = nit * 2048;            // LDS dwords per token
  const int64_t rb = F::row_bytes(n_in);
  const int gw = blockIdx.x * kFastWaves + wave;
  const int row0 = gw * rows_per_wave;
  const int row_end = min(row0 + rows_per_wave, n_out);

  // stage the activations: one 16-byte load (8 activations) per thread, token and pass
  for (int k0 = 8 * tid; k0 < nit * 4096; k0 += kStageChunk) {
    uint4 xv[TOK];
#pragma unroll
    for (int t = 0; t < TOK; t++) {
      const uint4 v = *reinterpret_cast<const uint4*>(x + (int64_t)min(t0 + t, m - 1) * n_in + (k0 < n_in ? k0 : 0));
      xv[t] = k0 < n_in ? v : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < TOK; t++) F::stage(xs + t * tok_dwords, k0, xv[t]);
  }
  __syncthreads();

  const uint32_t magic = opaque_vgpr(Ops::kMagic);
  constexpr float kOff = Ops::kOffset + ExtraOffset<F>::value;
  auto store = [&](int row, int t, float v) {
    v = wave_sum_to_lane63(v);
    if (lane == 63 && row < row_end && t0 + t < m)
      YElem<YT>::store(y + (int64_t)(t0 + t) * n_out, row, v + load_bias(bias, bias_dtype, row));
  };
  // dot products of one unit of one row with every token
  auto unit_tokens = [&](const typename F::Raw& buf, const typename F::Lane& Lu, int it, float (&acc)[TOK]) {
#pragma unroll
    for (int t = 0; t < TOK; t++) {
      uint32_t xr[32];
      float sx[F::kSums], off[F::kSums];
      load_x_regs(xs + t * tok_dwords, it, lane, xr);
      F::template sums<Ops>(xr, sx);
#pragma unroll
      for (int i = 0; i < F::kSums; i++) off[i] = kOff * sx[i];
      acc[t] += F::template unit_dot<Ops>(buf, Lu, xr, sx, off, magic);
    }
  };

  if (row_end - row0 < kBatch) {
    // few rows per wavefront: the batch runs along the row, kBatch groups of 64 units at a time
    for (int row = row0; row < row_end; row++) {
      float acc[TOK];
#pragma unroll
      for (int t = 0; t < TOK; t++) acc[t] = 0.f;
      for (int it0 = 0; it0 < nit; it0 += kBatch) {
        typename F::Raw buf[kBatch];
        typename F::Lane Ls[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; j++) {
          const int u = min(it0 + j, nit - 1) * 64 + lane;
          Ls[j].init(u < units ? u : 0);
          F::fetch(buf[j], w + rb * row, Ls[j], 0xFFFFFFFFu);
        }
#pragma unroll
        for (int j = 0; j < kBatch; j++)
          if (it0 + j < nit) unit_tokens(buf[j], Ls[j], it0 + j, acc);
      }
#pragma unroll
      for (int t = 0; t < TOK; t++) store(row, t, acc[t]);
    }
    return;
  }
  for (int base = row0; base < row_end; base += kBatch) {
    float acc[kBatch][TOK];
#pragma unroll
    for (int r = 0; r < kBatch; r++)
#pragma unroll
      for (int t = 0; t < TOK; t++) acc[r][t] = 0.f;
    for (int it = 0; it < nit; it++) {
      const int u = it * 64 + lane;
      typename F::Lane Lu;
      Lu.init(u < units ? u : 0);
      typename F::Raw buf[kBatch];
#pragma unroll
      for (int r = 0; r < kBatch; r++) F::fetch(buf[r], w + rb * min(base + r, row_end - 1), Lu, 0xFFFFFFFFu);
#pragma unroll
      for (int r = 0; r < kBatch; r++)
        if (base + r < row_end) unit_tokens(buf[r], Lu, it, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kBatch; r++)
#pragma unroll
      for (int t = 0; t < TOK; t++) store(base + r, t, acc[r][t]);
  }
}

// ------------------------------------------------------------------------------ launch
static int env_int(const char* name, int dflt) { return dev_knob(name, dflt); }

template <class F, class Ops, typename YT>
static hipError_t launch_fmt_t(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                               int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  static const int wg_per_cu = env_int("TTQ_GEMV_WG_PER_CU", 1);
  const int units = (int)(n_in / 64);
  const int nit = (units + 63) / 64;
  int64_t waves = (int64_t)device_num_cus() * wg_per_cu * kFastWaves;
  if (waves > n_out) waves = n_out;
  int rows_per_wave = (int)((n_out + waves - 1) / waves);
  const int64_t used_waves = (n_out + rows_per_wave - 1) / rows_per_wave;
  const dim3 grid((unsigned)((used_waves + kFastWaves - 1) / kFastWaves), (unsigned)m), block(kFastThreads);
  // staged pairs, and behind them the per-group activation sums of the long-row path
  const size_t lds = (size_t)nit * 2048 * sizeof(uint32_t) + (nit > 1 ? (size_t)nit * F::kSums * 64 * sizeof(float) : 0);
  // Long rows: with a batch of rows or more per wavefront the flat item ring (requests running
  // ahead across rows) wins (28672x8192 Q6_K: 46.6 -> 42.8 us); with fewer, one request of a
  // whole batch along the row does.  TTQ_GEMV_LONG_FLAT=0/1 forces either.
  static const int flat_env = env_int("TTQ_GEMV_LONG_FLAT", -1);
  const int flat = flat_env >= 0 ? flat_env : (rows_per_wave >= kBatch ? 1 : 0);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  const uint16_t* xb = static_cast<const uint16_t*>(x);
  if (nit == 1)
    hipLaunchKernelGGL((gemv_dot2_kernel<F, Ops, YT, true>), grid, block, lds, s, wb, xb,
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)n_in, rows_per_wave, 0);
  else {
    const bool big = n_in > kMaxGemvIn16 / 2;
    auto kernel = big ? gemv_dot2_kernel<F, Ops, YT, false, true> : gemv_dot2_kernel<F, Ops, YT, false, false>;
    static LargeLds configured[2];
    if (lds > 64 * 1024) {
      const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured[big ? 1 : 0]);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, s, wb, xb, static_cast<YT*>(y), bias, bias_dtype, (int)n_out,
                       (int)n_in, rows_per_wave, flat);
  }
  return hipGetLastError();
}

template <class F, class Ops>
static hipError_t launch_fmt_y(const void* w, const void* x, void* y, int y_dtype, const void* bias,
                               int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return launch_fmt_t<F, Ops, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_fmt_t<F, Ops, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_fmt_t<F, Ops, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

bool gemv_dot2_supported(int format, int x_dtype, int64_t n_in) {
  static const int disabled = env_int("TTQ_GEMV_NO_DOT2", 0);
  if (disabled) return false;
  return (format == kQ4_K || format == kQ6_K) && (x_dtype == kBF16 || x_dtype == kF16) && n_in <= kMaxGemvIn16;
}

hipError_t launch_gemv_dot2(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                            const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                            hipStream_t s) {
  if (format == kQ4_K) {
    if (x_dtype == kBF16) return launch_fmt_y<DotQ4K, OpsBF16>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    if (x_dtype == kF16) return launch_fmt_y<DotQ4K, OpsF16>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  } else if (format == kQ6_K) {
    if (x_dtype == kBF16) return launch_fmt_y<DotQ6K, OpsBF16>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    if (x_dtype == kF16) return launch_fmt_y<DotQ6K, OpsF16>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  }
  return hipErrorInvalidValue;
}


// ---- launch of the few-rows kernel
template <class F, class Ops, typename YT, int TOK>
static hipError_t launch_multi_t(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                                 int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  const int units = (int)(n_in / 64);
  const int nit = (units + 63) / 64;
  int64_t waves = (int64_t)device_num_cus() * kFastWaves;
  if (waves > n_out) waves = n_out;
  const int rows_per_wave = (int)((n_out + waves - 1) / waves);
  const int64_t used_waves = (n_out + rows_per_wave - 1) / rows_per_wave;
  const dim3 grid((unsigned)((used_waves + kFastWaves - 1) / kFastWaves), (unsigned)((m + TOK - 1) / TOK)),
      block(kFastThreads);
  const size_t lds = (size_t)TOK * nit * 2048 * sizeof(uint32_t);
  auto kernel = gemv_dot2_multi_kernel<F, Ops, YT, TOK>;
  static LargeLds configured;
  if (lds > 64 * 1024) {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, grid, block, lds, s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                     static_cast<YT*>(y), bias, bias_dtype, (int)m, (int)n_out, (int)n_in, rows_per_wave);
  return hipGetLastError();
}

template <class F, class Ops, int TOK>
static hipError_t launch_multi_y(const void* w, const void* x, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return launch_multi_t<F, Ops, float, TOK>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return launch_multi_t<F, Ops, f16_tag, TOK>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return launch_multi_t<F, Ops, bf16_tag, TOK>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

template <class F, int TOK>
static hipError_t launch_multi_x(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return launch_multi_y<F, OpsBF16, TOK>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return launch_multi_y<F, OpsF16, TOK>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

// Four tokens per pass while their staged activations fit LDS (n_in <= 16384), else two.
static int multi_tokens(int64_t m, int64_t n_in) {
  const int nit = (int)((n_in / 64 + 63) / 64);
  const size_t per_tok = (size_t)nit * 2048 * sizeof(uint32_t);
  if (m > 2 && 4 * per_tok <= 150 * 1024) return 4;
  return 2 * per_tok <= 150 * 1024 ? 2 : 0;
}

bool gemv_dot2_multi_supported(int format, int x_dtype, int64_t m, int64_t n_in) {
  static const int disabled = env_int("TTQ_GEMV_NO_BATCH", 0);
  return !disabled && m >= 2 && gemv_dot2_supported(format, x_dtype, n_in) && multi_tokens(m, n_in) != 0;
}

hipError_t launch_gemv_dot2_multi(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                  const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                  hipStream_t s) {
  const int tok = multi_tokens(m, n_in);
  if (format == kQ6_K) {
    if (tok == 4) return launch_multi_x<DotQ6K, 4>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    return launch_multi_x<DotQ6K, 2>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  }
  if (format == kQ4_K) {
    if (tok == 4) return launch_multi_x<DotQ4K, 4>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    return launch_multi_x<DotQ4K, 2>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace ttq
