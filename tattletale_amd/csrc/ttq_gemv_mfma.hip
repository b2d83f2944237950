// Decode GEMV for Q4_K weights and 16-bit activations on gfx950 through the int8 matrix cores.
//
// Same operator as ttq_gemv.hip (F.linear with a single-token activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81).  The packed-dot kernel in
// ttq_gemv_dot2.hip needs about 2.6 vector-ALU instructions per weight byte and is bound by
// them; this kernel leaves only the nibble split (3 instructions per 8 weights) on the
// vector ALU and hands the multiply-adds AND the reduction along the row to
// v_mfma_i32_16x16x64_i8.
//
// Arithmetic.  Per sub-block of 32 activations the kernel picks the power of two 2^E just
// below the largest |x| and turns every activation into a 15-bit integer
// v = rint(x * 2^(13-E)), split into two signed bytes v = 256*hi + lo (lo in [-128,127],
// |hi| <= 64).  sum(q*v) over a sub-block is then an exact integer (< 2^24), and
//       sum(q*x) = 2^(E-13) * (256 * sum(q*hi) + sum(q*lo))
// carries only the rounding of x to 14 bits below its sub-block maximum (relative error
// about 3e-5 of the row product; a unit-vector activation is exact, so the canonical
// dequantized weight d*sc*q - dmin*m is still reproduced bit for bit).  Scales and mins are
// applied once per sub-block in fp32, in the canonical order.
//
// Matrix shapes.  One MFMA multiplies A (16 x 64, the activations) by B (64 x 16, weights of
// 16 rows) into C (16 x 16).  The 16 rows of A are (sub-block j, plane t) = (0..7) x (hi, lo)
// of ONE super-block; a row is zero wherever the 64 k-positions of this MFMA do not belong to
// its sub-block, so C[2j+t][n] = sum over sub-block j of plane_t(x) * q for weight row n.
// Four MFMAs (two 64-byte halves of the 128 qs bytes, low and high nibbles) cover a
// super-block of 16 weight rows; 15/16 of the multiplies are by zero, which costs nothing that
// matters (the matrix cores are otherwise idle) and buys the per-sub-block separation the
// block scales need.  Lane (n = lane%16, g = lane/16) loads 16 qs bytes of weight row n,
// supplies them as B, and receives C rows 4g..4g+3, i.e. both planes of sub-blocks 2g and
// 2g+1 of its own row, whose scales it decodes from the header it loaded itself: no
// cross-lane traffic until the row is finished.
//
// Work distribution.  One workgroup of 16 wavefronts per CU.  A wavefront owns a group of 16
// consecutive rows and one of SL interleaved slices of the super-blocks, and walks it one
// step (16 rows x one super-block, 3 x 16 bytes per lane) at a time.  SL is chosen so that
// all 16 wavefronts have work even when a workgroup owns few rows.
#include <type_traits>

#include "ttq_gemv_mfma_common.h"

namespace ttq {

// Bit positions of the two 6-bit scales and mins a lane needs (sub-blocks 2g and 2g+1) inside
// the 12 packed bytes: sub-blocks 0..3 keep the whole field in bytes 0..7, sub-blocks 4..7
// keep 4 bits in bytes 8..11 and 2 bits on top of bytes 0..7.  Two bit-field extracts each,
// the second with width 0 in the simple case, so no branch is needed.
struct ScaleBits {
  bool upper;
  uint32_t wl, wh;
  uint32_t sc_lo[2], mn_lo[2], hi[2];
  __device__ __forceinline__ void init(int g) {
    upper = g >= 2;
    wl = upper ? 4u : 6u;
    wh = upper ? 2u : 0u;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const uint32_t jj = (2u * g + h) & 3u;
      sc_lo[h] = 8u * jj;
      mn_lo[h] = upper ? 8u * jj + 4u : 8u * jj;
      hi[h] = 8u * jj + 6u;
    }
  }
};

struct StepRaw { uint4 hdr, c0, c1; };

// Optional RMSNorm in front of the GEMV (NORM kernels): normalized = rms_norm(x [+ residual]) *
// gamma, as RmsNorm.forward / forward_with_residual compute it before a Linear
// (workspace/transformers/src/layers/norm.nim:23-38).  All buffers hold the activation type.

// LDS layout (bytes): plane table, then the per-sub-block constants [nsb][4] x float4
// {2^(E-13) of sub-blocks 2g, 2g+1, sum(x) of 2g, 2g+1}, then the partial row sums of the
// wavefronts [W][16] floats.
// The plane table holds, per super-block b, the A operands of its four MFMAs.  Entry (b, m, h),
// m = 2j + t, is plane t (0 = hi, 1 = lo) of the 16 activations x[256b + 32j + 16h ..]; as the A
// operand of MFMA q = 2P + nib (P = which 64 bytes of qs, nib = low/high nibbles), lane (m, ga)
// supplies that entry when k-group ga of this MFMA is sub-block j (j = 4P + 2(ga/2) + nib,
// h = ga%2) and zeros otherwise.  Two layouts:
//   wide    [nsb][4 MFMAs][64 lanes] x 16 bytes, zeros stored: every address is one register
//           plus an immediate.  4 KiB per super-block, so only for n_in <= 8192.
//   compact [nsb][32] x 16 bytes plus one zero entry.  A lane has at most one non-zero MFMA out
//           of the four and reads `base_q + sb * stride_q` with (base, stride) = (its entry, 512)
//           for that one and (the zero entry, 0) for the others: four more VALU instructions
//           per step (about 3 % at 14336 x 4096), any n_in the entry points accept.
//
// W wavefronts per workgroup, R steps in flight per wavefront.
//
// FUSE: the weight holds gate rows [0, n_out) followed by up rows [n_out, 2*n_out), as
// GatedMLP builds it (workspace/transformers/src/layers/mlp.nim:39), and the kernel writes
// silu(gate . x) * (up . x), the silu_and_mul of
// workspace/transformers/src/kernels/activations.nim:14-38, for its n_out outputs: row groups
// alternate between the gate rows and the up rows of the same 16 outputs, and the wavefronts'
// row sums meet in LDS at the end of every round.  rows_per_wg then counts outputs.
//
// NORM: every workgroup first normalizes the activation row itself (8 to 32 KiB, cheaper than a
// kernel launch): t = x + residual rounded to the activation type, normalized =
// t * rsqrt(mean(t^2) + eps) * gamma in fp32, rounded once to the activation type; the GEMV
// then consumes exactly those rounded values.  Workgroup 0 writes t and the normalized row out.
template <int W, int R, bool FUSE, bool COMPACT, bool NORM, typename XT, typename YT>
__global__ void __launch_bounds__(W * 64)
gemv_q4k_mfma_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                     const void* __restrict__ bias, int bias_dtype, int n_out, int nsb, int rows_per_wg,
                     int sl_log2, GemvNormArgs na) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const size_t table_bytes = COMPACT ? (size_t)nsb * 512 + 16 : (size_t)nsb * 4096;
  v4i_t* xa = reinterpret_cast<v4i_t*>(smem);
  float* tab = reinterpret_cast<float*>(smem + table_bytes);
  float* part = reinterpret_cast<float*>(smem + table_bytes + (size_t)nsb * 64);

  constexpr int kThreads = W * 64;
  // staging passes of 8 activations per thread: one covers everything the wide table can hold
  constexpr int XP = COMPACT ? (int)(kMaxMfmaIn / (8 * kThreads)) : (kMaxWideSb * 256 + 8 * kThreads - 1) / (8 * kThreads);
  const int SL = 1 << sl_log2;          // slices of the super-blocks
  const int G = W >> sl_log2;           // row groups per round
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int gi = wave >> sl_log2, sl = wave & (SL - 1);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nsb * 256;
  const uint16_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const uint32_t rb = (uint32_t)nsb * 144u;
  const int S = (nsb + SL - 1) >> sl_log2;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int per_round = FUSE ? 8 * G : 16 * G;   // rows (outputs when fused) of the workgroup per round
  const int rounds = (rows_per_wg + per_round - 1) / per_round;
  const int t_total = rounds * S;
  const int last = wg_row_end - 1;   // rows past the workgroup's share re-read its last row
  // Weights are requested with lane = 4 * row + k-group (the 64 bytes of a row that one request
  // covers lie in a quad of neighbouring lanes: the memory pipeline merges neighbours' accesses only,
  // so this is one look-up per row instead of four) and exchanged into the MFMA operand layout
  // lane = row + 16 * k-group when the step is consumed.
  const int ln = lane >> 2, lg = lane & 3;
  const int from_lane4 = 4 * (4 * n + g);
  // weight row that this lane requests in row group `grp` of the workgroup
  auto group_row_of = [&](int grp, int r) {
    if constexpr (FUSE) return min(wg_row0 + (grp >> 1) * 16 + r, last) + (grp & 1) * n_out;
    else return min(wg_row0 + grp * 16 + r, last);
  };

  // ---- activations: 16-byte loads (8 values) per thread, requested before any weights
  // (fp32 activations, plain kernel only: 32 bytes per thread; `x` then points at floats)
  constexpr bool kX32 = std::is_same<XT, float>::value;
  static_assert(!kX32 || !NORM, "the fused RMSNorm takes 16-bit activations");
  uint4 xraw[XP], xraw2[kX32 ? XP : 1];
#pragma unroll
  for (int p = 0; p < XP; p++) {
    const int k0 = 8 * (tid + p * kThreads);
    // a pass past the end re-reads the first pass's data (the compact table means n_in > 8192;
    // spread addresses, never used)
    const int kc = k0 < n_in ? k0 : (COMPACT ? (k0 & (8 * kThreads - 1)) : 0);
    if constexpr (kX32) {
      const float* xf = reinterpret_cast<const float*>(x) + (int64_t)blockIdx.y * n_in + kc;
      xraw[p] = *reinterpret_cast<const uint4*>(xf);
      xraw2[p] = *reinterpret_cast<const uint4*>(xf + 4);
    } else {
      xraw[p] = *reinterpret_cast<const uint4*>(xm + kc);
    }
  }
  uint4 rraw[NORM ? XP : 1], graw[NORM ? XP : 1];
  if constexpr (NORM) {
#pragma unroll
    for (int p = 0; p < XP; p++) {
      const int k0 = 8 * (tid + p * kThreads);
      const int kc = k0 < n_in ? k0 : (COMPACT ? (k0 & (8 * kThreads - 1)) : 0);
      graw[p] = *reinterpret_cast<const uint4*>(na.gamma + kc);
      rraw[p] = make_uint4(0, 0, 0, 0);
      if (na.residual != nullptr) rraw[p] = *reinterpret_cast<const uint4*>(na.residual + (int64_t)blockIdx.y * n_in + kc);
    }
  }
  // every wavefront's x request is queued before any weight request of this workgroup
  __builtin_amdgcn_s_barrier();

  // ---- weight stream: step t = (round r, slice step si); loads are unconditional (clamped)
  StepRaw ring[R];
  int ir = 0, isi = 0;                  // round and step-in-round of the next request
  auto issue = [&](StepRaw& dst) {
    const int sb = (isi << sl_log2) + sl;
    const bool ok = ir < rounds && sb < nsb;
    const int row = group_row_of(ir * G + gi, ln), hrow = group_row_of(ir * G + gi, n);
    const uint32_t o_hdr = ok ? (uint32_t)hrow * rb + (uint32_t)sb * 144u : 0u;
    const uint32_t o_q = (ok ? (uint32_t)row * rb + (uint32_t)sb * 144u : 0u) + 16u + 16u * (uint32_t)lg;
    dst.hdr = load16_a16(w + o_hdr);
    dst.c0 = load16_a16(w + o_q);
    dst.c1 = load16_a16(w + (o_q + 64u));
    if (++isi == S) { isi = 0; ir++; }
  };
#pragma unroll
  for (int i = 0; i < R; i++) issue(ring[i]);

  // ---- zero the plane-table entries that stay zero.  Wide entry (b, q, la): la = 16*ga + m,
  // m = 2j + t.  MFMA q = 2P + nib covers, in k-group ga, sub-block 4P + 2(ga/2) + nib.
  if constexpr (COMPACT) {
    if (tid < 4) reinterpret_cast<uint32_t*>(smem + (size_t)nsb * 512)[tid] = 0u;
  } else {
    const int la = tid & 63, q = (tid >> 6) & 3;
    const int j = (la & 15) >> 1, ga = la >> 4;
    const bool nonzero = (q == 2 * (j >> 2) + (j & 1)) && ((ga >> 1) == ((j & 3) >> 1));
    if (!nonzero) {
      const v4i_t z = {0, 0, 0, 0};
      for (int b = tid >> 8; b < nsb; b += W / 4) xa[(b * 4 + q) * 64 + la] = z;
    }
  }

  // ---- the activations as floats, normalized first if asked
  float xv[XP][8];
#pragma unroll
  for (int p = 0; p < XP; p++) {
    if constexpr (kX32) {
      const uint32_t d[8] = {xraw[p].x, xraw[p].y, xraw[p].z, xraw[p].w, xraw2[p].x, xraw2[p].y, xraw2[p].z, xraw2[p].w};
#pragma unroll
      for (int i = 0; i < 8; i++) xv[p][i] = __uint_as_float(d[i]);
    } else {
      widen8<XT>(xraw[p], xv[p]);
    }
  }
  if constexpr (NORM) {
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < XP; p++) {
      const int k0 = 8 * (tid + p * kThreads);
      if (k0 < n_in) {
        if (na.residual != nullptr) {
          float rf[8];
          widen8<XT>(rraw[p], rf);
#pragma unroll
          for (int i = 0; i < 8; i++) xv[p][i] += rf[i];
          const uint4 t = narrow8<XT>(xv[p]);     // the new residual, as the reference's add rounds it
          if (blockIdx.x == 0 && na.new_residual != nullptr)
            *reinterpret_cast<uint4*>(na.new_residual + (int64_t)blockIdx.y * n_in + k0) = t;
        }
#pragma unroll
        for (int i = 0; i < 8; i++) ss += xv[p][i] * xv[p][i];
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) part[wave] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < W; i++) total += part[i];
    const float rs = 1.f / sqrtf(total / (float)n_in + na.eps);
#pragma unroll
    for (int p = 0; p < XP; p++) {
      const int k0 = 8 * (tid + p * kThreads);
      if (k0 < n_in) {
        float gf[8];
        widen8<XT>(graw[p], gf);
#pragma unroll
        for (int i = 0; i < 8; i++) xv[p][i] = (xv[p][i] * rs) * gf[i];
        const uint4 t = narrow8<XT>(xv[p]);
        if (blockIdx.x == 0 && na.normed != nullptr)
          *reinterpret_cast<uint4*>(na.normed + (int64_t)blockIdx.y * n_in + k0) = t;
      }
    }
  }

  // ---- quantize the activations into the two byte planes
#pragma unroll
  for (int p = 0; p < XP; p++) {
    const int k0 = 8 * (tid + p * kThreads);
    if (k0 < n_in) {
      float (&xf)[8] = xv[p];
      float amax = 0.f, sum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        amax = fmaxf(amax, fabsf(xf[i]));
        sum += xf[i];
      }
      // the four threads of a sub-block are an aligned quad
      amax = fmaxf(amax, dpp_quad<0xB1>(amax));
      amax = fmaxf(amax, dpp_quad<0x4E>(amax));
      sum += dpp_quad<0xB1>(sum);
      sum += dpp_quad<0x4E>(sum);
      const uint32_t eb = __float_as_uint(amax) >> 23;      // biased exponent (amax >= 0)
      const uint32_t ec = eb < 14u ? 14u : eb;
      const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
      // non-finite activations poison the sub-block instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
      int hi[8], lo[8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int v = (int)rintf(xf[i] * mul);
        hi[i] = (v + 128) >> 8;
        lo[i] = v;                     // only the low byte is used
      }
      const int b = k0 >> 8, j = (k0 >> 5) & 7, h = (k0 >> 4) & 1, half8 = (k0 >> 3) & 1;
      const int q = 2 * (j >> 2) + (j & 1);
      const int ga = 2 * ((j & 3) >> 1) + h;
      // entry of the hi plane in 8-byte units, and the distance to the lo plane's
      const int e_hi = COMPACT ? (b * 32 + 4 * j + h) * 2 + half8 : ((b * 4 + q) * 64 + 16 * ga + 2 * j) * 2 + half8;
      constexpr int kLoStep = COMPACT ? 4 : 2;
      uint2* xa8 = reinterpret_cast<uint2*>(smem);
      xa8[e_hi] = make_uint2(pack_low_bytes(hi[0], hi[1], hi[2], hi[3]), pack_low_bytes(hi[4], hi[5], hi[6], hi[7]));
      xa8[e_hi + kLoStep] = make_uint2(pack_low_bytes(lo[0], lo[1], lo[2], lo[3]), pack_low_bytes(lo[4], lo[5], lo[6], lo[7]));
      if ((tid & 3) == 0) {
        float* e = tab + (b * 4 + (j >> 1)) * 4 + (j & 1);
        e[0] = f;
        e[2] = sum;
      }
    }
  }
  __syncthreads();

  // ---- main loop
  ScaleBits B;
  B.init(g);
  constexpr uint32_t N4 = 0x0F0F0F0Fu;
  // compact table: A-operand addresses of this lane (m = lane%16, ga = lane/16) for the four MFMAs
  uint32_t a_base[4], a_stride[4];
  {
    const int mrow = lane & 15, ga = lane >> 4, j = mrow >> 1;
    const bool valid = (ga >> 1) == ((j & 3) >> 1);
    const int qstar = 2 * (j >> 2) + (j & 1);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const bool mine = valid && q == qstar;
      a_base[q] = mine ? (uint32_t)(mrow * 2 + (ga & 1)) * 16u : (uint32_t)nsb * 512u;
      a_stride[q] = mine ? 512u : 0u;
    }
  }
  int cr = 0, csi = 0;                  // round and step-in-round being consumed
  float acc = 0.f;

  auto pull = [&](uint4& v) {
    v.x = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)v.x);
    v.y = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)v.y);
    v.z = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)v.z);
    v.w = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)v.w);
  };
  // `s` is the step in operand layout (see exchange below)
  auto consume = [&](const StepRaw& s) {
    const int sb = (csi << sl_log2) + sl;
    if (cr < rounds && sb < nsb) {
      v4i_t a0, a1, a2, a3;
      if constexpr (COMPACT) {
        a0 = *reinterpret_cast<const v4i_t*>(smem + a_base[0] + (uint32_t)sb * a_stride[0]);
        a1 = *reinterpret_cast<const v4i_t*>(smem + a_base[1] + (uint32_t)sb * a_stride[1]);
        a2 = *reinterpret_cast<const v4i_t*>(smem + a_base[2] + (uint32_t)sb * a_stride[2]);
        a3 = *reinterpret_cast<const v4i_t*>(smem + a_base[3] + (uint32_t)sb * a_stride[3]);
      } else {
        const v4i_t* xe = xa + (size_t)sb * 256 + lane;
        a0 = xe[0]; a1 = xe[64]; a2 = xe[128]; a3 = xe[192];
      }
      const float4 cst = *reinterpret_cast<const float4*>(tab + (sb * 4 + g) * 4);
      v4i_t L0, H0, L1, H1;
      L0[0] = (int)(s.c0.x & N4); H0[0] = (int)((s.c0.x >> 4) & N4);
      L0[1] = (int)(s.c0.y & N4); H0[1] = (int)((s.c0.y >> 4) & N4);
      L0[2] = (int)(s.c0.z & N4); H0[2] = (int)((s.c0.z >> 4) & N4);
      L0[3] = (int)(s.c0.w & N4); H0[3] = (int)((s.c0.w >> 4) & N4);
      L1[0] = (int)(s.c1.x & N4); H1[0] = (int)((s.c1.x >> 4) & N4);
      L1[1] = (int)(s.c1.y & N4); H1[1] = (int)((s.c1.y >> 4) & N4);
      L1[2] = (int)(s.c1.z & N4); H1[2] = (int)((s.c1.z >> 4) & N4);
      L1[3] = (int)(s.c1.w & N4); H1[3] = (int)((s.c1.w >> 4) & N4);
      // two independent chains; their non-zero rows are disjoint (sub-blocks 0-3 and 4-7)
      const v4i_t zero = {0, 0, 0, 0};
      v4i_t Ca = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, L0, zero, 0, 0, 0);
      v4i_t Cb = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, L1, zero, 0, 0, 0);
      Ca = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, H0, Ca, 0, 0, 0);
      Cb = __builtin_amdgcn_mfma_i32_16x16x64_i8(a3, H1, Cb, 0, 0, 0);
      const v4i_t C = Ca + Cb;

      const float d = f16_bits_to_f32((uint16_t)(s.hdr.x & 0xFFFFu));
      const float dmin = f16_bits_to_f32((uint16_t)(s.hdr.x >> 16));
      const uint32_t a_sc = B.upper ? s.hdr.w : s.hdr.y;   // bytes 8-11 or 0-3
      const uint32_t a_mn = B.upper ? s.hdr.w : s.hdr.z;   // bytes 8-11 or 4-7
      const uint32_t sc1 = __builtin_amdgcn_ubfe(a_sc, B.sc_lo[0], B.wl) | (__builtin_amdgcn_ubfe(s.hdr.y, B.hi[0], B.wh) << 4);
      const uint32_t sc2 = __builtin_amdgcn_ubfe(a_sc, B.sc_lo[1], B.wl) | (__builtin_amdgcn_ubfe(s.hdr.y, B.hi[1], B.wh) << 4);
      const uint32_t mn1 = __builtin_amdgcn_ubfe(a_mn, B.mn_lo[0], B.wl) | (__builtin_amdgcn_ubfe(s.hdr.z, B.hi[0], B.wh) << 4);
      const uint32_t mn2 = __builtin_amdgcn_ubfe(a_mn, B.mn_lo[1], B.wl) | (__builtin_amdgcn_ubfe(s.hdr.z, B.hi[1], B.wh) << 4);
      // exact integers below 2^24, scaled by a power of two: sum(q*x) of the sub-block
      const float q1 = (float)(C[0] * 256 + C[1]) * cst.x;
      const float q2 = (float)(C[2] * 256 + C[3]) * cst.y;
      acc = acc + (d * (float)sc1) * q1;
      acc = acc - (dmin * (float)mn1) * cst.z;
      acc = acc + (d * (float)sc2) * q2;
      acc = acc - (dmin * (float)mn2) * cst.w;
    }
    if (++csi == S) {
      // the row group is finished for this wavefront's slice: add the four k-groups
      float v = acc;
      v = add_xor16(v);
      v = add_xor32(v);
      if constexpr (FUSE) {
        // every wavefront ends its round after the same number of steps
        if (lane < 16) part[wave * 16 + n] = v;
        __syncthreads();
        if (cr < rounds && tid < 8 * G) {
          const int pair = tid >> 4, nn = tid & 15;
          float gate = 0.f, up = 0.f;
          for (int s2 = 0; s2 < SL; s2++) {
            gate += part[((2 * pair) * SL + s2) * 16 + nn];
            up += part[((2 * pair + 1) * SL + s2) * 16 + nn];
          }
          const int o = wg_row0 + (cr * (G >> 1) + pair) * 16 + nn;
          if (o < wg_row_end) {
            gate += load_bias(bias, bias_dtype, o);
            up += load_bias(bias, bias_dtype, (int64_t)n_out + o);
            YElem<YT>::store(ym, o, (gate / (1.f + expf(-gate))) * up);
          }
        }
        __syncthreads();
      } else if (cr < rounds) {
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

  // steady state: every consumed slot is re-requested R steps ahead; the last R steps drain
  for (int t0 = R; t0 < t_total; t0 += R) {
#pragma unroll
    for (int i = 0; i < R; i++) {
      // exchange into operand layout, re-request the slot, then do the arithmetic
      StepRaw t = ring[i];
      pull(t.c0); pull(t.c1);
      issue(ring[i]);
      consume(t);
    }
  }
#pragma unroll
  for (int i = 0; i < R; i++) {
    StepRaw t = ring[i];
    pull(t.c0); pull(t.c1);
    consume(t);
  }

  if (!FUSE && sl_log2 != 0) {
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

// ------------------------------------------------------------------------------ launch
template <bool FUSE, bool NORM, typename XT, typename YT>
static hipError_t launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                            int64_t m, int64_t n_out, int64_t n_in, const GemvNormArgs& na, hipStream_t s) {
  constexpr int W = kMfmaWaves;
  const int nsb = (int)(n_in / 256);
  static const int forced_wgs = mfma_env_int("TTQ_GEMV_MFMA_WGS", 0);
  int num_wg = forced_wgs > 0 ? forced_wgs : device_num_cus();
  const int64_t groups = (n_out + 15) / 16;
  if (num_wg > groups) num_wg = (int)groups;
  const int rows_per_wg = (int)((n_out + num_wg - 1) / num_wg);
  num_wg = (int)((n_out + rows_per_wg - 1) / rows_per_wg);
  // the most slices that still leave room for all the workgroup's rows (outputs when fused: each
  // needs a gate and an up row group) in one round
  constexpr int kMaxSl = FUSE ? W / 2 : W;
  constexpr int kRowsAllWaves = FUSE ? 8 * W : 16 * W;
  int sl_log2 = 0;
  while ((2 << sl_log2) <= kMaxSl && (2 << sl_log2) <= nsb && (kRowsAllWaves >> (sl_log2 + 1)) >= rows_per_wg)
    sl_log2++;
  const bool compact = nsb > kMaxWideSb;
  const size_t lds = (compact ? (size_t)nsb * 512 + 16 : (size_t)nsb * 4096) + (size_t)nsb * 64 + 1024;
  const dim3 grid((unsigned)num_wg, (unsigned)m), block(W * 64);
  const auto launch = [&](auto kernel, LargeLds& configured) -> hipError_t {
    {
      const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, s, static_cast<const uint8_t*>(w),
                       static_cast<const uint16_t*>(x), static_cast<YT*>(y), bias, bias_dtype, (int)n_out, nsb,
                       rows_per_wg, sl_log2, na);
    return hipGetLastError();
  };
  static LargeLds configured_wide, configured_compact;
  if (compact) return launch(gemv_q4k_mfma_kernel<W, kMfmaRing, FUSE, true, NORM, XT, YT>, configured_compact);
  return launch(gemv_q4k_mfma_kernel<W, kMfmaRing, FUSE, false, NORM, XT, YT>, configured_wide);
}

template <bool FUSE, bool NORM, typename XT>
static hipError_t launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                           int64_t m, int64_t n_out, int64_t n_in, const GemvNormArgs& na, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return launch_xy<FUSE, NORM, XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, na, s);
    case kF16: return launch_xy<FUSE, NORM, XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, na, s);
    case kBF16: return launch_xy<FUSE, NORM, XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, na, s);
    default: return hipErrorInvalidValue;
  }
}

template <bool FUSE, bool NORM>
static hipError_t launch_any(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                             int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, const GemvNormArgs& na,
                             hipStream_t s) {
  if (x_dtype == kBF16) return launch_x<FUSE, NORM, bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
  if (x_dtype == kF16) return launch_x<FUSE, NORM, f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
  if constexpr (!FUSE && !NORM) {
    if (x_dtype == kF32) return launch_x<false, false, float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
  }
  return hipErrorInvalidValue;
}

bool gemv_mfma_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  static const int disabled = mfma_env_int("TTQ_GEMV_NO_MFMA", 0);
  if (disabled) return false;
  // byte offsets into the weight buffer are 32-bit in the kernel; with fewer than eight rows per
  // CU the per-workgroup activation set-up outweighs the saving
  return n_out >= 2048 && format == kQ4_K && (x_dtype == kBF16 || x_dtype == kF16 || x_dtype == kF32) && n_in % 256 == 0 &&
         n_in <= kMaxMfmaIn && n_out * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_mfma(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  return launch_any<false, false>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, GemvNormArgs{}, s);
}

// Fused variants: gate/up projection + silu_and_mul (w holds 2*n_out rows, gate rows first,
// y has n_out columns) and/or RMSNorm in front (norm_gamma != null).  Supported for 16-bit
// activations, any n_in the entry points accept, n_out >= 16.
bool gemv_fused_supported(int format, int x_dtype, int64_t n_out, int64_t n_in, bool silu_mul) {
  return format == kQ4_K && (x_dtype == kBF16 || x_dtype == kF16) && n_in % 256 == 0 && n_in <= kMaxMfmaIn &&
         n_out >= 16 && (silu_mul ? 2 : 1) * n_out * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                             int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, bool silu_mul,
                             const void* norm_residual, const void* norm_gamma, float norm_eps,
                             void* new_residual_out, void* normed_out, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  GemvNormArgs na{};
  na.residual = static_cast<const uint16_t*>(norm_residual);
  na.gamma = static_cast<const uint16_t*>(norm_gamma);
  na.new_residual = static_cast<uint16_t*>(new_residual_out);
  na.normed = static_cast<uint16_t*>(normed_out);
  na.eps = norm_eps;
  if (norm_gamma != nullptr) {
    if (silu_mul) return launch_any<true, true>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
    return launch_any<false, true>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
  }
  if (silu_mul) return launch_any<true, false>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
  return launch_any<false, false>(w, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, na, s);
}

}  // namespace ttq
