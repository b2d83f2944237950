// Decode GEMV for Q4_K weights and a FEW activation rows (2 .. 32: batched decode, speculative
// decoding, very short prompts) on gfx950 through the int8 matrix cores.
//
// Same operator as ttq_gemv.hip (F.linear, workspace/libtorch/src/abi/neural_nets.nim:64-81, with
// the small batch*seq of workspace/transformers/src/layers/attn.nim:154-156).  Launching the
// single-row kernel once per row reads the weights once per row; the prefill GEMM dequantizes
// every weight to bf16 whatever the row count.  This kernel reads and unpacks the weights once
// for TOK = 8 or 16 activation rows ("tokens") and keeps the arithmetic of the single-row kernel
// (ttq_gemv_mfma.hip): activations as 15-bit block fixed point in two byte planes, exact integer
// sums per sub-block, scales and mins applied once per sub-block in fp32.  A unit-vector
// activation still reproduces the canonical dequantized weight bit for bit.
//
// Matrix shapes.  The tokens sit on the rows of the MFMA's A operand: with TOK = 8 row 2*tk + t
// is plane t (hi, lo) of token tk, with TOK = 16 row tk is token tk and the two planes take two
// MFMAs.  One MFMA handles ONE sub-block of 16 weight rows: its 64 k-positions are 32 low (or
// high) nibbles of two sub-blocks, so A is zero in the k-groups of the other one (a lane either
// reads its table entry or one shared zero entry).  Eight (sixteen) MFMAs per super-block of 16
// weight rows.  Lane (n = lane%16, g = lane/16) loads 16 qs bytes of weight row n, supplies
// them as B and receives C rows 4g..4g+3 of column n: everything of tokens 2g, 2g+1 (TOK = 8)
// or the plane sums of tokens 4g..4g+3 (TOK = 16) for its own weight row.  The vector ALU is
// the bottleneck of this kernel, so the sub-block scales are decoded once per row (two per lane)
// and spread over the row's four lanes, and the min term is summed, by fp32 matrix instructions.
//
// Work distribution as in ttq_gemv_mfma.hip, two steps in flight per wavefront; blockIdx.y walks
// the groups of TOK tokens.
#include "ttq_gemv_mfma_common.h"

namespace ttq {

struct BatchStep { uint4 hdr, c0, c1; };
typedef float v4f_t __attribute__((ext_vector_type(4)));

// LDS (bytes): plane table [nsb*8 sub-blocks][TOK/8 planes-in-own-slab][16 rows][2 halves] x 16,
// one zero entry (64 bytes reserved), then f = 2^(E-13) and sum(x) per (sub-block, token) as two
// float arrays [nsb*8][TOK].  The per-wavefront partial sums of the last step overlay the table.
template <int TOK, typename XT, typename YT>
__global__ void __launch_bounds__(kMfmaThreads)
gemv_q4k_batch_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                      const void* __restrict__ bias, int bias_dtype, int m, int n_out, int nsb, int rows_per_wg,
                      int sl_log2) {
  static_assert(TOK == 8 || TOK == 16, "tokens per workgroup");
  constexpr int W = kMfmaWaves;
  constexpr int TPL = TOK / 4;                   // tokens per lane
  constexpr int kSubBytes = 64 * TOK;            // plane table bytes per sub-block
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t table_bytes = (uint32_t)nsb * 8u * kSubBytes;
  const uint32_t zero_off = table_bytes;
  float* tf = reinterpret_cast<float*>(smem + table_bytes + 64);
  float* ts = tf + (size_t)nsb * 8 * TOK;
  float* part = reinterpret_cast<float*>(smem);

  const int SL = 1 << sl_log2, G = W >> sl_log2;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int gi = wave >> sl_log2, sl = wave & (SL - 1);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nsb * 256;
  const int t0 = blockIdx.y * TOK;
  const uint32_t rb = (uint32_t)nsb * 144u;
  const int S = (nsb + SL - 1) >> sl_log2;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int rounds = (rows_per_wg + 16 * G - 1) / (16 * G);
  const int t_total = rounds * S;
  const int last = wg_row_end - 1;   // rows past the workgroup's share re-read its last row

  // ---- activations, requested before any weights.  A thread stages 8 consecutive values; when
  // a row needs fewer than all threads, the threads split the tokens among `nrep` replicas.
  // Tokens past the end re-read the last one and are never stored.
  const int kthreads = n_in >> 3;                      // threads per token (n_in <= 8192)
  const int nrep = kMfmaThreads / kthreads;
  const int rep = tid / kthreads;
  const int k0 = 8 * (tid - rep * kthreads);
  const bool stager = rep < nrep;
  uint4 xraw[TOK];
#pragma unroll
  for (int it = 0; it < TOK; it++) {
    const int tk = rep + it * nrep;
    if (stager && tk < TOK) xraw[it] = *reinterpret_cast<const uint4*>(x + (int64_t)min(t0 + tk, m - 1) * n_in + k0);
  }
  __builtin_amdgcn_s_barrier();

  // ---- weight stream; loads are unconditional (clamped)
  // Two steps in flight per wavefront: a step keeps the wavefront busy for long enough that the
  // next one has to be on its way meanwhile.  (Four, i.e. nearly the whole share of a workgroup
  // requested before the activations are staged, measured slower.)
  constexpr int R = 2;
  BatchStep ring[R];
  int ir = 0, isi = 0;
  auto issue = [&](BatchStep& dst) {
    const int sb = (isi << sl_log2) + sl;
    const bool ok = ir < rounds && sb < nsb;
    const int row = min(wg_row0 + (ir * G + gi) * 16 + n, last);
    const uint32_t o_hdr = ok ? (uint32_t)row * rb + (uint32_t)sb * 144u : 0u;
    const uint32_t o_q = o_hdr + 16u + 16u * (uint32_t)g;
    dst.hdr = load16_a16(w + o_hdr);
    dst.c0 = load16_a16(w + o_q);
    dst.c1 = load16_a16(w + (o_q + 64u));
    if (++isi == S) { isi = 0; ir++; }
  };
#pragma unroll
  for (int i = 0; i < R; i++) issue(ring[i]);

  if (tid < 4) reinterpret_cast<uint32_t*>(smem + zero_off)[tid] = 0u;

  // ---- quantize the activations into the two byte planes
  if (stager) {
    const int sbg = k0 >> 5, h16 = (k0 >> 4) & 1, h8 = (k0 >> 3) & 1;
    uint2* xa8 = reinterpret_cast<uint2*>(smem);
#pragma unroll
    for (int it = 0; it < TOK; it++) {
      const int tk = rep + it * nrep;
      if (tk >= TOK) break;
      float xf[8];
      widen8<XT>(xraw[it], xf);
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
      // entries in 8-byte units: (sub-block, row, 16-k half) x 16 bytes, + the 8-k half
      int e_hi, e_lo;
      if (TOK == 8) {
        e_hi = ((sbg * 16 + 2 * tk) * 2 + h16) * 2 + h8;
        e_lo = e_hi + 4;
      } else {
        e_hi = ((sbg * 32 + tk) * 2 + h16) * 2 + h8;
        e_lo = e_hi + 64;
      }
      xa8[e_hi] = make_uint2(pack_low_bytes(hi[0], hi[1], hi[2], hi[3]), pack_low_bytes(hi[4], hi[5], hi[6], hi[7]));
      xa8[e_lo] = make_uint2(pack_low_bytes(lo[0], lo[1], lo[2], lo[3]), pack_low_bytes(lo[4], lo[5], lo[6], lo[7]));
      if ((tid & 3) == 0) {
        tf[sbg * TOK + tk] = f;
        ts[sbg * TOK + tk] = sum;
      }
    }
  }
  __syncthreads();

  // ---- main loop
  constexpr uint32_t N4 = 0x0F0F0F0Fu;
  // A operand of this lane (row = lane%16, k-group ga = lane/16): its entry inside a sub-block
  const uint32_t act_off = (uint32_t)((lane & 15) * 2 + (g & 1)) * 16u;
  const bool upper_half = (g >> 1) != 0;         // k-groups 2, 3 carry sub-blocks 2, 3 (6, 7)
  // The fp32 matrix instruction v_mfma_f32_16x16x4_f32 does two side jobs per step (A operand:
  // lane (i = lane%16, kk = lane/16) supplies A[i][kk]; B operand: lane (n, kk) supplies B[kk][n]):
  //  * all-gather of the sub-block scales: every lane decodes d*sc of sub-blocks g and 4+g of its
  //    own row; with A[i][kk] = (kk == i%4) the product hands lane (n, g) the values of lanes
  //    (n, 0..3) in its four C registers (1.0 * value + zeros: exact);
  //  * the min term sum_j dmin*m_j * sum(x) of sub-block j: A[i][kk] = sum(x) of the token that C
  //    row i belongs to (sub-block kk, then 4+kk), B[kk][n] = dmin*m of sub-block kk of row n,
  //    accumulated over the whole round in fp32.
  const float sel = ((lane >> 4) == (lane & 3)) ? 1.f : 0.f;
  // token of C row i = lane%16 (TOK = 8: rows 4g', 4g'+1 are tokens 2g', 2g'+1, the others unused)
  const int mrow = lane & 15;
  const bool row_used = TOK == 16 || (mrow & 3) < 2;
  const int row_tok = TOK == 16 ? mrow : 2 * (mrow >> 2) + (mrow & 3);
  // byte offset of ts[(sb*8 + kk) * TOK + token] relative to ts + sb*8*TOK (unused rows: zero entry)
  const uint32_t ts_base = (uint32_t)(reinterpret_cast<uint8_t*>(ts) - smem);
  const uint32_t ts_lane = row_used ? ts_base + (uint32_t)(g * TOK + row_tok) * 4u : zero_off;
  const uint32_t ts_step = row_used ? (uint32_t)(8 * TOK * 4) : 0u;
  int cr = 0, csi = 0;
  float acc[TPL];
#pragma unroll
  for (int i = 0; i < TPL; i++) acc[i] = 0.f;
  v4f_t cmin = {0.f, 0.f, 0.f, 0.f};

  auto store_row = [&](int row, int tk, float v) {
    if (row < wg_row_end && t0 + tk < m)
      YElem<YT>::store(y + (int64_t)(t0 + tk) * n_out, row, v + load_bias(bias, bias_dtype, row));
  };

  auto consume = [&](const BatchStep& s) {
    const int sb = (csi << sl_log2) + sl;
    if (cr < rounds && sb < nsb) {
      v4i_t Bq[4];   // L0, H0, L1, H1
      const uint32_t c0[4] = {s.c0.x, s.c0.y, s.c0.z, s.c0.w}, c1[4] = {s.c1.x, s.c1.y, s.c1.z, s.c1.w};
#pragma unroll
      for (int i = 0; i < 4; i++) {
        Bq[0][i] = (int)(c0[i] & N4);
        Bq[1][i] = (int)((c0[i] >> 4) & N4);
        Bq[2][i] = (int)(c1[i] & N4);
        Bq[3][i] = (int)((c1[i] >> 4) & N4);
      }
      const float d = f16_bits_to_f32((uint16_t)(s.hdr.x & 0xFFFFu));
      const float dmin = f16_bits_to_f32((uint16_t)(s.hdr.x >> 16));
      // scales and mins of sub-blocks g and 4+g of this lane's row (the 6-bit fields of
      // q4k_scale_min with a run-time sub-block)
      const uint32_t sh = 8u * (uint32_t)g;
      const uint32_t sc_lo = (s.hdr.y >> sh) & 63u, mn_lo = (s.hdr.z >> sh) & 63u;
      const uint32_t sc_hi = ((s.hdr.w >> sh) & 0xFu) | (((s.hdr.y >> (sh + 6u)) & 3u) << 4);
      const uint32_t mn_hi = ((s.hdr.w >> (sh + 4u)) & 0xFu) | (((s.hdr.z >> (sh + 6u)) & 3u) << 4);
      const v4f_t fzero = {0.f, 0.f, 0.f, 0.f};
      const v4f_t dsc03 = __builtin_amdgcn_mfma_f32_16x16x4f32(sel, d * (float)sc_lo, fzero, 0, 0, 0);
      const v4f_t dsc47 = __builtin_amdgcn_mfma_f32_16x16x4f32(sel, d * (float)sc_hi, fzero, 0, 0, 0);
      {
        const uint32_t ta = ts_lane + (uint32_t)sb * ts_step;
        const float s_lo = *reinterpret_cast<const float*>(smem + ta);
        const float s_hi = *reinterpret_cast<const float*>(smem + ta + (row_used ? (uint32_t)(4 * TOK * 4) : 0u));
        cmin = __builtin_amdgcn_mfma_f32_16x16x4f32(s_lo, dmin * (float)mn_lo, cmin, 0, 0, 0);
        cmin = __builtin_amdgcn_mfma_f32_16x16x4f32(s_hi, dmin * (float)mn_hi, cmin, 0, 0, 0);
      }
      const v4i_t zero = {0, 0, 0, 0};
      // Sub-block j: nibble plane j%2 of qs bytes 64*(j/4) + 32*((j%4)/2) .. +32, i.e. B operand
      // 2*(j/4) + j%2, k-groups 2*((j%4)/2) and +1.  The sub-blocks are taken kGroup at a time:
      // all LDS reads of a group, then its MFMAs back to back, then the scaling -- left alone the
      // compiler issues read, wait, MFMA, wait, scale for one sub-block after the other and the
      // wavefront sits out every latency eight times per step.
      constexpr int kGroup = TOK == 8 ? 4 : 2;
#pragma unroll
      for (int j0 = 0; j0 < 8; j0 += kGroup) {
        v4i_t A[kGroup][TOK / 8];
        float ff[kGroup][TPL];
#pragma unroll
        for (int jj = 0; jj < kGroup; jj++) {
          const int j = j0 + jj;
          const bool mine = (((j & 3) >> 1) != 0) == upper_half;
          const uint32_t sbg = (uint32_t)sb * 8u + j;
          const uint32_t a_addr = mine ? sbg * kSubBytes + act_off : zero_off;
          A[jj][0] = *reinterpret_cast<const v4i_t*>(smem + a_addr);
          if (TOK == 16) A[jj][TOK / 8 - 1] = *reinterpret_cast<const v4i_t*>(smem + a_addr + (mine ? 512u : 0u));
          if (TOK == 8) {
            const float2 f2 = *reinterpret_cast<const float2*>(tf + sbg * TOK + 2 * g);
            ff[jj][0] = f2.x; ff[jj][TPL - 1] = f2.y;
          } else {
            const float4 f4 = *reinterpret_cast<const float4*>(tf + sbg * TOK + 4 * g);
            ff[jj][0] = f4.x; ff[jj][1] = f4.y; ff[jj][TPL - 2] = f4.z; ff[jj][TPL - 1] = f4.w;
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        v4i_t C[kGroup][TOK / 8];
#pragma unroll
        for (int jj = 0; jj < kGroup; jj++) {
          const int j = j0 + jj;
          const v4i_t& B = Bq[2 * (j >> 2) + (j & 1)];
#pragma unroll
          for (int pl = 0; pl < TOK / 8; pl++) C[jj][pl] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[jj][pl], B, zero, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int jj = 0; jj < kGroup; jj++) {
          const int j = j0 + jj;
          const float dsc = j < 4 ? dsc03[j & 3] : dsc47[j & 3];
          // exact integers below 2^24, scaled by a power of two: sum(q*x) of the sub-block
          if (TOK == 8) {
            const float q0 = (float)(C[jj][0][0] * 256 + C[jj][0][1]) * ff[jj][0];
            const float q1 = (float)(C[jj][0][2] * 256 + C[jj][0][3]) * ff[jj][TPL - 1];
            acc[0] = acc[0] + dsc * q0;
            acc[TPL - 1] = acc[TPL - 1] + dsc * q1;
          } else {
#pragma unroll
            for (int i = 0; i < TPL; i++) {
              const float q = (float)(C[jj][0][i] * 256 + C[jj][TOK / 8 - 1][i]) * ff[jj][i];
              acc[i] = acc[i] + dsc * q;
            }
          }
        }
      }
    }
    if (++csi == S) {
      // the row group is finished for this wavefront's slice
      if (sl_log2 == 0) {
        if (cr < rounds) {
          const int row = wg_row0 + (cr * G + gi) * 16 + n;
#pragma unroll
          for (int i = 0; i < TPL; i++) store_row(row, TPL * g + i, acc[i] - cmin[i]);
        }
#pragma unroll
        for (int i = 0; i < TPL; i++) acc[i] = 0.f;
        cmin = v4f_t{0.f, 0.f, 0.f, 0.f};
      }
      // with slices there is one round only: the sums stay in registers until the table is free
      csi = 0;
      cr++;
    }
  };

  // steady state: every consumed slot is re-requested R steps ahead (past the end: one harmless
  // line, never consumed); the last R steps drain
  for (int t = R; t < t_total; t += R) {
#pragma unroll
    for (int i = 0; i < R; i++) {
      consume(ring[i]);
      issue(ring[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < R; i++) consume(ring[i]);

  if (sl_log2 != 0) {
    __syncthreads();                   // every wavefront is done with the plane table
#pragma unroll
    for (int i = 0; i < TPL; i++) part[(wave * 64 + lane) * TPL + i] = acc[i] - cmin[i];
    __syncthreads();
    // add the slices in a fixed order
    for (int idx = tid; idx < 16 * G * TOK; idx += kMfmaThreads) {
      const int nn = idx & 15, tk = (idx >> 4) % TOK, grp = idx / (16 * TOK);
      const int src = (nn + 16 * (tk / TPL)) * TPL + tk % TPL;
      float v = 0.f;
      for (int s2 = 0; s2 < SL; s2++) v += part[(grp * SL + s2) * 64 * TPL + src];
      store_row(wg_row0 + grp * 16 + nn, tk, v);
    }
  }
}

// ------------------------------------------------------------------------------ launch
template <int TOK>
static size_t batch_lds_bytes(int nsb) {
  const size_t table = (size_t)nsb * 8 * 64 * TOK, tabs = (size_t)nsb * 8 * TOK * 8;
  const size_t part = (size_t)kMfmaWaves * 64 * (TOK / 4) * 4;
  return (table > part ? table : part) + 64 + tabs;
}

template <int TOK, typename XT, typename YT>
static hipError_t batch_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                                  int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  constexpr int W = kMfmaWaves;
  const int nsb = (int)(n_in / 256);
  int num_wg = device_num_cus();
  const int64_t groups = (n_out + 15) / 16;
  if (num_wg > groups) num_wg = (int)groups;
  const int rows_per_wg = (int)((n_out + num_wg - 1) / num_wg);
  num_wg = (int)((n_out + rows_per_wg - 1) / rows_per_wg);
  int sl_log2 = 0;
  while ((2 << sl_log2) <= W && (2 << sl_log2) <= nsb && (16 * W >> (sl_log2 + 1)) >= rows_per_wg) sl_log2++;
  auto kernel = gemv_q4k_batch_kernel<TOK, XT, YT>;
  static LargeLds configured;
  {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)num_wg, (unsigned)((m + TOK - 1) / TOK)), dim3(W * 64),
                     batch_lds_bytes<TOK>(nsb), s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                     static_cast<YT*>(y), bias, bias_dtype, (int)m, (int)n_out, nsb, rows_per_wg, sl_log2);
  return hipGetLastError();
}

template <int TOK, typename XT>
static hipError_t batch_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return batch_launch_xy<TOK, XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return batch_launch_xy<TOK, XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return batch_launch_xy<TOK, XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

// Tokens per workgroup for this shape, 0 if the kernel does not apply: 16 when their plane table
// fits LDS and there are more than 8 tokens, else 8.
static int batch_tokens(int64_t m, int64_t n_in) {
  const int nsb = (int)(n_in / 256);
  const bool fits16 = batch_lds_bytes<16>(nsb) <= 160 * 1024, fits8 = batch_lds_bytes<8>(nsb) <= 160 * 1024;
  if (m > 8 && fits16) return 16;
  return fits8 ? 8 : 0;
}

int gemv_q4k_batch_tokens(int64_t m, int64_t n_in) { return batch_tokens(m, n_in); }

bool gemv_q4k_batch_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in) {
  static const int disabled = mfma_env_int("TTQ_GEMV_NO_BATCH", 0) || mfma_env_int("TTQ_GEMV_NO_MFMA", 0);
  // one staging pass of 8 activations per thread; 32-bit byte offsets into the weights
  return !disabled && format == kQ4_K && (x_dtype == kBF16 || x_dtype == kF16) && m >= 2 && n_out >= 2048 &&
         n_in % 256 == 0 && n_in <= 8 * kMfmaThreads && batch_tokens(m, n_in) != 0 &&
         n_out * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_q4k_batch(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  const int tok = batch_tokens(m, n_in);
  if (tok == 16) {
    if (x_dtype == kBF16) return batch_launch_x<16, bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    if (x_dtype == kF16) return batch_launch_x<16, f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  } else if (tok == 8) {
    if (x_dtype == kBF16) return batch_launch_x<8, bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
    if (x_dtype == kF16) return batch_launch_x<8, f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace ttq
