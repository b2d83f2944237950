// Decode GEMV for Q4_K weights and up to FOUR activation rows per pass on gfx950, through the
// int8 matrix cores, for rows as long as the GEMV entry points accept (n_in <= 16384).
//
// Same operator and arithmetic as ttq_gemv_q4k_batch.hip (F.linear,
// workspace/libtorch/src/abi/neural_nets.nim:64-81, with a small batch*seq; activations as 15-bit
// block fixed point in two byte planes, exact integer sums per sub-block, scales and mins applied
// once per sub-block in fp32, unit vectors bit-exact).  The 8- and 16-token forms keep 64 bytes of
// LDS per token and sub-block and stop at n_in = 8192 / 4096; the down projection of a gated MLP
// (4096 x 14336 in Llama-3-8B) is longer.  Four tokens need half of that and fit.
//
// Matrix shapes.  One MFMA covers two sub-blocks (k-groups 0-1 and 2-3 of a nibble plane), as in
// the single-row kernel, and the A rows are (token t, which of the two sub-blocks h, plane p):
// row 4t + 2h + p is non-zero in the k-groups of sub-block h only.  Four MFMAs per super-block
// of 16 weight rows -- as many as for one token.  Lane (n = lane%16, g = lane/16) loads 16 qs
// bytes of weight row n, supplies them as B and receives C rows 4g..4g+3: both planes of both
// sub-blocks of TOKEN g for its own weight row.  A lane's A entry is either non-zero in all four
// MFMAs or in none (that depends only on the lane), so half of the lanes read one shared zero
// entry throughout.
//
// Work distribution as in ttq_gemv_mfma.hip; blockIdx.y walks the groups of four tokens.
#include "ttq_gemv_mfma_common.h"

namespace ttq {

struct Batch4Step { uint4 hdr, c0, c1; };

// LDS (bytes): plane table [nsb][4 MFMAs][16 rows][2 halves] x 16 (2 KiB per super-block), one
// zero entry (64 bytes reserved), then per (super-block, MFMA, token) a float4
// {2^(E-13) of the two sub-blocks, sum(x) of the two sub-blocks}.  The per-wavefront partial sums
// of the last step overlay the table.
template <typename XT, typename YT>
__global__ void __launch_bounds__(kMfmaThreads)
gemv_q4k_batch4_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                       const void* __restrict__ bias, int bias_dtype, int m, int n_out, int nsb, int rows_per_wg,
                       int sl_log2) {
  constexpr int W = kMfmaWaves, TOK = 4;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t table_bytes = (uint32_t)nsb * 2048u;
  const uint32_t zero_off = table_bytes;
  float4* tab = reinterpret_cast<float4*>(smem + table_bytes + 64);
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

  // ---- activations, requested before any weights: item = (token, 8 consecutive values); the
  // items are dealt to the threads in passes.  Tokens past the end re-read the last one.
  constexpr int XP = (int)(TOK * kMaxMfmaIn / (8 * kMfmaThreads));      // 8 passes cover 4 x 16384
  const int kitems = n_in >> 3;                 // items per token
  uint4 xraw[XP];
#pragma unroll
  for (int p = 0; p < XP; p++) {
    const int it = tid + p * kMfmaThreads;
    const int tk = it / kitems, k0 = 8 * (it - tk * kitems);
    const bool ok = tk < TOK;
    // passes past the end re-read spread addresses of the first token (never used)
    xraw[p] = *reinterpret_cast<const uint4*>(x + (int64_t)min(t0 + (ok ? tk : 0), m - 1) * n_in + (ok ? k0 : (k0 & 2047)));
  }
  __builtin_amdgcn_s_barrier();

  // ---- weight stream, two steps in flight; loads are unconditional (clamped)
  constexpr int R = 2;
  Batch4Step ring[R];
  int ir = 0, isi = 0;
  auto issue = [&](Batch4Step& dst) {
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
#pragma unroll
  for (int p = 0; p < XP; p++) {
    const int it = tid + p * kMfmaThreads;
    const int tk = it / kitems, k0 = 8 * (it - tk * kitems);
    if (tk < TOK) {
      float xf[8];
      widen8<XT>(xraw[p], xf);
      float amax = 0.f, sum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        amax = fmaxf(amax, fabsf(xf[i]));
        sum += xf[i];
      }
      // the four threads of a sub-block are an aligned quad (kitems is a multiple of 32)
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
      // sub-block j of super-block b: MFMA q = 2*(j/4) + j%2, second sub-block of it if (j%4)/2
      const int b = k0 >> 8, j = (k0 >> 5) & 7, h16 = (k0 >> 4) & 1, h8 = (k0 >> 3) & 1;
      const int q = 2 * (j >> 2) + (j & 1), hh = (j & 3) >> 1;
      const int row = 4 * tk + 2 * hh;              // hi plane; lo plane is the next row
      uint2* xa8 = reinterpret_cast<uint2*>(smem);
      const int e_hi = (((b * 4 + q) * 16 + row) * 2 + h16) * 2 + h8;     // in 8-byte units
      xa8[e_hi] = make_uint2(pack_low_bytes(hi[0], hi[1], hi[2], hi[3]), pack_low_bytes(hi[4], hi[5], hi[6], hi[7]));
      xa8[e_hi + 4] = make_uint2(pack_low_bytes(lo[0], lo[1], lo[2], lo[3]), pack_low_bytes(lo[4], lo[5], lo[6], lo[7]));
      if ((tid & 3) == 0) {
        float* e = reinterpret_cast<float*>(tab + (b * 4 + q) * TOK + tk);
        e[hh] = f;
        e[2 + hh] = sum;
      }
    }
  }
  __syncthreads();

  // ---- main loop
  constexpr uint32_t N4 = 0x0F0F0F0Fu;
  // A operand of this lane (row = lane%16 = 4t + 2h + p, k-group ga = lane/16): its sub-block is
  // the one of k-groups 2h, 2h+1
  const bool active = (g >> 1) == ((lane >> 1) & 1);
  const uint32_t a_lane = active ? (uint32_t)((lane & 15) * 2 + (g & 1)) * 16u : zero_off;
  const uint32_t a_step = active ? 2048u : 0u, a_q = active ? 512u : 0u;
  int cr = 0, csi = 0;
  float acc = 0.f;

  auto store_row = [&](int row, int tk, float v) {
    if (row < wg_row_end && t0 + tk < m)
      YElem<YT>::store(y + (int64_t)(t0 + tk) * n_out, row, v + load_bias(bias, bias_dtype, row));
  };

  auto consume = [&](const Batch4Step& s) {
    const int sb = (csi << sl_log2) + sl;
    if (cr < rounds && sb < nsb) {
      const uint32_t c0[4] = {s.c0.x, s.c0.y, s.c0.z, s.c0.w}, c1[4] = {s.c1.x, s.c1.y, s.c1.z, s.c1.w};
      v4i_t Bq[4];   // MFMA q = 2P + nib: L0, H0, L1, H1
#pragma unroll
      for (int i = 0; i < 4; i++) {
        Bq[0][i] = (int)(c0[i] & N4);
        Bq[1][i] = (int)((c0[i] >> 4) & N4);
        Bq[2][i] = (int)(c1[i] & N4);
        Bq[3][i] = (int)((c1[i] >> 4) & N4);
      }
      const uint32_t a0 = a_lane + (uint32_t)sb * a_step;
      v4i_t A[4];
      float4 cst[4];
#pragma unroll
      for (int q = 0; q < 4; q++) {
        A[q] = *reinterpret_cast<const v4i_t*>(smem + a0 + q * a_q);
        cst[q] = tab[(sb * 4 + q) * TOK + g];
      }
      const v4i_t zero = {0, 0, 0, 0};
      v4i_t C[4];
#pragma unroll
      for (int q = 0; q < 4; q++) C[q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[q], Bq[q], zero, 0, 0, 0);
      const float d = f16_bits_to_f32((uint16_t)(s.hdr.x & 0xFFFFu));
      const float dmin = f16_bits_to_f32((uint16_t)(s.hdr.x >> 16));
#pragma unroll
      for (int q = 0; q < 4; q++) {
        // MFMA q: sub-blocks 4*(q/2) + q%2 (C rows 0, 1 of the lane) and + 2 (C rows 2, 3)
        const int j = 4 * (q >> 1) + (q & 1);
        uint32_t sc1, mn1, sc2, mn2;
        q4k_scale_min(s.hdr.y, s.hdr.z, s.hdr.w, j, sc1, mn1);
        q4k_scale_min(s.hdr.y, s.hdr.z, s.hdr.w, j + 2, sc2, mn2);
        // exact integers below 2^24, scaled by a power of two: sum(q*x) of the sub-block
        const float q1 = (float)(C[q][0] * 256 + C[q][1]) * cst[q].x;
        const float q2 = (float)(C[q][2] * 256 + C[q][3]) * cst[q].y;
        acc = acc + (d * (float)sc1) * q1;
        acc = acc - (dmin * (float)mn1) * cst[q].z;
        acc = acc + (d * (float)sc2) * q2;
        acc = acc - (dmin * (float)mn2) * cst[q].w;
      }
    }
    if (++csi == S) {
      // the row group is finished for this wavefront's slice; lane (n, g) holds token g of row n
      if (sl_log2 == 0) {
        if (cr < rounds) store_row(wg_row0 + (cr * G + gi) * 16 + n, g, acc);
        acc = 0.f;
      }
      // with slices there is one round only: the sum stays in its register until the table is free
      csi = 0;
      cr++;
    }
  };

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
    part[wave * 64 + lane] = acc;
    __syncthreads();
    // add the slices in a fixed order
    if (tid < 64 * G) {
      const int grp = tid >> 6, l = tid & 63;
      float v = 0.f;
      for (int s2 = 0; s2 < SL; s2++) v += part[(grp * SL + s2) * 64 + l];
      store_row(wg_row0 + grp * 16 + (l & 15), l >> 4, v);
    }
  }
}

// ------------------------------------------------------------------------------ launch
static size_t batch4_lds_bytes(int nsb) { return (size_t)nsb * 2048 + 64 + (size_t)nsb * 4 * 4 * 16; }

template <typename XT, typename YT>
static hipError_t batch4_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
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
  auto kernel = gemv_q4k_batch4_kernel<XT, YT>;
  static LargeLds configured;
  {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)num_wg, (unsigned)((m + 3) / 4)), dim3(W * 64), batch4_lds_bytes(nsb), s,
                     static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x), static_cast<YT*>(y), bias,
                     bias_dtype, (int)m, (int)n_out, nsb, rows_per_wg, sl_log2);
  return hipGetLastError();
}

template <typename XT>
static hipError_t batch4_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return batch4_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return batch4_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return batch4_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

bool gemv_q4k_batch4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in) {
  static const int disabled = mfma_env_int("TTQ_GEMV_NO_BATCH", 0) || mfma_env_int("TTQ_GEMV_NO_MFMA", 0);
  // 32-bit byte offsets into the weights; the plane table of four tokens within LDS
  return !disabled && format == kQ4_K && (x_dtype == kBF16 || x_dtype == kF16) && m >= 2 && n_out >= 2048 &&
         n_in % 256 == 0 && n_in <= kMaxMfmaIn && batch4_lds_bytes((int)(n_in / 256)) <= 160 * 1024 &&
         n_out * (n_in / 256) * 144 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_q4k_batch4(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return batch4_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return batch4_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
