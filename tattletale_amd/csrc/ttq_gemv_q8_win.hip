// Decode GEMV for Q8_0 weights on gfx950 through the int8 matrix cores, aligned-window form.
//
// Same operator and arithmetic as ttq_gemv_q8_mfma.hip (F.linear with a single-token activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81; activations as block fixed point in byte
// planes, exact integer plane sums per block, one fp32 multiply by d * 2^(E-shift) per block).
// What changes is how the weights reach the matrix cores.  A Q8_0 block is 34 bytes (fp16 d,
// 32 int8), so the quants of a row never sit on 16-byte boundaries, and loading "the quants of
// block b" makes every 64-lane load touch two or three cache lines per row.  Here a wavefront
// reads the rows as they lie: a chunk of 8 blocks is 272 bytes = 17 aligned 16-byte pieces, five
// loads per lane and 16 rows, each touching one 64-byte segment per row.  The bytes then go into
// the MFMA as they are -- quants AND scale bytes -- and the A operand sorts them out:
//   * window w (the 64 bytes 64w .. 64w+63 of the chunk, w = 0..3, plus the 16 bytes of piece 16)
//     holds parts of up to three blocks.  Its A operand has, for a k position that is quant q of
//     block b, plane t of x[32b + q] in row 4*(b%4) + t and zero elsewhere (so also at the
//     positions of scale bytes).  Block b always lands in C rows 4*(b%4) .. +3, i.e. in lane
//     (n, g = b%4); blocks 0-3 accumulate in one C, blocks 4-7 in another (window 2 holds a part
//     of block 3 and parts of blocks 4 and 5: it is multiplied twice, with two tables).
//   * the scales: a 0/1 A operand picks the two bytes of d of block g (C rows 4g, 4g+1) and of
//     block 4+g (rows 4g+2, 4g+3) out of the same B operands: four more MFMAs, exact.
// Ten MFMAs per chunk of 16 rows; the matrix cores are idle otherwise.  Lane (n, g) ends up with
// the plane sums and the scale bits of blocks g and 4+g of its own row: no cross-lane traffic.
#include "ttq_gemv_mfma_common.h"

namespace ttq {

constexpr int kQ8WinMaxChunks = 64;     // n_in <= 16384, the limit of the GEMV entry points

template <typename XT> struct Q8WX;
template <> struct Q8WX<float> {
  static constexpr int kPlanes = 3, kShift = 21;
  typedef float elem_t;
  static __device__ __forceinline__ void load8(const float* p, float (&f)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
};
template <> struct Q8WX<bf16_tag> {
  static constexpr int kPlanes = 2, kShift = 13;
  typedef uint16_t elem_t;
  static __device__ __forceinline__ void load8(const uint16_t* p, float (&f)[8]) {
    widen8<bf16_tag>(*reinterpret_cast<const uint4*>(p), f);
  }
};
template <> struct Q8WX<f16_tag> {
  static constexpr int kPlanes = 2, kShift = 13;
  typedef uint16_t elem_t;
  static __device__ __forceinline__ void load8(const uint16_t* p, float (&f)[8]) {
    widen8<f16_tag>(*reinterpret_cast<const uint4*>(p), f);
  }
};

struct Q8WinStep { uint4 p[5]; };

// The plane tables are stored compactly.  Block b has quants in the 16-byte pieces
// (34b+2)/16 .. (34b+33)/16 of the chunk: three pieces each for blocks 0-6, two for block 7, 23
// (block, piece) pairs in all.  A pair holds one 16-byte entry per plane: the plane bytes at the
// positions of the block's quants in that piece, zero elsewhere.  As the A operand of the MFMA for
// window w, lane (row = 4*slot + plane, k-group ga) supplies the entry of (the block of that slot
// in piece 4w + ga, plane) if there is one, else zeros.
__device__ __forceinline__ int q8win_first_piece(int b) { return (34 * b + 2) >> 4; }
__device__ __forceinline__ int q8win_pair(int b, int piece) { return 3 * b + (piece - q8win_first_piece(b)); }
constexpr int kQ8WinPairs = 23;
// For short rows the tables are kept wide instead: [nch][6 MFMAs][64 lanes] x 16 bytes with the
// zeros stored, so that every A address is one register plus an immediate (6 KiB per chunk;
// 0.35 us faster at 4096 x 4096).
constexpr int kQ8WinMaxWideChunks = 24;

// wide layout: table index of the window that holds chunk byte `byte` of block `b` (b = 0..7):
// windows 0, 1, 2 (block 3 only), 2 (blocks 4, 5), 3, 4
__device__ __forceinline__ int q8win_table(int byte, int b) {
  const int w = byte >> 6;
  return w < 2 ? w : (w == 2 ? (b == 3 ? 2 : 3) : w + 1);
}

// LDS layout (bytes): plane tables [nch][23 pairs][T planes] x 16, one zero entry (64 bytes
// reserved), then the per-block factors [nch][8] floats 2^(E - shift), then the partial row sums of
// the wavefronts [16][16] floats.
// TOK activation rows ("tokens") per pass over the weights (compact tables only when TOK > 1): the
// B operands and the scale MFMAs are shared, every token has its own plane tables, six plane
// MFMAs and two scalings per step.  blockIdx.y walks the groups of TOK tokens; tokens past the
// end re-read the last one and are not stored.
template <bool COMPACT, int TOK, typename XT, typename YT>
__global__ void __launch_bounds__(kMfmaThreads)
gemv_q8_win_kernel(const uint8_t* __restrict__ w, const typename Q8WX<XT>::elem_t* __restrict__ x,
                   YT* __restrict__ y, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int nch,
                   int rows_per_wg, int sl_log2, int exch_min_steps) {
  static_assert(COMPACT || TOK == 1, "several tokens use the compact tables");
  using X = Q8WX<XT>;
  constexpr int W = kMfmaWaves, T = X::kPlanes;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr uint32_t kChunkBytes = COMPACT ? kQ8WinPairs * T * 16 : 6 * 1024;
  const uint32_t tok_bytes = (uint32_t)nch * kChunkBytes;          // plane tables of one token
  const uint32_t table_bytes = TOK * tok_bytes;
  const uint32_t zero_off = table_bytes;
  float* tab = reinterpret_cast<float*>(smem + table_bytes + 64);   // [TOK][nch * 8]
  float* part = reinterpret_cast<float*>(smem + table_bytes + 64 + (size_t)TOK * nch * 32);   // [TOK][16][16]

  const int SL = 1 << sl_log2, G = W >> sl_log2;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int gi = wave >> sl_log2, sl = wave & (SL - 1);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nch * 256;
  const int t0 = blockIdx.y * TOK;
  const uint32_t rb = (uint32_t)nch * 272u;
  const int S = (nch + SL - 1) >> sl_log2;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int rounds = (rows_per_wg + 16 * G - 1) / (16 * G);
  const int t_total = rounds * S;
  const bool exch = t_total >= exch_min_steps;
  const int last = wg_row_end - 1;   // rows past the workgroup's share re-read its last row

  // ---- activations: 8 values per thread and pass, requested before any weights
  constexpr int XP = ((COMPACT ? kQ8WinMaxChunks : kQ8WinMaxWideChunks) * 256 + 8 * kMfmaThreads - 1) / (8 * kMfmaThreads);
  float xf[TOK][XP][8];
#pragma unroll
  for (int t = 0; t < TOK; t++) {
    const typename X::elem_t* xm = x + (int64_t)min(t0 + t, m - 1) * n_in;
#pragma unroll
    for (int p = 0; p < XP; p++) {
      const int k0 = 8 * (tid + p * kMfmaThreads);
      X::load8(xm + (k0 < n_in ? k0 : 0), xf[t][p]);
    }
  }
  __builtin_amdgcn_s_barrier();

  // ---- weight stream: one step (16 rows x one chunk) in flight; loads are unconditional (clamped)
  Q8WinStep cur;
  int ir = 0, isi = 0;
  auto issue = [&](Q8WinStep& dst) {
    const int ch = (isi << sl_log2) + sl;
    const bool ok = ir < rounds && ch < nch;
    // pieces 0..15 with lane = 4 * row + k-group, so that the 64 bytes of a row that one request
    // covers lie in a quad of neighbouring lanes (the memory pipeline merges neighbours' accesses
    // only); they are exchanged into the operand layout lane = row + 16 * k-group when the step is
    // consumed.  Piece 16 is the same for a row's four lanes and is requested in operand layout.
    // The exchange costs a wavefront latency once per step, which only pays when it has several
    // steps to overlap it with; with fewer, everything is requested in operand layout.
    const int row = min(wg_row0 + (ir * G + gi) * 16 + n, last);
    const int qrow = min(wg_row0 + (ir * G + gi) * 16 + (exch ? lane >> 2 : n), last);
    const uint32_t o = (ok ? (uint32_t)qrow * rb + (uint32_t)ch * 272u : 0u) + 16u * (uint32_t)(exch ? lane & 3 : g);
#pragma unroll
    for (int i = 0; i < 4; i++) dst.p[i] = load16_a16(w + (o + 64u * i));
    dst.p[4] = load16_a16(w + ((ok ? (uint32_t)row * rb + (uint32_t)ch * 272u : 0u) + 256u));
    if (++isi == S) { isi = 0; ir++; }
  };
  issue(cur);

  // ---- clear the plane tables
  {
    const v4i_t z = {0, 0, 0, 0};
    v4i_t* xa = reinterpret_cast<v4i_t*>(smem);
    for (int e = tid; e < TOK * nch * (int)(kChunkBytes / 16) + 1; e += kMfmaThreads) xa[e] = z;   // + the zero entry
  }
  __syncthreads();

  // ---- quantize the activations into byte planes and scatter them to their windows
#pragma unroll
  for (int t = 0; t < TOK; t++)
#pragma unroll
  for (int p = 0; p < XP; p++) {
    const int k0 = 8 * (tid + p * kMfmaThreads);
    if (k0 < n_in) {
      uint32_t amax = amax_bits(xf[t][p]);
      // the four threads of a block are an aligned quad
      amax = umax(amax, dpp_quad_u32<0xB1>(amax));
      amax = umax(amax, dpp_quad_u32<0x4E>(amax));
      const uint32_t eb = amax >> 23;                             // biased exponent of max |x|; 255 for Inf and NaN
      const uint32_t ec = eb < (uint32_t)(X::kShift + 1) ? (uint32_t)(X::kShift + 1) : eb;
      const float mul = __uint_as_float((254u + (uint32_t)X::kShift - ec) << 23);   // 2^(shift-E)
      // non-finite activations poison the block instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - (uint32_t)X::kShift) << 23);
      int pl[3][8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int v = (int)rintf(xf[t][p][i] * mul);
        if (T == 3) {
          const int v1 = (v + 128) >> 8;
          pl[2][i] = v;                  // only the low byte is used
          pl[1][i] = v1;
          pl[0][i] = (v1 + 128) >> 8;
        } else {
          pl[1][i] = v;
          pl[0][i] = (v + 128) >> 8;
          pl[2][i] = 0;
        }
      }
      const int blk = k0 >> 5, ch = blk >> 3, b = blk & 7, q0 = k0 & 31;
      // the 8 quants sit at chunk bytes 34b + 2 + q0 .. +7: an even start, so pairs of bytes never
      // straddle a 16-byte piece (nor a window)
#pragma unroll
      for (int i2 = 0; i2 < 4; i2++) {
        const int byte = 34 * b + 2 + q0 + 2 * i2;
        const int pos = byte & 63;
        uint8_t* e = smem + (size_t)t * tok_bytes + (size_t)ch * kChunkBytes +
                     (COMPACT ? (size_t)(q8win_pair(b, byte >> 4) * T * 16 + (byte & 15))
                              : (size_t)((q8win_table(byte, b) * 64 + 16 * (pos >> 4) + 4 * (b & 3)) * 16 + (pos & 15)));
#pragma unroll
        for (int pi = 0; pi < T; pi++)
          *reinterpret_cast<uint16_t*>(e + 16 * pi) =
              (uint16_t)((pl[pi][2 * i2] & 0xFF) | ((pl[pi][2 * i2 + 1] & 0xFF) << 8));
      }
      if ((tid & 3) == 0) tab[t * nch * 8 + blk] = f;
    }
  }
  __syncthreads();

  // ---- the 0/1 A operands that pick the scale bytes: C row m = lane%16 = 4*gg + 2*hh + byte is
  // byte `byte` of d of block b = gg + 4*hh, at chunk byte 34b + byte, in window (34b)/64
  v4i_t sel[4];
  {
    const int m = lane & 15, b = (m >> 2) + 4 * ((m >> 1) & 1);
    const int at = 34 * b + (m & 1);
    const int w_at = at >> 6, pos = at & 63;
    const bool here = (pos >> 4) == g;
    const uint32_t one = 1u << (8 * (pos & 3));
    const int dw = (pos & 15) >> 2;
#pragma unroll
    for (int wi = 0; wi < 4; wi++) {
      const bool on = here && w_at == wi;
#pragma unroll
      for (int c = 0; c < 4; c++) sel[wi][c] = (on && c == dw) ? (int)one : 0;
    }
  }

  // ---- A operand addresses of this lane for the six plane MFMAs: windows 0, 1, 2 (block 3 only),
  // 2 (blocks 4, 5), 3, 4
  uint32_t a_base[6], a_stride[6], a_tok[6];
  {
    const int slot = (lane & 15) >> 2, pln = lane & 3;
#pragma unroll
    for (int ti = 0; ti < 6; ti++) {
      const int wdw = ti < 2 ? ti : (ti < 4 ? 2 : ti - 1);
      const int piece = 4 * wdw + g;
      int off = -1;
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const int b = slot + 4 * hh;
        const bool in_table = ti == 2 ? b == 3 : (ti == 3 ? b >= 4 : true);
        const bool touches = piece >= q8win_first_piece(b) && piece <= ((34 * b + 33) >> 4) && (wdw < 4 || g == 0);
        if (pln < T && in_table && touches) off = (q8win_pair(b, piece) * T + pln) * 16;
      }
      if (!COMPACT) off = (ti * 64 + lane) * 16;
      a_base[ti] = off >= 0 ? (uint32_t)off : zero_off;
      a_stride[ti] = off >= 0 ? kChunkBytes : 0u;
      a_tok[ti] = off >= 0 ? tok_bytes : 0u;
    }
  }

  // ---- main loop
  int cr = 0, csi = 0;
  float acc[TOK];
#pragma unroll
  for (int t = 0; t < TOK; t++) acc[t] = 0.f;
  auto store_row = [&](int row, int t, float v) {
    if (row < wg_row_end && t0 + t < m)
      YElem<YT>::store(y + (int64_t)(t0 + t) * n_out, row, v + load_bias(bias, bias_dtype, row));
  };
  const int from_lane4 = 4 * (4 * n + g);
  auto exchange = [&](Q8WinStep& t) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      t.p[i].x = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)t.p[i].x);
      t.p[i].y = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)t.p[i].y);
      t.p[i].z = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)t.p[i].z);
      t.p[i].w = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane4, (int)t.p[i].w);
    }
  };
  auto consume = [&](const Q8WinStep& s) {
    const int ch = (csi << sl_log2) + sl;
    if (cr < rounds && ch < nch) {
      v4i_t B[5];
#pragma unroll
      for (int i = 0; i < 5; i++) {
        B[i][0] = (int)s.p[i].x; B[i][1] = (int)s.p[i].y; B[i][2] = (int)s.p[i].z; B[i][3] = (int)s.p[i].w;
      }
      const v4i_t zero = {0, 0, 0, 0};
      v4i_t cd = __builtin_amdgcn_mfma_i32_16x16x64_i8(sel[0], B[0], zero, 0, 0, 0);
      cd = __builtin_amdgcn_mfma_i32_16x16x64_i8(sel[1], B[1], cd, 0, 0, 0);
      cd = __builtin_amdgcn_mfma_i32_16x16x64_i8(sel[2], B[2], cd, 0, 0, 0);
      cd = __builtin_amdgcn_mfma_i32_16x16x64_i8(sel[3], B[3], cd, 0, 0, 0);
      const float d0 = f16_bits_to_f32((uint16_t)(((uint32_t)cd[1] & 0xFFu) << 8 | ((uint32_t)cd[0] & 0xFFu)));
      const float d1 = f16_bits_to_f32((uint16_t)(((uint32_t)cd[3] & 0xFFu) << 8 | ((uint32_t)cd[2] & 0xFFu)));
#pragma unroll
      for (int t = 0; t < TOK; t++) {
        v4i_t A[6];
#pragma unroll
        for (int ti = 0; ti < 6; ti++) {
          if (COMPACT)
            A[ti] = *reinterpret_cast<const v4i_t*>(smem + a_base[ti] + (uint32_t)ch * a_stride[ti] + (uint32_t)t * a_tok[ti]);
          else
            A[ti] = reinterpret_cast<const v4i_t*>(smem)[(size_t)ch * 384 + ti * 64 + lane];
        }
        v4i_t c03 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[0], B[0], zero, 0, 0, 0);
        v4i_t c47 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[3], B[2], zero, 0, 0, 0);
        c03 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[1], B[1], c03, 0, 0, 0);
        c47 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[4], B[3], c47, 0, 0, 0);
        c03 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[2], B[2], c03, 0, 0, 0);
        c47 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[5], B[4], c47, 0, 0, 0);
        const float f0 = tab[t * nch * 8 + ch * 8 + g], f1 = tab[t * nch * 8 + ch * 8 + 4 + g];
        float s0, s1;
        if (T == 3) {
          s0 = ((float)c03[0] * 65536.f + (float)c03[1] * 256.f) + (float)c03[2];
          s1 = ((float)c47[0] * 65536.f + (float)c47[1] * 256.f) + (float)c47[2];
        } else {
          s0 = (float)(c03[0] * 256 + c03[1]);
          s1 = (float)(c47[0] * 256 + c47[1]);
        }
        acc[t] = acc[t] + d0 * (s0 * f0);
        acc[t] = acc[t] + d1 * (s1 * f1);
      }
    }
    if (++csi == S) {
#pragma unroll
      for (int t = 0; t < TOK; t++) {
        float v = acc[t];
        v = add_xor16(v);
        v = add_xor32(v);
        if (cr < rounds) {
          if (sl_log2 == 0) {
            if (lane < 16) store_row(wg_row0 + (cr * G + gi) * 16 + n, t, v);
          } else {
            if (lane < 16) part[(t * W + wave) * 16 + n] = v;
          }
        }
        acc[t] = 0.f;
      }
      csi = 0;
      cr++;
    }
  };
  for (int t = 1; t < t_total; t++) {
    Q8WinStep now = cur;
    if (exch) exchange(now);
    issue(cur);
    consume(now);
  }
  if (exch) exchange(cur);
  consume(cur);

  if (sl_log2 != 0) {
    // one round only: add the slices in a fixed order
    __syncthreads();
    for (int idx = tid; idx < 16 * G * TOK; idx += kMfmaThreads) {
      const int nn = idx & 15, grp = (idx >> 4) % G, t = idx / (16 * G);
      float v = 0.f;
      for (int s2 = 0; s2 < SL; s2++) v += part[(t * W + grp * SL + s2) * 16 + nn];
      store_row(wg_row0 + grp * 16 + nn, t, v);
    }
  }
}

// ------------------------------------------------------------------------------ launch
template <typename XT, typename YT>
static hipError_t q8win_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype,
                                  int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  constexpr int W = kMfmaWaves;
  const int nch = (int)(n_in / 256);
  int num_wg = device_num_cus();
  const int64_t groups = (n_out + 15) / 16;
  if (num_wg > groups) num_wg = (int)groups;
  const int rows_per_wg = (int)((n_out + num_wg - 1) / num_wg);
  num_wg = (int)((n_out + rows_per_wg - 1) / rows_per_wg);
  int sl_log2 = 0;
  while ((2 << sl_log2) <= W && (2 << sl_log2) <= nch && (16 * W >> (sl_log2 + 1)) >= rows_per_wg) sl_log2++;
  constexpr int T = Q8WX<XT>::kPlanes;
  const auto lds_for = [&](bool compact, int tok) {
    return (size_t)tok * nch * (compact ? kQ8WinPairs * T * 16 : 6 * 1024) + 64 + (size_t)tok * nch * 32 +
           (size_t)tok * 1024;
  };
  // tokens per pass: four (two) when their compact tables fit LDS
  int tok = 1;
  if (m >= 2) tok = (m > 2 && lds_for(true, 4) <= 150 * 1024) ? 4 : (lds_for(true, 2) <= 150 * 1024 ? 2 : 1);
  const bool compact = tok > 1 || nch > kQ8WinMaxWideChunks;
  const size_t lds = lds_for(compact, tok);
  const dim3 grid((unsigned)num_wg, (unsigned)((m + tok - 1) / tok));
  static const int exch_min_steps = mfma_env_int("TTQ_GEMV_Q8_EXCHANGE_MIN_STEPS", 2);
  const auto launch = [&](auto kernel, LargeLds& configured) -> hipError_t {
    {
      const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(W * 64), lds, s, static_cast<const uint8_t*>(w),
                       static_cast<const typename Q8WX<XT>::elem_t*>(x), static_cast<YT*>(y), bias, bias_dtype, (int)m,
                       (int)n_out, nch, rows_per_wg, sl_log2, exch_min_steps);
    return hipGetLastError();
  };
  static LargeLds configured_wide, configured_compact, configured_2, configured_4;
  if (tok == 4) return launch(gemv_q8_win_kernel<true, 4, XT, YT>, configured_4);
  if (tok == 2) return launch(gemv_q8_win_kernel<true, 2, XT, YT>, configured_2);
  if (compact) return launch(gemv_q8_win_kernel<true, 1, XT, YT>, configured_compact);
  return launch(gemv_q8_win_kernel<false, 1, XT, YT>, configured_wide);
}

template <typename XT>
static hipError_t q8win_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q8win_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return q8win_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return q8win_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

// Tokens per pass the launcher above picks (see q8win_launch_xy).
int gemv_q8_win_tokens(int x_dtype, int64_t m, int64_t n_in) {
  const int nch = (int)(n_in / 256), planes = x_dtype == kF32 ? 3 : 2;
  const auto lds_for = [&](int tok) {
    return (size_t)tok * nch * kQ8WinPairs * planes * 16 + 64 + (size_t)tok * nch * 32 + (size_t)tok * 1024;
  };
  if (m < 2) return 1;
  return (m > 2 && lds_for(4) <= 150 * 1024) ? 4 : (lds_for(2) <= 150 * 1024 ? 2 : 1);
}

bool gemv_q8_win_supported(int format, int64_t n_out, int64_t n_in) {
  static const int disabled = mfma_env_int("TTQ_GEMV_NO_MFMA", 0) || mfma_env_int("TTQ_GEMV_NO_Q8_WIN", 0);
  // whole chunks of 8 blocks (rows then start 16-byte aligned); plane tables within LDS; byte
  // offsets into the weight buffer are 32-bit in the kernel
  // (from 1024 weight rows on; the dispatch sends small matrices with up to four activation rows elsewhere)
  return !disabled && format == kQ8_0 && n_out >= 1024 && n_in % 256 == 0 && n_in / 256 <= kQ8WinMaxChunks &&
         n_out * (n_in / 32) * 34 < ((int64_t)1 << 32);
}

hipError_t launch_gemv_q8_win(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                              int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kF32) return q8win_launch_x<float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kBF16) return q8win_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return q8win_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
