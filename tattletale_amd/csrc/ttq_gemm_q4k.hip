// Prefill GEMM for Q4_K weights on gfx950:  Y (m, n_out) = X (m, n_in) * W^T -- the dispatch of the GEMM entry
// points (launch_gemm, at the end of this file) and the single-role tiled kernel, which serves activation matrices
// of more than 4 GiB (64-bit row offsets); everything smaller runs the few-row kernel (ttq_gemm_skinny.hip) or the
// producer/consumer kernels (ttq_gemm_pc.hip, ttq_gemm_pcd.hip).
//
// Replaces F.linear(x, weight) for a multi-row bf16 activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81; the prefill case of
//  workspace/transformers/src/layers/attn.nim:154-156).
//
// Tiling.  A workgroup of four wavefronts owns a 256 x BN tile of Y (BN = 112 or 128, picked so
// that the tiles fill the 256 CUs as evenly as possible); each wavefront owns 64 rows of it
// and all BN columns: 4 x BN/16 accumulators of v_mfma_f32_16x16x32_bf16.
//   W side: the tile's packed super-blocks are loaded straight from HBM into registers once
//           per 256 k (5 x 16 B per thread), dequantized 64 k at a time with the canonical
//           arithmetic (d*sc*q - dmin*m, which one fused multiply-add reproduces exactly
//           because d*sc*q has at most 21 significant bits), rounded to bf16 nearest-even and
//           written to LDS in MFMA fragment order, double-buffered.  Each weight is therefore
//           dequantized once per 256 rows of X, and fragment reads are linear and free of
//           bank conflicts.
//   X side: every wavefront reads the A fragments of its own 64 rows directly from
//           global memory (a fragment is 16 contiguous bytes per lane), one 64-k step ahead.
//           X never goes through LDS, which halves the LDS traffic per MFMA.
// One barrier per 64-k step.
#include "ttq_device.h"
#include "ttq_internal.h"

#include <stdlib.h>
#include <type_traits>

namespace ttq {

// Developer timeline instrumentation, compiled in only with -DTTQ_PHASE_TRACE: wavefront 0 of
// workgroup 0 stores the shader clock at a few points of every step.
#ifdef TTQ_PHASE_TRACE
__device__ long long* g_gemm_trace = nullptr;
#define TTQ_GEMM_TRACE(idx)                                                                     \
  do {                                                                                          \
    if (g_gemm_trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0)                         \
      g_gemm_trace[(idx)] = __builtin_readcyclecounter();                                       \
  } while (0)
#else
#define TTQ_GEMM_TRACE(idx) do { } while (0)
#endif

constexpr int kGemmThreads = 256;
constexpr int kGemmBM = 256;      // rows of X per workgroup (4 wavefronts x 64)
constexpr int kWaveM = 64;

// LDS: one buffer holds a BN x 64 bf16 tile of W as [ksub 2][j BN/16][g 4][n 16] units of 16 bytes
// (8 consecutive k of one column), i.e. exactly the B operand of lane g*16+n for column block j.
template <int NJ> struct WTile { static constexpr int kUnits = 2 * NJ * 64; };

template <int NJ, typename YT, bool WEAVE>
__global__ void __launch_bounds__(kGemmThreads)
gemm_q4k_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                int n_tiles, int m_tiles, int xcds_per_mtile) {
  constexpr int BN = NJ * 16;
  __shared__ uint4 sw[2][WTile<NJ>::kUnits];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Tile assignment.  Workgroups are dealt to the 8 XCDs round-robin (XCD = id % 8) and every XCD
  // has its own L2.  All workgroups of one row tile read the same 256 x n_in slab of X, so when
  // the row tiles divide the XCDs evenly each XCD is given workgroups of ONE row tile only: its L2
  // then holds a single slab of X instead of all of them, and X stops falling out to HBM.
  int n_tile, m_tile;
  if (xcds_per_mtile > 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    m_tile = xcd / xcds_per_mtile;
    n_tile = slot * xcds_per_mtile + xcd % xcds_per_mtile;
  } else {
    m_tile = blockIdx.x % m_tiles;
    n_tile = blockIdx.x / m_tiles;
  }
  if (n_tile >= n_tiles) return;
  const int n0 = n_tile * BN, m0 = m_tile * kGemmBM + wave * kWaveM;
  const int64_t row_bytes = (int64_t)(n_in >> 8) * 144;

  // ---- W loader role: thread -> (tile row, 16-byte half of every 32-byte chunk)
  // (with BN = 112 the last 32 threads mirror threads 0..31: same loads, same LDS writes of the
  // same values, so that the step body stays free of branches)
  const int wt = tid < 2 * BN ? tid : tid - 2 * BN;
  const int wr = wt % BN, whalf = wt / BN;
  const int wrow = min(n0 + wr, n_out - 1);           // clamped: rows past the end are never stored
  const uint8_t* wptr = w + row_bytes * (int64_t)wrow;
  const int wj = wr >> 4, wn = wr & 15;

  // ---- X fragment role: lane -> (row lane%16 of each 16-row block, k group lane/16)
  const int fr = lane & 15, fg = lane >> 4;
  const uint16_t* xptr[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = min(m0 + 16 * i + fr, m - 1);     // clamped likewise
    xptr[i] = x + (int64_t)row * n_in + 8 * fg;
  }

  f32x4_t acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // One super-block of this thread's row: header + its 16 bytes of each of the 4 chunks.
  struct WRaw { uint4 hdr, q[4]; };
  auto load_w = [&](WRaw& dst, int b) {
    const uint8_t* p = wptr + 144 * (int64_t)b;
    dst.hdr = load16_a16(p);
#pragma unroll
    for (int c = 0; c < 4; c++) dst.q[c] = load16_a16(p + 16 + 32 * c + 16 * whalf);
  };
  auto load_x = [&](uint4 (&dst)[2][4], int ks) {   // A fragments of one 64-k step: [ksub][row block]
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int i = 0; i < 4; i++) dst[s][i] = *reinterpret_cast<const uint4*>(xptr[i] + ks * 64 + 32 * s);
  };

  // dequantize chunk c (compile-time) of a held super-block into LDS buffer `buf`
  auto dequant_to_lds = [&](const WRaw& r, auto cc, int buf) {
    constexpr int c = decltype(cc)::value;
    const float d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    uint32_t sc1, mn1, sc2, mn2;
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * c, sc1, mn1);
    q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * c + 1, sc2, mn2);
    const float d1 = d * (float)sc1, nm1 = -(dmin * (float)mn1);
    const float d2 = d * (float)sc2, nm2 = -(dmin * (float)mn2);
    const uint32_t qd[4] = {r.q[c].x, r.q[c].y, r.q[c].z, r.q[c].w};
    uint32_t lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t l4 = qd[i] & 0x0F0F0F0Fu, h4 = (qd[i] >> 4) & 0x0F0F0F0Fu;
      float fl[4], fh[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        // fused multiply-add == canonical two-step form here (the product is exact)
        fl[k] = fmaf_(d1, (float)((l4 >> (8 * k)) & 0xFFu), nm1);
        fh[k] = fmaf_(d2, (float)((h4 >> (8 * k)) & 0xFFu), nm2);
      }
      lo[2 * i] = pack_bf16x2(fl[0], fl[1]);
      lo[2 * i + 1] = pack_bf16x2(fl[2], fl[3]);
      hi[2 * i] = pack_bf16x2(fh[0], fh[1]);
      hi[2 * i + 1] = pack_bf16x2(fh[2], fh[3]);
    }
    // low nibbles: k = 16*half + e  -> ksub 0, groups 2*half and 2*half+1; high nibbles: ksub 1
    uint4* base = &sw[buf][0];
    const int u0 = (wj * 4 + 2 * whalf) * 16 + wn;
    base[u0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    base[u0 + 16] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    base[NJ * 64 + u0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    base[NJ * 64 + u0 + 16] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
  };
  // plain step: all MFMAs of a step in one run (B fragments from LDS, A fragments from registers)
  auto mfma_step = [&](const uint4 (&xa)[2][4], int buf) {
#pragma unroll
    for (int s = 0; s < 2; s++) {
      bf16x8_t bfrag[NJ];
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        const uint4 v = sw[buf][(s * NJ + j) * 64 + lane];
        __builtin_memcpy(&bfrag[j], &v, 16);
      }
#pragma unroll
      for (int i = 0; i < 4; i++) {
        bf16x8_t afrag;
        __builtin_memcpy(&afrag, &xa[s][i], 16);
#pragma unroll
        for (int j = 0; j < NJ; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag, bfrag[j], acc[i][j], 0, 0, 0);
      }
    }
  };

  // One 64-k step with the dequantization of the NEXT step's chunk woven into the MFMA stream.
  // Left to itself the compiler emits all MFMAs of a step and then ~130 VALU instructions of
  // dequantization, so the matrix pipe idles while the VALU runs.  Here the dequantization is cut
  // into 33 small pieces (2-4 VALU instructions each) and one piece is placed after (almost)
  // every MFMA; __builtin_amdgcn_sched_barrier(0) pins that order.  An MFMA occupies the matrix
  // pipe for 16 cycles, during which the wavefront issues the piece.
  struct DqState {
    float d, dmin, d1, nm1, d2, nm2;
    uint32_t sc1, mn1, sc2, mn2;
    uint32_t l4, h4;
    float f0, f1, f2, f3;
    uint32_t lo[8], hi[8];
  };
  auto dq_piece = [&](DqState& st, const WRaw& r, auto cc, auto pp, int buf) {
    constexpr int c = decltype(cc)::value;
    constexpr int P = decltype(pp)::value;
    if constexpr (P == 0) {
      st.d = f16_bits_to_f32((uint16_t)(r.hdr.x & 0xFFFF));
      st.dmin = f16_bits_to_f32((uint16_t)(r.hdr.x >> 16));
    } else if constexpr (P == 1) {
      q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * c, st.sc1, st.mn1);
    } else if constexpr (P == 2) {
      q4k_scale_min(r.hdr.y, r.hdr.z, r.hdr.w, 2 * c + 1, st.sc2, st.mn2);
    } else if constexpr (P == 3) {
      st.d1 = st.d * (float)st.sc1;
      st.nm1 = -(st.dmin * (float)st.mn1);
    } else if constexpr (P == 4) {
      st.d2 = st.d * (float)st.sc2;
      st.nm2 = -(st.dmin * (float)st.mn2);
    } else if constexpr (P < 29) {
      constexpr int i = (P - 5) / 6, sub = (P - 5) % 6;
      const uint32_t q = i == 0 ? r.q[c].x : i == 1 ? r.q[c].y : i == 2 ? r.q[c].z : r.q[c].w;
      // fused multiply-add == canonical two-step form here (the product d*sc*q is exact)
      if constexpr (sub == 0) {
        st.l4 = q & 0x0F0F0F0Fu;
        st.h4 = (q >> 4) & 0x0F0F0F0Fu;
      } else if constexpr (sub == 1) {
        st.f0 = fmaf_(st.d1, (float)(st.l4 & 0xFFu), st.nm1);
        st.f1 = fmaf_(st.d1, (float)((st.l4 >> 8) & 0xFFu), st.nm1);
      } else if constexpr (sub == 2) {
        st.f2 = fmaf_(st.d1, (float)((st.l4 >> 16) & 0xFFu), st.nm1);
        st.f3 = fmaf_(st.d1, (float)(st.l4 >> 24), st.nm1);
        st.lo[2 * i] = pack_bf16x2(st.f0, st.f1);
      } else if constexpr (sub == 3) {
        st.lo[2 * i + 1] = pack_bf16x2(st.f2, st.f3);
        st.f0 = fmaf_(st.d2, (float)(st.h4 & 0xFFu), st.nm2);
        st.f1 = fmaf_(st.d2, (float)((st.h4 >> 8) & 0xFFu), st.nm2);
      } else if constexpr (sub == 4) {
        st.f2 = fmaf_(st.d2, (float)((st.h4 >> 16) & 0xFFu), st.nm2);
        st.f3 = fmaf_(st.d2, (float)(st.h4 >> 24), st.nm2);
        st.hi[2 * i] = pack_bf16x2(st.f0, st.f1);
      } else {
        st.hi[2 * i + 1] = pack_bf16x2(st.f2, st.f3);
      }
    } else {
      // low nibbles: k = 16*half + e -> ksub 0, groups 2*half and 2*half+1; high nibbles: ksub 1
      uint4* base = &sw[buf][0];
      const int u0 = (wj * 4 + 2 * whalf) * 16 + wn;
      if constexpr (P == 29) base[u0] = make_uint4(st.lo[0], st.lo[1], st.lo[2], st.lo[3]);
      else if constexpr (P == 30) base[u0 + 16] = make_uint4(st.lo[4], st.lo[5], st.lo[6], st.lo[7]);
      else if constexpr (P == 31) base[NJ * 64 + u0] = make_uint4(st.hi[0], st.hi[1], st.hi[2], st.hi[3]);
      else base[NJ * 64 + u0 + 16] = make_uint4(st.hi[4], st.hi[5], st.hi[6], st.hi[7]);
    }
  };
  constexpr int kPieces = 33;
  constexpr int kMfmas = 8 * NJ;

  // MFMA t = (s*4 + i)*NJ + j of a step, followed by the dequant pieces that fall into its slot
  // The global loads of a step are spread over the slots as well: a wavefront that issues its
  // eight X-fragment loads back to back sits in the issue stage for about a thousand cycles
  // (the vector-memory unit takes ~128 clk per such load), and no MFMA goes out meanwhile.
  auto step_slot = [&](auto tt, const uint4 (&xa)[2][4], uint4 (&xdst)[2][4], int ks_next, WRaw& wdst,
                       int b_next, auto loadw, const bf16x8_t (&bf)[2][NJ], DqState& st, const WRaw& r,
                       auto cc, int buf_next) {
    constexpr int t = decltype(tt)::value;
    constexpr int s = t / (4 * NJ), i = (t / NJ) % 4, j = t % NJ;
    constexpr bool kLoadW = decltype(loadw)::value;
    bf16x8_t afrag;
    __builtin_memcpy(&afrag, &xa[s][i], 16);
    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag, bf[s][j], acc[i][j], 0, 0, 0);
    if constexpr (t == 1) TTQ_GEMM_TRACE(4 * ks_next + 1);
    if constexpr (t == 4 * NJ + 1) TTQ_GEMM_TRACE(4 * ks_next + 3);
    if constexpr (j == 0)
      xdst[s][i] = *reinterpret_cast<const uint4*>(xptr[i] + ks_next * 64 + 32 * s);
    if constexpr (kLoadW && j == 3 && (t / NJ) < 5) {
      constexpr int piece = t / NJ;   // 0: header, 1..4: the thread's 16 bytes of chunk piece-1
      const uint8_t* p = wptr + 144 * (int64_t)b_next;
      if constexpr (piece == 0) wdst.hdr = load16_a16(p);
      else wdst.q[piece - 1] = load16_a16(p + 16 + 32 * (piece - 1) + 16 * whalf);
    }
    constexpr int p0 = t * kPieces / kMfmas, p1 = (t + 1) * kPieces / kMfmas;
    if constexpr (p1 > p0) dq_piece(st, r, cc, std::integral_constant<int, p0>{}, buf_next);
    if constexpr (p1 > p0 + 1) dq_piece(st, r, cc, std::integral_constant<int, p0 + 1>{}, buf_next);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto run_slots = [&](auto self, auto tt, const uint4 (&xa)[2][4], uint4 (&xdst)[2][4], int ks_next,
                       WRaw& wdst, int b_next, auto loadw, const bf16x8_t (&bf)[2][NJ], DqState& st,
                       const WRaw& r, auto cc, int buf_next) -> void {
    constexpr int t = decltype(tt)::value;
    if constexpr (t < kMfmas) {
      step_slot(tt, xa, xdst, ks_next, wdst, b_next, loadw, bf, st, r, cc, buf_next);
      self(self, std::integral_constant<int, t + 1>{}, xa, xdst, ks_next, wdst, b_next, loadw, bf, st, r, cc,
           buf_next);
    }
  };
  // step: B fragments of both k halves are read from LDS buffer `buf` up front, then the slots
  auto step = [&](const uint4 (&xa)[2][4], uint4 (&xdst)[2][4], int ks_next, WRaw& wdst, int b_next,
                  auto loadw, int buf, const WRaw& r, auto cc) {
    bf16x8_t bf[2][NJ];
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        const uint4 v = sw[buf][(s * NJ + j) * 64 + lane];
        __builtin_memcpy(&bf[s][j], &v, 16);
      }
    DqState st;
    __builtin_amdgcn_sched_barrier(0);
    TTQ_GEMM_TRACE(4 * ks_next + 0);
    run_slots(run_slots, std::integral_constant<int, 0>{}, xa, xdst, ks_next, wdst, b_next, loadw, bf, st, r,
              cc, buf ^ 1);
    TTQ_GEMM_TRACE(4 * ks_next + 2);
  };

  // Software pipeline, one super-block (4 steps of 64 k) per outer iteration.  X fragments
  // travel through a ring of four step buffers, requested three steps ahead (a global load
  // takes longer than one step of MFMAs); the raw super-block b+1 is requested at the first
  // step of block b; the dequantized chunk of step ks+1 is written to the other LDS buffer
  // while the MFMAs of step ks run.
  const int nblocks = n_in >> 8;
  const int ksteps = n_in >> 6;
  WRaw wcur, wnext;
  uint4 xr[4][2][4];
  load_w(wcur, 0);
  load_x(xr[0], 0);
  load_x(xr[1], min(1, ksteps - 1));
  load_x(xr[2], min(2, ksteps - 1));
  dequant_to_lds(wcur, std::integral_constant<int, 0>{}, 0);
  wnext = wcur;
  __syncthreads();

  for (int b = 0; b < nblocks; b++) {
    const int ks = 4 * b;
    // loads past the end are clamped to the last block / step: harmless re-reads that keep the
    // step bodies straight-line (the chunk dequantized from them in the last step is never read)
    const int bn = min(b + 1, nblocks - 1);
    using T = std::true_type;
    using Fz = std::false_type;
    if constexpr (WEAVE) {
      step(xr[0], xr[3], min(ks + 3, ksteps - 1), wnext, bn, T{}, 0, wcur, std::integral_constant<int, 1>{});
      __syncthreads();
      step(xr[1], xr[0], min(ks + 4, ksteps - 1), wnext, bn, Fz{}, 1, wcur, std::integral_constant<int, 2>{});
      __syncthreads();
      step(xr[2], xr[1], min(ks + 5, ksteps - 1), wnext, bn, Fz{}, 0, wcur, std::integral_constant<int, 3>{});
      __syncthreads();
      step(xr[3], xr[2], min(ks + 6, ksteps - 1), wnext, bn, Fz{}, 1, wnext, std::integral_constant<int, 0>{});
      __syncthreads();
    } else {
      load_w(wnext, bn);
      load_x(xr[3], min(ks + 3, ksteps - 1));
      mfma_step(xr[0], 0); dequant_to_lds(wcur, std::integral_constant<int, 1>{}, 1);
      __syncthreads();
      load_x(xr[0], min(ks + 4, ksteps - 1));
      mfma_step(xr[1], 1); dequant_to_lds(wcur, std::integral_constant<int, 2>{}, 0);
      __syncthreads();
      load_x(xr[1], min(ks + 5, ksteps - 1));
      mfma_step(xr[2], 0); dequant_to_lds(wcur, std::integral_constant<int, 3>{}, 1);
      __syncthreads();
      load_x(xr[2], min(ks + 6, ksteps - 1));
      mfma_step(xr[3], 1); dequant_to_lds(wnext, std::integral_constant<int, 0>{}, 0);
      __syncthreads();
    }
    wcur = wnext;
  }

  // ---- epilogue: lane holds Y[m0 + 16i + 4*(lane/16) + r][n0 + 16j + lane%16], r = 0..3
  const int cn = lane & 15, rb4 = (lane >> 4) * 4;
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int n = n0 + 16 * j + cn;
    if (n >= n_out) continue;
    const float bv = load_bias(bias, bias_dtype, n);
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int mm = m0 + 16 * i + rb4 + r;
        if (mm < m) YElem<YT>::store(y, (int64_t)mm * n_out + n, acc[i][j][r] + bv);
      }
    }
  }
}

static int env_flag(const char* name, int dflt) { return dev_knob(name, dflt); }

template <int NJ, typename YT>
static hipError_t launch_nj_y(const uint8_t* wb, const uint16_t* x, YT* y, const void* bias, int bias_dtype,
                              int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  constexpr int BN = NJ * 16;
  static const int weave = env_flag("TTQ_GEMM_WEAVE", 1);
  static const int xcd_map = env_flag("TTQ_GEMM_XCD_MAP", 1);
  const int n_tiles = (int)((n_out + BN - 1) / BN), m_tiles = (int)((m + kGemmBM - 1) / kGemmBM);
  int xcds_per_mtile = 0;
  unsigned nwg = (unsigned)(n_tiles * m_tiles);
  if (xcd_map && m_tiles >= 2 && m_tiles <= 8 && 8 % m_tiles == 0) {
    xcds_per_mtile = 8 / m_tiles;
    nwg = (unsigned)(((n_tiles + xcds_per_mtile - 1) / xcds_per_mtile) * 8);
  }
  const dim3 grid(nwg), block(kGemmThreads);
  if (weave)
    hipLaunchKernelGGL((gemm_q4k_kernel<NJ, YT, true>), grid, block, 0, s, wb, x, y, bias, bias_dtype, (int)m,
                       (int)n_out, (int)n_in, n_tiles, m_tiles, xcds_per_mtile);
  else
    hipLaunchKernelGGL((gemm_q4k_kernel<NJ, YT, false>), grid, block, 0, s, wb, x, y, bias, bias_dtype, (int)m,
                       (int)n_out, (int)n_in, n_tiles, m_tiles, xcds_per_mtile);
  return hipGetLastError();
}

template <int NJ>
static hipError_t launch_nj(const uint8_t* wb, const uint16_t* x, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (y_dtype == kBF16)
    return launch_nj_y<NJ, bf16_tag>(wb, x, static_cast<bf16_tag*>(y), bias, bias_dtype, m, n_out, n_in, s);
  if (y_dtype == kF32)
    return launch_nj_y<NJ, float>(wb, x, static_cast<float*>(y), bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

// The few-row kernel (ttq_gemm_skinny.hip: up to 64 rows, weights dequantized in registers, no tile
// of W in LDS) where it exists for the shape and is estimated to be faster than the tiled kernel.
static bool prefer_skinny(int format, int64_t m, int64_t n_out, int64_t n_in) {
  return gemm_skinny_supported(format, m, n_out, n_in) &&
         (!gemm_pc_supported(format, m, n_out, n_in, 112) ||
          gemm_skinny_estimate_us(format, m, n_out, n_in) < gemm_pc_estimate_us(format, m, n_out, n_in));
}

// 65 .. 256 rows on a matrix with few columns (attention output, down projection: 4096 columns are 37 tiles of
// 112 for 256 compute units) leave the tiled kernel one short round whose length is the latency of its K loop.
// It then splits K over copies of the grid (ttq_gemm_pc.hip); where the rows are too short for that, two or
// three launches of the few-row kernel, 64 rows each, can still be faster.  The margin covers the tiled
// kernel's estimate, which is fitted to full rounds and is about a third too high for a single short one.
static float skinny_chunks_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in) {
  const int64_t full = m / 64, rest = m % 64;
  float us = (float)full * gemm_skinny_estimate_us(format, 64, n_out, n_in);
  if (rest) us += gemm_skinny_estimate_us(format, rest, n_out, n_in);
  return us;
}
static bool prefer_skinny_chunks(int format, int64_t m, int64_t n_out, int64_t n_in) {
  if (m <= 64 || m > 256 || !gemm_skinny_supported(format, 64, n_out, n_in)) return false;
  if (!gemm_pc_supported(format, m, n_out, n_in, 112)) return false;
  return skinny_chunks_estimate_us(format, m, n_out, n_in) < 0.65f * gemm_pc_estimate_us(format, m, n_out, n_in);
}

bool gemm_supported(int format, int64_t m, int64_t n_out, int64_t n_in) {
  // Q4_K also has the single-role tiled kernel of this file, which takes any size
  return format == kQ4_K || gemm_skinny_supported(format, m, n_out, n_in) ||
         gemm_pc_supported(format, m, n_out, n_in, 112);
}

float gemm_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in) {
  float us = gemm_pc_estimate_us(format, m, n_out, n_in);
  if (gemm_skinny_supported(format, m, n_out, n_in)) us = fminf(us, gemm_skinny_estimate_us(format, m, n_out, n_in));
  return us;
}

hipError_t launch_gemm(int format, const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                       int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (prefer_skinny(format, m, n_out, n_in))
    TTQ_ROUTE(kRouteGemmSkinny, launch_gemm_skinny(format, w, x_bf16, kBF16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (prefer_skinny_chunks(format, m, n_out, n_in))
    TTQ_ROUTE(kRouteGemmSkinnyChunked,
              launch_gemm_skinny_chunked(format, w, x_bf16, kBF16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s));
  if (format != kQ4_K) {
    if (!gemm_pc_supported(format, m, n_out, n_in, 112)) return hipErrorInvalidValue;
    return launch_gemm_pc(format, w, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  }
  // The producer/consumer kernel (ttq_gemm_pc.hip, 112- and 64-column tiles) wherever it takes the shape: it is
  // faster than this file's single-role kernel also where 128-column tiles would save a round of workgroups
  // (28672 x 4096 at 2048 rows: 547 us here, 420 us there).
  if (gemm_pc_supported(kQ4_K, m, n_out, n_in, 112))
    return launch_gemm_pc(kQ4_K, w, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  // What is left (activations beyond 4 GiB): the tile width that needs the least time, rounds of tiles over the
  // CUs times tile width.
  const int64_t cus = device_num_cus();
  const int64_t mt = (m + kGemmBM - 1) / kGemmBM;
  auto cost = [&](int64_t bn) { return ((((n_out + bn - 1) / bn) * mt + cus - 1) / cus) * bn; };
  static const int forced = dev_knob("TTQ_GEMM_BN", 0);
  const bool use112 = forced ? forced == 112 : cost(112) < cost(128);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  TTQ_ROUTE(kRouteGemmQ4kTiles, (use112 ? launch_nj<7>(wb, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s)
                                        : launch_nj<8>(wb, x_bf16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s)));
}

}  // namespace ttq
