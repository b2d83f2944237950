// Prefill GEMM for Q4_K, Q6_K and Q8_0 weights on gfx950, producer/consumer form with the activations read
// straight from global memory into the consumers' registers: Y (m, n_out) = X (m, n_in) * W^T.
//
// Replaces F.linear(x, weight) for a multi-row bf16 activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81; the prefill case of
//  workspace/transformers/src/layers/attn.nim:154-156).
//
// A workgroup of eight wavefronts (two per SIMD) owns a (64 * MB) x BN tile of Y:
//   consumers (wavefronts 0-3, 16 * MB rows of the tile each): v_mfma_f32_16x16x32_bf16, B fragments from the W
//       tile in LDS, A fragments by buffer loads, three steps' worth of registers rotating by name: the fragments
//       of step s+2 are requested during step s.
//   producers (wavefronts 4-7): pc_produce_w of ttq_gemm_pc.h -- packed blocks, canonical dequantization, bf16
//       nearest-even, B fragments into the double-buffered W tile.
// One barrier per 64-k step.
//
// The activations come from a copy of X in fragment order (pack_activations below, one pass over X per call):
//     Xp[step ks][row block rb][half h][lane l] = 16 bytes: row 16 rb + l % 16, k = 64 ks + 32 h + 8 (l / 16) .. + 7
// so that an A fragment is one load instruction over 1 KB of consecutive bytes.  Read from the row-major X itself
// the same fragment is 16 bytes from each of 16 rows per quarter wavefront, the vector memory path then handles a
// lane at a time, and the consumers wait for their requests longer than they multiply (measured: 65 us against 43
// for the consumers alone at M = 512).
//
// Why X bypasses LDS: every byte written to LDS goes through one port of about 85 bytes per cycle and compute unit,
// whoever writes (ds_write or global_load_lds), and LDS reads queue behind waiting ds_writes.  With X staged through
// LDS a step writes 32 KB of X and 14 KB of W and reads 88 KB of fragments; here it writes 14 KB and reads 56 KB.
//
// ABL (a bit mask, 0 in the product) switches stages off for the measurement ladder of ttq_ladder_gemm.hip:
// 1 the consumers' MFMAs and B reads, 2 their A requests, 4 / 8 / 16 the producers' LDS stores / arithmetic / global
// loads, 512 cycle counts around the barriers, 1024 no barriers, 4096 real values in the W tile at the start.
#pragma once

#include "ttq_gemm_pc.h"

namespace ttq {

constexpr int pcd_threads(int nc) { return (nc + 4) * 64; }   // NC consumers, 4 W producers

// 16-byte buffer load the compiler neither moves nor waits for: left to itself it sinks the requests of the next
// steps down to their first use (to save registers) and then waits for each of them in turn.  The caller counts
// outstanding requests itself (wait_vmcnt) before it touches the result.
template <int IMM>
__device__ __forceinline__ void buffer_load16_async(u32x4_t& dst, u32x4_t rsrc, int voffset, int soffset) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4"
               : "=v"(dst) : "v"(voffset), "s"(rsrc), "s"(soffset), "n"(IMM) : "memory");
}

// XT: the 16-bit type of the packed activations, and the type the producers round the weights to (bf16, or fp16
// for fp16 activations: the operator then computes in the activations' own type, with weights that keep 11 bits).
template <int NJ, int FMT, int MB, bool FUSE, int ABL = 0, int NC = 4, class XT = bf16_tag>
__global__ void __launch_bounds__(pcd_threads(NC))
gemm_pcd_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ xp, void* __restrict__ yv,
                int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                int n_tiles, int m_tiles, int xcds_per_mtile, PcSplit sp, const float* __restrict__ row_scale) {
  constexpr int BN = NJ * 16;
  constexpr int kWUnits = 2 * NJ * 64;
  constexpr int kPcBM = NC * 16 * MB;
  constexpr int kPcdThreads = pcd_threads(NC);
  constexpr int kStgBytes = 16 * MB * (BN * 2 + 16);      // a consumer's epilogue staging area
  __shared__ uint4 sw[2 * kWUnits];
  __shared__ __attribute__((aligned(16))) uint8_t stg[NC * kStgBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  [[maybe_unused]] uint32_t t_bar = 0;
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
        t[2] = 0;
        t[3] = (uint32_t)(__builtin_amdgcn_s_memrealtime() - rt_begin);     // 100 MHz ticks
      }
    }
  };
  // Tile assignment: as in gemm_pc_kernel (one X slab per XCD L2 when the row tiles divide the XCDs evenly; copies
  // of the tile grid when the launch is split along K).
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
    const uint4* src = reinterpret_cast<const uint4*>(xp);
    const int lim = min(m, 256) * n_in / 8;
    for (int i = tid; i < 2 * kWUnits; i += kPcdThreads) sw[i] = src[(i * 5 + (int)blockIdx.x * 32 + 4096) % lim];
    __syncthreads();
  }

  // One barrier per 64-k step, numbered s = -1 .. ksteps-1.  Barrier s means: the W fragments of step s+1 are
  // complete in LDS (buffer (s+1) % 2) and every LDS read of step s has finished.  The consumers pass it near the
  // end of step s, the producers after preparing step s+1.
  if (wave >= NC) {
    pc_produce_w<NJ, FMT, FUSE, ABL, XT>(w, tid - NC * 64, n0, n_out, row_blocks, block0, nblocks,
                                     (uint32_t)(size_t)(lptr_t)(&sw[0]), bar);
    trace_out();
    return;
  }

  // -------------------------------------------------------------------- consumer
  const int m0 = m_tile * kPcBM + wave * (16 * MB);
  // A fragment (row block ib of this consumer, half h of step ks): 1 KB at ((ks * RB + rb0 + ib) * 2 + h) * 1024 of
  // the packed copy, RB = row blocks of the whole activation.  Buffer loads take the per-lane offset (loop-invariant),
  // the uniform offset of the step and the half as an immediate: no address arithmetic per request.  Row blocks past
  // the end are clamped (never stored to Y).
  const int row_blocks_x = (m + 15) >> 4;
  const uint64_t xaddr = (uint64_t)(size_t)xp;
  // raw buffer descriptor: base, stride 0, bytes (< 4 GiB: the launcher checks), 32-bit untyped data
  u32x4_t xrsrc = {(uint32_t)xaddr, (uint32_t)(xaddr >> 32) & 0xFFFFu, (uint32_t)row_blocks_x * (uint32_t)(n_in * 32),
                   0x00020000u};
#pragma unroll
  for (int q = 0; q < 4; q++) xrsrc[q] = (uint32_t)__builtin_amdgcn_readfirstlane((int)xrsrc[q]);
  int aoff[MB];
#pragma unroll
  for (int ib = 0; ib < MB; ib++) aoff[ib] = min((m0 >> 4) + ib, row_blocks_x - 1) * 2048 + lane * 16;
  struct ASet { u32x4_t v[2][MB]; };
  auto request_one = [&](ASet& dst, int koff, int h, int ib) {   // koff: byte offset of the step in the packed copy
    if constexpr ((ABL & 2) != 0) return;
    if (h == 0) buffer_load16_async<0>(dst.v[0][ib], xrsrc, aoff[ib], koff);
    else buffer_load16_async<1024>(dst.v[1][ib], xrsrc, aoff[ib], koff);
  };
  // (past the last step: a harmless re-read)
  auto step_koff = [&](int ks) { return (4 * block0 + min(ks, ksteps - 1)) * (row_blocks_x * 2048); };
  // A step is 2*NJ groups of MB MFMAs: group g uses the A fragments of half g/NJ and the B fragment of column block
  // g%NJ.  B fragments are read two groups ahead into a ring of four, the A fragments of step ks+2 are requested one
  // per group at the start of step ks, and __builtin_amdgcn_sched_barrier pins that order.
  constexpr int G = 2 * NJ;
  static_assert(2 * MB <= G, "one A request per group");
  bf16x8_t bring[4];
  auto read_b = [&](bf16x8_t& dst, int buf, int g) {   // g = half * NJ + j
    const uint4 v = sw[buf * kWUnits + g * 64 + lane];
    __builtin_memcpy(&dst, &v, 16);
  };

  f32x4_t acc[MB][NJ];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // one step: `cur` holds its A fragments, `into` receives those of step ks+2; BUF is its W buffer and fixes the
  // ring slot of its first group (2*NJ is 2 mod 4 for the tiles built here, or 0).
  auto step = [&](const ASet& cur, ASet& into, auto bufc, int ks) {
    constexpr int BUF = decltype(bufc)::value;
    constexpr int SO = (BUF * G) & 3;
    if constexpr ((ABL & 1) != 0) { bar(); return; }
    // Requests complete in order: all but the youngest 2 * MB (those of step ks+1) have landed, `cur` among them.
    wait_vmcnt<2 * MB>();
    const int koff2 = step_koff(ks + 2);
#pragma unroll
    for (int g = 0; g < G; g++) {
      if (g == G - 2) bar();     // barrier ks: step ks+1 is in LDS, reads of step ks done
      if (g + 2 < G) read_b(bring[(g + 2 + SO) & 3], BUF, g + 2);
      else read_b(bring[(g + 2 + SO) & 3], BUF ^ 1, g + 2 - G);
      // request r of the step (row block r / 2, half r % 2) goes out with group r * G / (2 * MB)
#pragma unroll
      for (int r = 0; r < 2 * MB; r++)
        if (r * G / (2 * MB) == g) request_one(into, koff2, r % 2, r / 2);
      __builtin_amdgcn_sched_barrier(0);
      const int half = g / NJ, j = g % NJ;
#pragma unroll
      for (int i = 0; i < MB; i++) {
        if constexpr (__is_same(XT, f16_tag)) {
          f16x8_t a, b;
          __builtin_memcpy(&a, &cur.v[half][i], 16);
          __builtin_memcpy(&b, &bring[(g + SO) & 3], 16);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[i][j], 0, 0, 0);
        } else {
          bf16x8_t a;
          __builtin_memcpy(&a, &cur.v[half][i], 16);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bring[(g + SO) & 3], acc[i][j], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  ASet a0{}, a1{}, a2{};
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_one(a0, step_koff(0), h, ib);
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_one(a1, step_koff(1), h, ib);
  bar();                         // barrier -1: the W fragments of step 0 are in LDS
  read_b(bring[0], 0, 0);
  read_b(bring[1], 0, 1);
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  static_assert(((2 * G) & 3) == 0, "two steps bring the B ring back to slot 0");
  // (ksteps is a multiple of four; the register sets rotate with period three, the W buffers with period two)
  for (int ks = 0; ks < ksteps; ks += 6) {
    step(a0, a2, C0{}, ks);
    step(a1, a0, C1{}, ks + 1);
    if (ks + 2 >= ksteps) break;
    step(a2, a1, C0{}, ks + 2);
    step(a0, a2, C1{}, ks + 3);
    if (ks + 4 >= ksteps) break;
    step(a1, a0, C0{}, ks + 4);
    step(a2, a1, C1{}, ks + 5);
  }
  wait_vmcnt<0>();               // the re-reads past the last step
  trace_out();

  PcEpi epi{sp, ksplit, m_tile, n_tile, n_tiles, wave, lane, stg + wave * kStgBytes, yv, y_dtype, bias, bias_dtype, m, n_out,
            n0, m0};
  // (constants in the bf16 kernels, whose epilogue stays what it was)
  if constexpr (__is_same(XT, f16_tag)) {
    epi.row_scale = row_scale;
    epi.f16_rows = true;
  }
  pc_epilogue<NJ, MB, FUSE, NC>(acc, epi);
}

// X (m, n_in) in any activation type -> its copy in fragment order as DT (bf16, or fp16 for the fp16 GEMM; rows past
// m as zeros).  A workgroup moves 16 rows x 256 k: whole 128-byte lines in, whole kilobytes out.
template <typename XT, typename DT = bf16_tag>
__global__ void __launch_bounds__(256) pack_activations_kernel(const XT* __restrict__ x, uint16_t* __restrict__ xp, int m,
                                                               int n_in, int row_blocks) {
  const int t = threadIdx.x;
  const int rb = blockIdx.y, ks = blockIdx.x * 4 + (t >> 6);        // a wavefront per 64-k step
  const int l = t & 63, r = l >> 2, c2 = l & 3;                     // lane: row r, chunks 2 c2 and 2 c2 + 1 of the step
  const int row = rb * 16 + r;
  if (ks * 64 >= n_in) return;
  uint4 v[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if constexpr (std::is_same<XT, DT>::value) {
    if (row < m) {
      const uint4* src = reinterpret_cast<const uint4*>(x + (int64_t)row * n_in + ks * 64 + c2 * 16);
      v[0] = src[0];
      v[1] = src[1];
    }
  } else if (row < m) {
    const XT* src = x + (int64_t)row * n_in + ks * 64 + c2 * 16;
    float f[16];
#pragma unroll
    for (int i = 0; i < 16; i++) f[i] = XElem<XT>::load(src, i);
    v[0] = make_uint4(pack_x2<DT>(f[0], f[1]), pack_x2<DT>(f[2], f[3]), pack_x2<DT>(f[4], f[5]), pack_x2<DT>(f[6], f[7]));
    v[1] = make_uint4(pack_x2<DT>(f[8], f[9]), pack_x2<DT>(f[10], f[11]), pack_x2<DT>(f[12], f[13]), pack_x2<DT>(f[14], f[15]));
  }
  uint8_t* dst = reinterpret_cast<uint8_t*>(xp) + ((int64_t)ks * row_blocks + rb) * 2048;
#pragma unroll
  for (int q = 0; q < 2; q++) {
    const int chunk = 2 * c2 + q;                                   // 8 k of the row: half chunk / 4, k-group chunk % 4
    *reinterpret_cast<uint4*>(dst + (chunk >> 2) * 1024 + ((chunk & 3) * 16 + r) * 16) = v[q];
  }
}

// fp32 X (m, n_in) -> fp16 in fragment order with a power-of-two factor per row: the row's largest magnitude lands in
// [2^14, 2^15), so that any finite row fits fp16 and keeps its 11 bits whatever its size; inv[row] = 1 / factor for the
// GEMM's epilogue.  A row with a non-finite value, or of zeros, is not scaled (factor 1): its non-finite values
// convert as they are and poison that row's outputs only.  Two launches: a workgroup per row finds the factor, then
// the packing pass of pack_activations_kernel multiplies by it.
static __global__ void __launch_bounds__(256) row_scale_factors_kernel(const float* __restrict__ x, float* __restrict__ inv,
                                                                       int n_in) {
  __shared__ float part[9];
  const float fi = block_row_inverse_factor(x + (int64_t)blockIdx.x * n_in, n_in, part);
  if (threadIdx.x == 0) inv[blockIdx.x] = fi;
}

static __global__ void __launch_bounds__(256) pack_activations_scaled_kernel(const float* __restrict__ x, uint16_t* __restrict__ xp,
                                                                             const float* __restrict__ inv, int m, int n_in,
                                                                             int row_blocks) {
  const int t = threadIdx.x;
  const int rb = blockIdx.y, ks = blockIdx.x * 4 + (t >> 6);        // a wavefront per 64-k step
  const int l = t & 63, r = l >> 2, c2 = l & 3;                     // lane: row r, chunks 2 c2 and 2 c2 + 1 of the step
  const int row = rb * 16 + r;
  if (ks * 64 >= n_in) return;
  uint4 v[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  if (row < m) {
    const float f = row_factor_of_inverse(inv[row]);
    const float4* src = reinterpret_cast<const float4*>(x + (int64_t)row * n_in + ks * 64 + c2 * 16);
    const float4 a = src[0], b = src[1], c = src[2], d = src[3];
    v[0] = make_uint4(pack_f16x2(a.x * f, a.y * f), pack_f16x2(a.z * f, a.w * f), pack_f16x2(b.x * f, b.y * f),
                      pack_f16x2(b.z * f, b.w * f));
    v[1] = make_uint4(pack_f16x2(c.x * f, c.y * f), pack_f16x2(c.z * f, c.w * f), pack_f16x2(d.x * f, d.y * f),
                      pack_f16x2(d.z * f, d.w * f));
  }
  uint8_t* dst = reinterpret_cast<uint8_t*>(xp) + ((int64_t)ks * row_blocks + rb) * 2048;
#pragma unroll
  for (int q = 0; q < 2; q++) {
    const int chunk = 2 * c2 + q;                                   // 8 k of the row: half chunk / 4, k-group chunk % 4
    *reinterpret_cast<uint4*>(dst + (chunk >> 2) * 1024 + ((chunk & 3) * 16 + r) * 16) = v[q];
  }
}

inline hipError_t launch_pack_activations_scaled(const float* x, uint16_t* xp, float* inv, int64_t m, int64_t n_in,
                                                 hipStream_t s) {
  const int row_blocks = (int)((m + 15) / 16);
  hipLaunchKernelGGL(row_scale_factors_kernel, dim3((unsigned)m), dim3(256), 0, s, x, inv, (int)n_in);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 grid((unsigned)((n_in / 64 + 3) / 4), (unsigned)row_blocks), block(256);
  hipLaunchKernelGGL(pack_activations_scaled_kernel, grid, block, 0, s, x, xp, inv, (int)m, (int)n_in, row_blocks);
  return hipGetLastError();
}

inline size_t packed_activation_bytes(int64_t m, int64_t n_in) { return (size_t)((m + 15) / 16) * 16 * (size_t)n_in * 2; }

// keep_f16: fp16 activations stay fp16 (for the fp16 GEMM); everything else becomes bf16
inline hipError_t launch_pack_activations(const void* x, int x_dtype, uint16_t* xp, int64_t m, int64_t n_in, hipStream_t s,
                                          bool keep_f16 = false) {
  const int row_blocks = (int)((m + 15) / 16);
  const dim3 grid((unsigned)((n_in / 64 + 3) / 4), (unsigned)row_blocks), block(256);
  if (keep_f16) {
    if (x_dtype != kF16) return hipErrorInvalidValue;
    hipLaunchKernelGGL((pack_activations_kernel<f16_tag, f16_tag>), grid, block, 0, s, static_cast<const f16_tag*>(x), xp,
                       (int)m, (int)n_in, row_blocks);
    return hipGetLastError();
  }
  switch (x_dtype) {
    case kBF16:
      hipLaunchKernelGGL(pack_activations_kernel<bf16_tag>, grid, block, 0, s, static_cast<const bf16_tag*>(x), xp, (int)m,
                         (int)n_in, row_blocks);
      break;
    case kF16:
      hipLaunchKernelGGL(pack_activations_kernel<f16_tag>, grid, block, 0, s, static_cast<const f16_tag*>(x), xp, (int)m,
                         (int)n_in, row_blocks);
      break;
    case kF32:
      hipLaunchKernelGGL(pack_activations_kernel<float>, grid, block, 0, s, static_cast<const float*>(x), xp, (int)m,
                         (int)n_in, row_blocks);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// xp: the packed copy of the activations.  The caller owns the split-K workspace: sp.splits == 1 (no partials, no
// counters) or a prepared PcSplit whose tile_wgs this function fills in.
template <int FMT, int MB, int NJ, bool FUSE, int ABL = 0, int NC = 4, class XT = bf16_tag>
static hipError_t launch_pcd_grid(const uint8_t* wb, const uint16_t* x, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp, hipStream_t s,
                                  const float* row_scale = nullptr) {
  constexpr int BO = FUSE ? NJ * 8 : NJ * 16, BM = NC * 16 * MB;
  const int n_tiles = (int)((n_out + BO - 1) / BO), m_tiles = (int)((m + BM - 1) / BM);
  int xcds_per_mtile = 0;
  unsigned nwg = (unsigned)(n_tiles * m_tiles);
  if (m_tiles >= 2 && m_tiles <= 8 && 8 % m_tiles == 0) {
    xcds_per_mtile = 8 / m_tiles;
    nwg = (unsigned)(((n_tiles + xcds_per_mtile - 1) / xcds_per_mtile) * 8);
  }
  sp.tile_wgs = (int)nwg;
  hipLaunchKernelGGL((gemm_pcd_kernel<NJ, FMT, MB, FUSE, ABL, NC, XT>), dim3(nwg * (unsigned)sp.splits), dim3(pcd_threads(NC)), 0, s,
                     wb, x, y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles, xcds_per_mtile, sp,
                     row_scale);
  return hipGetLastError();
}

}  // namespace ttq
