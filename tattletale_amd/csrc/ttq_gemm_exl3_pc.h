// Trellis-coded (EXL3-style) linear layer for many activation rows as a producer/consumer GEMM on gfx950:
//   Y = svh o H( T * Xr^T ),  Xr = H(suh o X) / sqrt(128) rounded to fp16 (made by a pass of its own),
// the prefill side of Linear.forward (workspace/transformers/src/layers/linear.nim:45-57; the projections see seq_len
// rows at prefill, workspace/transformers/src/layers/attn.nim:154-156).
//
// The workgroup is that of ttq_gemm_pcd.h -- four consumers (v_mfma_f32_16x16x32_f16, B fragments from LDS, A
// fragments by buffer loads from a copy of Xr in fragment order) and W producers, one barrier per 64-k step --
// with 128 columns to a tile, which is one Hadamard group of output channels:
//   producers: eight wavefronts (a wavefront issues a vector instruction every four to five clocks whatever else
//       runs on its SIMD, and the decode is a chain of them: two producers per SIMD beside the consumer keep up with
//       the matrix cores, one does not).  Wavefront p decodes k-tile 4 s + p % 4 of step s for four of the tile's
//       eight column blocks.  The 4 x 32 x bits bytes of those tiles are consecutive in trellis[k_tile][n_tile]; they
//       come by LDS DMA into a ring of eight steps private to the wavefront (3 us ahead of their use, no registers
//       held), a lane reads the two dwords that hold its four windows, swaps their halves (MSB-first 16-bit words -> a
//       big-endian bit string), decodes four weights as in the decode GEMV (XmLane) and stores them as half of a B
//       fragment unit.  A decoded tile thus serves every row of the tile (64 * MB) instead of 64.  (Tiles of 256 rows:
//       four producers with eight column blocks each, see xg_producers.)
//   epilogue: after the copies of a launch split along K have met, a consumer rotates the 128 sums of each of its
//       rows in registers (butterflies over the column blocks in place, over the columns of a block by DPP moves),
//       applies svh and the bias and stores.
#pragma once

#include "ttq_exl3_common.h"
#include "ttq_gemm_pcd.h"

namespace ttq {

// Two shapes of workgroup.  Tiles of 64 or 128 rows (MB = 1, 2): eight producers and four consumers, 168 registers
// each.  Tiles of 256 rows (MB = 4; for launches whose 256-row tiles alone fill the compute units): the consumers
// need 256 registers, which leaves room for four producers only, two k-tiles' worth of column blocks each -- the
// decode is slower per step, but it is paid once per 256 rows.
constexpr int xg_producers(int mb) { return mb == 4 ? 4 : 8; }
constexpr int xg_threads(int mb) { return (4 + xg_producers(mb)) * 64; }
// steps the producers' requests run ahead (a ring slot per step): about 3 us either way
constexpr int xg_ahead(int mb) { return mb == 4 ? 4 : 8; }

// what a producer wavefront handles per step, and the LDS its ring takes
template <int BITS, int MB>
struct XgGeom {
  static constexpr int kTiles = 32 / xg_producers(MB);               // tiles (column blocks of one k-tile) per step
  static constexpr int kRunBytes = kTiles * 32 * BITS;               // consecutive in trellis[k_tile][n_tile]
  static constexpr int kReq = (kRunBytes + 1023) / 1024;             // requests of 64 x 16 bytes
  static constexpr int kSlotBytes = kReq * 1024;
  static constexpr int kRingBytes = xg_ahead(MB) * kSlotBytes;
};

template <int BITS, int CB, int MB>
__global__ void __launch_bounds__(xg_threads(MB))
gemm_exl3_pc_kernel(const uint8_t* __restrict__ trellis, const uint16_t* __restrict__ svh, const uint16_t* __restrict__ xp,
                    void* __restrict__ yv, int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out,
                    int n_in, int n_tiles, int m_tiles, int xcds_per_mtile, PcSplit sp) {
  constexpr int NJ = 8, NC = 4;
  constexpr int BN = NJ * 16;
  constexpr int kWUnits = 2 * NJ * 64;
  constexpr int kPcBM = NC * 16 * MB;
  constexpr int kStgBytes = 16 * MB * (BN * 2 + 16);      // a consumer's epilogue staging area
  using RG = XgGeom<BITS, MB>;
  constexpr int kXgProducers = xg_producers(MB), kXgTiles = RG::kTiles, kXgAhead = xg_ahead(MB);
  static_assert(kXgTiles == 4 || kXgTiles == 8, "tiles in groups of four");
  __shared__ uint4 sw[2 * kWUnits];
  __shared__ __attribute__((aligned(16))) uint8_t stg[NC * kStgBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t raw[kXgProducers * RG::kRingBytes];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  auto bar = [&]() { lds_barrier(); };

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
  const int n0 = n_tile * BN;
  const int all_steps = n_in >> 6;
  const int ksteps = sp.splits > 1 ? all_steps / sp.splits : all_steps;     // a multiple of four
  const int step0 = ksplit * ksteps;

  // One barrier per 64-k step, numbered s = -1 .. ksteps-1.  Barrier s means: the W fragments of step s+1 are
  // complete in LDS (buffer (s+1) % 2) and every LDS read of step s has finished.
  if (wave >= NC) {
    // ------------------------------------------------------------------ W producer
    const int pw = wave - NC;
    const int ktl = pw & 3, nt0 = (pw >> 2) * kXgTiles;               // k-tile of the step, first column block
    const int j = lane & 15, q = lane >> 4;
    XmLane<BITS> ln;
    ln.init(lane);
    constexpr int kWin = XmLane<BITS>::kWin;
    constexpr int kTileDw = 8 * BITS;
    // byte offsets, inside a tile, of the two dwords of each window (the bit string of a tile is cyclic)
    uint32_t woff[kWin][2];
#pragma unroll
    for (int w = 0; w < kWin; w++) {
      woff[w][0] = (uint32_t)(((ln.dw[w] + kTileDw) % kTileDw) * 4);
      woff[w][1] = (uint32_t)(((ln.dw[w] + 1) % kTileDw) * 4);
    }
    const int nt_n = n_out >> 4;
    const int64_t kt_bytes = (int64_t)nt_n * (32 * BITS);             // one k-tile of the whole matrix
    const uint8_t* run0 = trellis + (int64_t)((n0 >> 4) + nt0) * (32 * BITS);  // this wavefront's column blocks, k-tile 0
    uint8_t* ring = raw + pw * RG::kRingBytes;
    const uint32_t ring_addr = (uint32_t)(size_t)(lptr_t)ring;
    // lane's share of a request: 16 bytes, the last ones of the run again where the run is shorter than the request
    int roff[RG::kReq];
#pragma unroll
    for (int r = 0; r < RG::kReq; r++) roff[r] = min(r * 1024 + lane * 16, RG::kRunBytes - 16);
    auto request = [&](int s) {                                       // step s of this workgroup (clamped by the caller)
      const uint8_t* src = run0 + (int64_t)(4 * (step0 + s) + ktl) * kt_bytes;
      uint8_t* dst = ring + (s & (kXgAhead - 1)) * RG::kSlotBytes;
#pragma unroll
      for (int r = 0; r < RG::kReq; r++)
        __builtin_amdgcn_global_load_lds((gptr_t)(src + roff[r]), (lptr_t)(dst + r * 1024), 16, 0, 0);
    };
    const uint32_t sw_addr = (uint32_t)(size_t)(lptr_t)(&sw[0]);
    // B fragment unit of (k-tile ktl of the step, column block nt, this lane): ksub = ktl / 2, k-group 2 (ktl % 2) + q / 2,
    // column j; the lane's four weights are the lower or upper half of the unit's eight
    const uint32_t unit0 = (uint32_t)((ktl >> 1) * (NJ * 64) + nt0 * 64 + (((ktl & 1) * 2 + (q >> 1)) * 16) + j) * 16u +
                           (uint32_t)((q & 1) * 8);
    // The window dwords of four tiles are read by one statement and waited for by another, so that their LDS
    // latencies overlap (the reads are inline asm: the compiler would put a wait for every request in flight in front
    // of a read of the ring that it can see).
    struct Win4 { uint32_t v[4][kWin][2]; };
    auto read4 = [&](uint32_t slot, auto ntc, Win4& r) {
      constexpr int NT0 = decltype(ntc)::value;
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int w = 0; w < kWin; w++) {
          const uint32_t a0 = slot + woff[w][0], a1 = slot + woff[w][1];
          asm volatile("ds_read_b32 %0, %2 offset:%4\n\tds_read_b32 %1, %3 offset:%4"
                       : "=&v"(r.v[t][w][0]), "=&v"(r.v[t][w][1])
                       : "v"(a0), "v"(a1), "n"((NT0 + t) * 32 * BITS)
                       : "memory");
        }
    };
    auto settle4 = [&](Win4& r) {
      if constexpr (kWin == 1)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(r.v[0][0][0]), "+v"(r.v[0][0][1]), "+v"(r.v[1][0][0]), "+v"(r.v[1][0][1]), "+v"(r.v[2][0][0]),
                       "+v"(r.v[2][0][1]), "+v"(r.v[3][0][0]), "+v"(r.v[3][0][1])
                     :
                     : "memory");
      else
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(r.v[0][0][0]), "+v"(r.v[0][0][1]), "+v"(r.v[1][0][0]), "+v"(r.v[1][0][1]), "+v"(r.v[2][0][0]),
                       "+v"(r.v[2][0][1]), "+v"(r.v[3][0][0]), "+v"(r.v[3][0][1]), "+v"(r.v[0][kWin - 1][0]),
                       "+v"(r.v[0][kWin - 1][1]), "+v"(r.v[1][kWin - 1][0]), "+v"(r.v[1][kWin - 1][1]),
                       "+v"(r.v[2][kWin - 1][0]), "+v"(r.v[2][kWin - 1][1]), "+v"(r.v[3][kWin - 1][0]),
                       "+v"(r.v[3][kWin - 1][1])
                     :
                     : "memory");
    };
    auto decode4 = [&](uint32_t dst, auto ntc, const Win4& r) {
      constexpr int NT0 = decltype(ntc)::value;
#pragma unroll
      for (int t = 0; t < 4; t++) {
        uint32_t c[kWin][2];
#pragma unroll
        for (int w = 0; w < kWin; w++) {
          c[w][0] = __builtin_amdgcn_alignbit(r.v[t][w][0], r.v[t][w][0], 16);
          c[w][1] = __builtin_amdgcn_alignbit(r.v[t][w][1], r.v[t][w][1], 16);
        }
        const f16x4_t v = ln.template decode<CB>(c);
        uint64_t bits64;
        __builtin_memcpy(&bits64, &v, 8);
        asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(dst), "v"(bits64), "n"((NT0 + t) * 1024) : "memory");
      }
    };
    auto produce = [&](int s, int buf) {
      const uint32_t slot = ring_addr + (uint32_t)((s & (kXgAhead - 1)) * RG::kSlotBytes);
      const uint32_t dst = sw_addr + (uint32_t)(buf * kWUnits * 16) + unit0;
      Win4 ra;
      read4(slot, std::integral_constant<int, 0>{}, ra);
      if constexpr (kXgTiles == 8) {
        Win4 rb;
        read4(slot, std::integral_constant<int, 4>{}, rb);
        settle4(ra);                     // (waits for rb's reads too: they are issued, and complete in order)
        decode4(dst, std::integral_constant<int, 0>{}, ra);
        settle4(rb);
        decode4(dst, std::integral_constant<int, 4>{}, rb);
      } else {
        settle4(ra);
        decode4(dst, std::integral_constant<int, 0>{}, ra);
      }
    };
    // requests complete in order: all but the youngest kXgAhead - 1 steps' worth have landed
    auto wait_step = [&]() { wait_vmcnt<(kXgAhead - 1) * RG::kReq>(); };
#pragma unroll
    for (int s = 0; s < kXgAhead; s++) request(min(s, ksteps - 1));
    wait_step();
    produce(0, 0);
    bar();                               // barrier -1
    for (int s = 0; s < ksteps; s++) {
      // step s has been decoded: its slot takes the requests of step s + kXgAhead; then step s + 1 is decoded
      request(min(s + kXgAhead, ksteps - 1));
      wait_step();
      if (s + 1 < ksteps) produce(s + 1, (s + 1) & 1);
      bar();                             // barrier s
    }
    wait_vmcnt<0>();
    return;
  }

  // -------------------------------------------------------------------- consumer (as in gemm_pcd_kernel)
  const int m0 = m_tile * kPcBM + wave * (16 * MB);
  const int row_blocks_x = (m + 15) >> 4;
  const uint64_t xaddr = (uint64_t)(size_t)xp;
  u32x4_t xrsrc = {(uint32_t)xaddr, (uint32_t)(xaddr >> 32) & 0xFFFFu, (uint32_t)row_blocks_x * (uint32_t)(n_in * 32),
                   0x00020000u};
#pragma unroll
  for (int q = 0; q < 4; q++) xrsrc[q] = (uint32_t)__builtin_amdgcn_readfirstlane((int)xrsrc[q]);
  int aoff[MB];
#pragma unroll
  for (int ib = 0; ib < MB; ib++) aoff[ib] = min((m0 >> 4) + ib, row_blocks_x - 1) * 2048 + lane * 16;
  auto step_koff = [&](int ks) { return (step0 + min(ks, ksteps - 1)) * (row_blocks_x * 2048); };
  constexpr int G = 2 * NJ;
  f32x4_t acc[MB][NJ];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int jj = 0; jj < NJ; jj++) acc[i][jj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto finish = [&]() {
    wait_vmcnt<0>();               // the re-reads past the last step
    PcEpi epi{sp, ksplit, m_tile, n_tile, n_tiles, wave, lane, stg + wave * kStgBytes, yv, y_dtype, bias, bias_dtype, m,
              n_out, n0, m0};
    epi.col_scale = svh;
    pc_epilogue<NJ, MB, false, NC, true>(acc, epi);
  };

  if constexpr (MB == 4) {
    // 256-row tiles: 128 accumulators leave room for the A fragments of four half steps (32 k: MB requests, 4 MB
    // registers each) rotating by position: the fragments of half step q + 3 are requested during half step q.  A
    // group is four matrix instructions, so B fragments two groups ahead in a ring of four are enough.
    struct AHalf { u32x4_t v[MB]; };
    auto request_half = [&](AHalf& dst, int koff, auto hc, int ib) {
      if constexpr (decltype(hc)::value == 0) buffer_load16_async<0>(dst.v[ib], xrsrc, aoff[ib], koff);
      else buffer_load16_async<1024>(dst.v[ib], xrsrc, aoff[ib], koff);
    };
    f16x8_t bring[4];
    auto read_b = [&](f16x8_t& dst, int buf, int g) {
      const uint4 v = sw[buf * kWUnits + g * 64 + lane];
      __builtin_memcpy(&dst, &v, 16);
    };
    static_assert((G & 3) == 0 && MB <= NJ, "a step brings the B ring back to slot 0; one A request per group");
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    auto half_step = [&](const AHalf& cur, AHalf& into, auto bufc, auto hc, int ks) {
      constexpr int BUF = decltype(bufc)::value, HALF = decltype(hc)::value;
      // requests complete in order: all but those of the next two half steps have landed, `cur` among them
      wait_vmcnt<2 * MB>();
      const int koff3 = step_koff(ks + (HALF + 3) / 2);
#pragma unroll
      for (int j = 0; j < NJ; j++) {
        const int g = HALF * NJ + j;
        if (g == G - 2) bar();     // barrier ks: step ks+1 is in LDS, reads of step ks done
        if (g + 2 < G) read_b(bring[(g + 2) & 3], BUF, g + 2);
        else read_b(bring[(g + 2) & 3], BUF ^ 1, g + 2 - G);
#pragma unroll
        for (int r = 0; r < MB; r++)
          if (r * NJ / MB == j) request_half(into, koff3, std::integral_constant<int, (HALF + 3) & 1>{}, r);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MB; i++) {
          f16x8_t a;
          __builtin_memcpy(&a, &cur.v[i], 16);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bring[g & 3], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    AHalf h0{}, h1{}, h2{}, h3{};
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_half(h0, step_koff(0), H0{}, ib);
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_half(h1, step_koff(0), H1{}, ib);
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_half(h2, step_koff(1), H0{}, ib);
    bar();                         // barrier -1: the W fragments of step 0 are in LDS
    read_b(bring[0], 0, 0);
    read_b(bring[1], 0, 1);
    // (the number of steps is even: the half-step sets and the W buffers both come round after two steps)
    for (int ks = 0; ks < ksteps; ks += 2) {
      half_step(h0, h3, H0{}, H0{}, ks);
      half_step(h1, h0, H0{}, H1{}, ks);
      half_step(h2, h1, H1{}, H0{}, ks + 1);
      half_step(h3, h2, H1{}, H1{}, ks + 1);
    }
    finish();
    return;
  }

  struct ASet { u32x4_t v[2][MB]; };
  auto request_one = [&](ASet& dst, int koff, int h, int ib) {
    if (h == 0) buffer_load16_async<0>(dst.v[0][ib], xrsrc, aoff[ib], koff);
    else buffer_load16_async<1024>(dst.v[1][ib], xrsrc, aoff[ib], koff);
  };
  static_assert(2 * MB <= G, "one A request per group");
  // B fragments are read kAheadB groups ahead of their use into a ring of kRing: a group is only MB matrix
  // instructions (16 clocks each), and an LDS read takes more than a hundred clocks to come back
  constexpr int kRing = MB == 1 ? 16 : 8, kAheadB = kRing - 2;
  static_assert(G % kRing == 0 && kAheadB < G, "a step brings the ring back to slot 0");
  f16x8_t bring[kRing];
  auto read_b = [&](f16x8_t& dst, int buf, int g) {   // g = half * NJ + j
    const uint4 v = sw[buf * kWUnits + g * 64 + lane];
    __builtin_memcpy(&dst, &v, 16);
  };
  // A fragments run kDepth - 1 steps ahead of their use: the copy of Xr was written by the pass before this one, so a
  // step's fragments come from the memory side of the L2 (more than a microsecond away) for the first workgroup of
  // an XCD that asks, and steps are short here (a third of a microsecond with 64-row tiles).
  constexpr int kDepth = MB == 1 ? 6 : 3;      // (more would not fit the 168 registers of twelve wavefronts at MB = 2)
  constexpr int kUnroll = kDepth % 2 == 0 ? kDepth : 2 * kDepth;
  auto step = [&](const ASet& cur, ASet& into, auto bufc, int ks) {
    constexpr int BUF = decltype(bufc)::value;
    // requests complete in order: all but those of the kDepth - 2 steps after this one have landed
    wait_vmcnt<(kDepth - 2) * 2 * MB>();
    const int koff2 = step_koff(ks + kDepth - 1);
#pragma unroll
    for (int g = 0; g < G; g++) {
      if (g == G - kAheadB) bar();     // barrier ks: step ks+1 is in LDS, reads of step ks done
      if (g + kAheadB < G) read_b(bring[(g + kAheadB) % kRing], BUF, g + kAheadB);
      else read_b(bring[(g + kAheadB) % kRing], BUF ^ 1, g + kAheadB - G);
#pragma unroll
      for (int r = 0; r < 2 * MB; r++)
        if (r * G / (2 * MB) == g) request_one(into, koff2, r % 2, r / 2);
      __builtin_amdgcn_sched_barrier(0);
      const int half = g / NJ, jj = g % NJ;
#pragma unroll
      for (int i = 0; i < MB; i++) {
        f16x8_t a;
        __builtin_memcpy(&a, &cur.v[half][i], 16);
        acc[i][jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bring[g % kRing], acc[i][jj], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  ASet sets[kDepth];
#pragma unroll
  for (int d = 0; d < kDepth - 1; d++)
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int ib = 0; ib < MB; ib++) request_one(sets[d], step_koff(d), h, ib);
  bar();                         // barrier -1: the W fragments of step 0 are in LDS
#pragma unroll
  for (int g = 0; g < kAheadB; g++) read_b(bring[g], 0, g);
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  // (the number of steps is even; the register sets rotate with period kDepth, the W buffers with period two)
  for (int ks = 0; ks < ksteps; ks += kUnroll) {
#pragma unroll
    for (int u = 0; u < kUnroll; u += 2) {
      if (ks + u >= ksteps) break;
      step(sets[u % kDepth], sets[(u + kDepth - 1) % kDepth], C0{}, ks + u);
      step(sets[(u + 1) % kDepth], sets[u % kDepth], C1{}, ks + u + 1);
    }
  }
  finish();
}

template <int BITS, int CB, int MB>
static hipError_t launch_exl3_pc_grid(const uint8_t* trellis, const uint16_t* svh, const uint16_t* xp, void* y, int y_dtype,
                                      const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, PcSplit sp,
                                      hipStream_t s) {
  constexpr int BN = 128, BM = 64 * MB;
  const int n_tiles = (int)(n_out / BN), m_tiles = (int)((m + BM - 1) / BM);
  int xcds_per_mtile = 0;
  unsigned nwg = (unsigned)(n_tiles * m_tiles);
  if (m_tiles >= 2 && m_tiles <= 8 && 8 % m_tiles == 0) {
    xcds_per_mtile = 8 / m_tiles;
    nwg = (unsigned)(((n_tiles + xcds_per_mtile - 1) / xcds_per_mtile) * 8);
  }
  sp.tile_wgs = (int)nwg;
  hipLaunchKernelGGL((gemm_exl3_pc_kernel<BITS, CB, MB>), dim3(nwg * (unsigned)sp.splits), dim3(xg_threads(MB)), 0, s,
                     trellis, svh, xp, y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles,
                     xcds_per_mtile, sp);
  return hipGetLastError();
}

}  // namespace ttq
