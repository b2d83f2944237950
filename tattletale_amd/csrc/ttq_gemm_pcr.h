// Measurement only (built into the ladder library, not into libttq_hip.so): the producer/consumer prefill GEMM of
// ttq_gemm_pcd.h as a persistent workgroup that walks several tiles, with a ring of W stages and counters in LDS in
// place of the per-step barrier.  Y (m, n_out) = X (m, n_in) * W^T.  It passes the same parity tests as the one-tile
// kernel but is 8-15 % slower on Q4_K 14336 x 4096 (m = 512 and 2048).  Beside the accumulators, a consumer's
// registers leave room for A fragments only one and a half steps ahead when the loop also has to carry them across
// tiles (the one-tile kernel keeps two whole steps in flight, which is what the L2 latency under load needs); looking
// at the producers' counters early, so that the consumers never wait for that LDS read, did not change the time.
// Kept so that the ladder can show the number.
//
// Replaces F.linear(x, weight) for a multi-row bf16 activation
// (workspace/libtorch/src/abi/neural_nets.nim:64-81; the prefill case of
//  workspace/transformers/src/layers/attn.nim:154-156).
//
// Roles as in ttq_gemm_pcd.h: four consumers (MFMA, B fragments from LDS, A fragments by buffer loads from the
// packed copy of X), four W producers (packed blocks -> canonical dequantization -> bf16 -> B fragments in LDS).
// What differs:
//   * One launch puts a workgroup on every compute unit and each walks its tiles (virtual workgroup ids
//     blockIdx.x, + gridDim.x, ...: the same tile of every XCD-aware grid the one-tile kernel would have been
//     launched with, so all tiles of a workgroup share their rows of X).  The roles treat the tiles' K loops as one
//     long sequence of steps: while the consumers convert and store a finished tile, the producers fill the ring
//     with the first steps of the next, and the A requests of those steps are already in flight.
//   * W stages form a ring of four.  Producer p counts the steps it has completed in prod[p], consumer c the steps
//     whose B fragments it has finished reading in cons[c] (LDS words; a wavefront's LDS operations execute in
//     order, so a count written after the data -- or after the reads -- is seen after them).  A consumer starts
//     step g once min(prod) > g, a producer writes step g once min(cons) >= g - 3; each keeps the last minimum it
//     saw and looks again only when that is not enough.  Nobody meets at a barrier: a wavefront that falls behind
//     for a step delays only those that really need its data, and only once the ring's slack is used up.
//   * Every wait is bounded (a spin count far above anything a live partner needs); a wavefront that gives up goes
//     on with what it has, so a kernel always ends (its results are then wrong, which the parity tests would show).
#pragma once

#include "ttq_gemm_pcd.h"

namespace ttq {

constexpr int kPcrThreads = 512;         // 4 consumers, 4 W producers
constexpr int kPcrStages = 4;            // W stages in the ring (the step loop is unrolled over them)
constexpr int kPcrSpinLimit = 1 << 20;  // polls of a few hundred cycles each: a fraction of a second

// the smallest of four consecutive LDS words, as a wavefront-uniform value
__device__ __forceinline__ uint32_t lds_min4_uniform(uint32_t lds_addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_addr) : "memory");
  const uint32_t a = v[0] < v[1] ? v[0] : v[1], b = v[2] < v[3] ? v[2] : v[3];
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)(a < b ? a : b));
}

// one LDS word written by lane 0, after every LDS operation the wavefront has issued before
__device__ __forceinline__ void lds_post(uint32_t lds_addr, uint32_t value, int lane) {
  asm volatile("" ::: "memory");
  if (lane == 0) asm volatile("ds_write_b32 %0, %1" : : "v"(lds_addr), "v"(value) : "memory");
}

template <int NJ, int FMT, int MB, bool FUSE>
__global__ void __launch_bounds__(kPcrThreads)
gemm_pcr_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ xp, void* __restrict__ yv,
                int y_dtype, const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in,
                int n_tiles, int m_tiles, int xcds_per_mtile, int virtual_wgs) {
  constexpr int BN = NJ * 16;
  constexpr int NW = kPcrStages;
  constexpr int kWUnits = 2 * NJ * 64;
  constexpr int kPcBM = 64 * MB;
  constexpr int kStgBytes = 16 * MB * (BN * 2 + 16);      // a consumer's epilogue staging area
  constexpr int BO = FUSE ? BN / 2 : BN;                  // outputs per tile
  __shared__ uint4 sw[NW * kWUnits];
  __shared__ __attribute__((aligned(16))) uint8_t stg[4 * kStgBytes];
  __shared__ __attribute__((aligned(16))) uint32_t counts[8];   // prod[0..3], cons[0..3]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid < 8) counts[tid] = 0u;
  __syncthreads();
  const uint32_t prod_addr = (uint32_t)(size_t)(lptr_t)(&counts[0]);
  const uint32_t cons_addr = (uint32_t)(size_t)(lptr_t)(&counts[4]);

  // This workgroup's tiles: virtual workgroup ids vb = blockIdx.x + i * gridDim.x, mapped to tiles as the one-tile
  // kernels map blockIdx.x (ids past the last column tile of an XCD-aware grid name no tile and are skipped, by
  // both roles alike).  With the XCD-aware map (gridDim.x a multiple of 8) all of them share one row tile.
  auto tile_of = [&](int vb, int& m_tile, int& n_tile) {
    if (xcds_per_mtile > 0) {
      const int xcd = vb & 7, slot = vb >> 3;
      m_tile = xcd / xcds_per_mtile;
      n_tile = slot * xcds_per_mtile + xcd % xcds_per_mtile;
    } else {
      m_tile = vb % m_tiles;
      n_tile = vb / m_tiles;
    }
    return n_tile < n_tiles;
  };
  const int ksteps = n_in >> 6;
  const int nblocks = n_in >> 8;                   // super-blocks (256 k) in a row of W
  int my_tiles = 0;
  for (int vb = blockIdx.x; vb < virtual_wgs; vb += gridDim.x) {
    int mt, nt;
    if (tile_of(vb, mt, nt)) my_tiles++;
  }
  if (my_tiles == 0) return;
  const uint32_t total_steps = (uint32_t)my_tiles * (uint32_t)ksteps;

  if (wave >= 4) {
    // ------------------------------------------------------------------ W producer
    const int pt = tid - 256;
    constexpr bool kSpare = 4 * BN <= 256;
    const bool widle = kSpare && pt >= 2 * BN;
    const int wt = pt < 2 * BN ? pt : (kSpare ? pt % (2 * BN) : pt - 2 * BN);
    const int wr = wt >> 1, whalf = wt & 1;          // the two halves of a row in adjacent lanes
    const int wj = wr >> 4, wn = wr & 15;
    using WF = WFmt<FMT>;
    using WRaw = typename WF::Raw;
    const uint32_t sw_addr = (uint32_t)(size_t)(lptr_t)(&sw[0]);
    // flattened blocks: fb = (tile index in this workgroup's list) * nblocks + b.  The list is walked once, in order,
    // by a cursor that only moves forward.
    int cur_vb = blockIdx.x - (int)gridDim.x, cur_idx = -1;
    const uint8_t* cur_row = w;
    auto row_of_tile = [&](int idx) {      // idx >= cur_idx
      while (cur_idx < idx) {
        int mt, nt;
        do {
          cur_vb += (int)gridDim.x;
        } while (!tile_of(cur_vb, mt, nt));
        cur_idx++;
        const int n0 = nt * BO;
        // clamped: rows past the end are never stored
        const int wrow = FUSE ? min(n0 + 8 * (wr >> 4) + (wr & 7), n_out - 1) + ((wr >> 3) & 1) * n_out
                              : min(n0 + wr, n_out - 1);
        cur_row = w + (int64_t)nblocks * WF::kUnitBytes * (int64_t)wrow;
      }
      return cur_row;
    };
    const int total_blocks = my_tiles * nblocks;
    auto load_w = [&](WRaw& dst, int fb) {
      if (widle) return;
      fb = min(fb, total_blocks - 1);                 // past the end: a harmless re-read
      const int idx = fb / nblocks, b = fb - idx * nblocks;
      WF::load(dst, row_of_tile(idx) + WF::kUnitBytes * (int64_t)b, whalf);
    };
    uint32_t cons_seen = 0;
    bool gave_up = false;                  // a wait ran out: no further waiting, the kernel just ends
    auto produce = [&](const WRaw& r, auto cc, uint32_t g) {
      // stage g % NW is free once every consumer has finished reading step g - NW
      if (g >= (uint32_t)NW && cons_seen < g + 1u - (uint32_t)NW && !gave_up) {
        int spin = 0;
        for (; spin < kPcrSpinLimit; spin++) {
          cons_seen = lds_min4_uniform(cons_addr);
          if (cons_seen >= g + 1u - (uint32_t)NW) break;
          __builtin_amdgcn_s_sleep(1);
        }
        gave_up = spin == kPcrSpinLimit;
      }
      if (!widle) pc_dequant_to_lds<NJ, FMT, 0, decltype(cc)::value>(r, (int)(g % (uint32_t)NW), whalf, wj, wn, sw_addr);
      lds_post(prod_addr + 4u * (uint32_t)(wave - 4), g + 1u, lane);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // Block fb + 2 is requested at the start of block fb, into the register set block fb - 1 used: three sets rotate
    // by name.  These wavefronts issue no other global loads, so the compiler's own counting of outstanding
    // requests is exact.
    auto do_block = [&](const WRaw& cur, WRaw& into, int fb) {
      load_w(into, fb + 2);
      const uint32_t g0 = 4u * (uint32_t)fb;
      produce(cur, I0{}, g0);
      produce(cur, I1{}, g0 + 1u);
      produce(cur, I2{}, g0 + 2u);
      produce(cur, I3{}, g0 + 3u);
    };
    WRaw wa{}, wb{}, wc{};
    load_w(wa, 0);
    load_w(wb, 1);
    for (int fb = 0; fb < total_blocks; fb += 3) {
      do_block(wa, wc, fb);
      if (fb + 1 < total_blocks) do_block(wb, wa, fb + 1);
      if (fb + 2 < total_blocks) do_block(wc, wb, fb + 2);
    }
    return;
  }

  // -------------------------------------------------------------------- consumer
  int vb = blockIdx.x, m_tile = 0, n_tile = 0;
  while (!tile_of(vb, m_tile, n_tile)) vb += (int)gridDim.x;
  int m0 = m_tile * kPcBM + wave * (16 * MB);
  // A fragments from the packed copy (see ttq_gemm_pcd.h); all tiles of this workgroup share their rows when the
  // grid is XCD-aware, otherwise the offsets are set again at every tile
  const int row_blocks_x = (m + 15) >> 4;
  const uint64_t xaddr = (uint64_t)(size_t)xp;
  u32x4_t xrsrc = {(uint32_t)xaddr, (uint32_t)(xaddr >> 32) & 0xFFFFu, (uint32_t)row_blocks_x * (uint32_t)(n_in * 32),
                   0x00020000u};
#pragma unroll
  for (int q = 0; q < 4; q++) xrsrc[q] = (uint32_t)__builtin_amdgcn_readfirstlane((int)xrsrc[q]);
  int aoff[MB];
  auto set_rows = [&]() {
#pragma unroll
    for (int ib = 0; ib < MB; ib++) aoff[ib] = min((m0 >> 4) + ib, row_blocks_x - 1) * 2048 + lane * 16;
  };
  set_rows();
  // A fragments by half steps (32 k: MB requests, 4 MB registers) in a ring of four sets that rotate by name: the
  // fragments of half step q + 3 are requested during half step q.
  struct AHalf { u32x4_t v[MB]; };
  auto request_one = [&](AHalf& dst, int koff, auto hc, int ib) {
    if constexpr (decltype(hc)::value == 0) buffer_load16_async<0>(dst.v[ib], xrsrc, aoff[ib], koff);
    else buffer_load16_async<1024>(dst.v[ib], xrsrc, aoff[ib], koff);
  };
  const int step_bytes = row_blocks_x * 2048;      // a 64-k step of the packed copy
  constexpr int G = 2 * NJ;
  static_assert(MB <= NJ && NJ >= 4, "one A request per group; the early poll sits in the second half step");
  static_assert(((2 * G) & 3) == 0, "two steps bring the B ring back to slot 0");
  static_assert(NW == 4, "the step loop is unrolled over four stages");
  bf16x8_t bring[4];
  auto read_b = [&](bf16x8_t& dst, int stage, int g) {   // g = half * NJ + j
    const uint4 v = sw[stage * kWUnits + g * 64 + lane];
    __builtin_memcpy(&dst, &v, 16);
  };

  f32x4_t acc[MB][NJ];
  auto clear_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
      for (int j = 0; j < NJ; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  };
  clear_acc();

  uint32_t gstep = 0, prod_seen = 0;      // global step of this workgroup; the producers' progress as last seen
  int ks = 0;                             // step inside the current tile
  bool gave_up = false;                   // a wait ran out: no further waiting, the kernel just ends
  auto wait_prod = [&](uint32_t need) {   // until all producers have completed `need` steps
    if (need > total_steps) need = total_steps;
    if (prod_seen >= need || gave_up) return;
    for (int spin = 0; spin < kPcrSpinLimit; spin++) {
      prod_seen = lds_min4_uniform(prod_addr);
      if (prod_seen >= need) return;
      __builtin_amdgcn_s_sleep(1);
    }
    gave_up = true;
  };
  // Half a step: NJ groups of MB MFMAs.  `cur` holds its A fragments, `into` receives those of the half step three
  // further on (of the next tile near the end of this one: same rows, the K offset wraps); ST is the step's W stage
  // and fixes the B ring slot of its first group.  B fragments are read two groups ahead, across half and step ends.
  auto half_step = [&](const AHalf& cur, AHalf& into, auto stc, auto hc) {
    constexpr int ST = decltype(stc)::value, STN = (ST + 1) % NW, HALF = decltype(hc)::value;
    constexpr int SO = ((ST & 1) * G) & 3;
    // requests complete in order: all but the youngest 2 * MB (the next two half steps) have landed, `cur` among them
    wait_vmcnt<2 * MB>();
    int ks3 = ks + (HALF + 3) / 2;
    if (ks3 >= ksteps) ks3 -= ksteps;
    const int koff3 = ks3 * step_bytes;
    u32x4_t polled = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < NJ; j++) {
      const int g = HALF * NJ + j;
      if (g == G - 4) {
        // look at the producers' counters two groups before the answer is needed: the read is then complete without
        // a wait of its own (the B reads of two groups are the only LDS operations younger than it)
        asm volatile("ds_read_b128 %0, %1" : "=v"(polled) : "v"(prod_addr) : "memory");
      }
      if (g == G - 2) {
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(polled) : : "memory");
        if (!gave_up) {
          const uint32_t a = polled[0] < polled[1] ? polled[0] : polled[1];
          const uint32_t b = polled[2] < polled[3] ? polled[2] : polled[3];
          prod_seen = (uint32_t)__builtin_amdgcn_readfirstlane((int)(a < b ? a : b));
        }
        // every B read of this step has been issued: its stage is free once they have executed.  The next step's
        // fragments must be complete before its first two groups are read.
        lds_post(cons_addr + 4u * (uint32_t)wave, gstep + 1u, lane);
        wait_prod(gstep + 2u);
      }
      if (g + 2 < G) read_b(bring[(g + 2 + SO) & 3], ST, g + 2);
      else read_b(bring[(g + 2 + SO) & 3], STN, g + 2 - G);
#pragma unroll
      for (int r = 0; r < MB; r++)
        if (r * NJ / MB == j) request_one(into, koff3, std::integral_constant<int, (HALF + 3) & 1>{}, r);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MB; i++) {
        bf16x8_t a;
        __builtin_memcpy(&a, &cur.v[i], 16);
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bring[(g + SO) & 3], acc[i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (HALF == 1) {
      gstep++;
      ks++;
    }
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using C2 = std::integral_constant<int, 2>;
  using C3 = std::integral_constant<int, 3>;

  AHalf h0{}, h1{}, h2{}, h3{};
  auto start_rows = [&]() {      // the first three half steps of a tile
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_one(h0, 0, C0{}, ib);
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_one(h1, 0, C1{}, ib);
#pragma unroll
    for (int ib = 0; ib < MB; ib++) request_one(h2, step_bytes, C0{}, ib);
  };
  start_rows();
  wait_prod(1u);
  read_b(bring[0], 0, 0);
  read_b(bring[1], 0, 1);
  // Four steps per pass (the half-step sets rotate with period two steps, the stages with period four); a tile is a
  // whole number of passes (its steps are a multiple of four).
  int tiles_done = 0;
  for (;;) {
    half_step(h0, h3, C0{}, C0{});
    half_step(h1, h0, C0{}, C1{});
    half_step(h2, h1, C1{}, C0{});
    half_step(h3, h2, C1{}, C1{});
    half_step(h0, h3, C2{}, C0{});
    half_step(h1, h0, C2{}, C1{});
    half_step(h2, h1, C3{}, C0{});
    half_step(h3, h2, C3{}, C1{});
    if (ks < ksteps) continue;
    // ---- a tile is finished: store it (the producers are already at work on the next, and its first A fragments
    // have been requested; they are waited for here, so that nothing the compiler does with registers in the
    // epilogue can touch one that a request still writes to)
    wait_vmcnt<0>();
    pc_epilogue<NJ, MB, FUSE, 4>(acc, PcEpi{PcSplit{1, 0, nullptr, nullptr}, 0, m_tile, n_tile, n_tiles, wave, lane,
                                            stg + wave * kStgBytes, yv, y_dtype, bias, bias_dtype, m, n_out, n_tile * BO,
                                            m0});
    if (++tiles_done == my_tiles) break;
    clear_acc();
    ks = 0;
    const int prev_m_tile = m_tile;
    do {
      vb += (int)gridDim.x;
    } while (!tile_of(vb, m_tile, n_tile));
    if (m_tile != prev_m_tile) {
      // (only without the XCD-aware map) the fragments requested ahead belong to the old rows: start again
      m0 = m_tile * kPcBM + wave * (16 * MB);
      set_rows();
      start_rows();
    }
  }
  wait_vmcnt<0>();               // the re-reads past the last step
}

// One workgroup per compute unit (fewer when there are fewer tiles); grid_wgs must be a multiple of 8 when the map is
// XCD-aware.  The launch is not split along K.
template <int FMT, int MB, int NJ, bool FUSE>
static hipError_t launch_pcr_grid(const uint8_t* wb, const uint16_t* xp, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int grid_cap, hipStream_t s) {
  constexpr int BO = FUSE ? NJ * 8 : NJ * 16, BM = 64 * MB;
  const int n_tiles = (int)((n_out + BO - 1) / BO), m_tiles = (int)((m + BM - 1) / BM);
  int xcds_per_mtile = 0;
  int virtual_wgs = n_tiles * m_tiles;
  if (m_tiles >= 2 && m_tiles <= 8 && 8 % m_tiles == 0) {
    xcds_per_mtile = 8 / m_tiles;
    virtual_wgs = ((n_tiles + xcds_per_mtile - 1) / xcds_per_mtile) * 8;
  }
  int grid = virtual_wgs < grid_cap ? virtual_wgs : grid_cap;
  if (xcds_per_mtile > 0) grid = grid / 8 * 8;
  if (grid <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL((gemm_pcr_kernel<NJ, FMT, MB, FUSE>), dim3((unsigned)grid), dim3(kPcrThreads), 0, s, wb, xp, y,
                     y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, n_tiles, m_tiles, xcds_per_mtile, virtual_wgs);
  return hipGetLastError();
}

}  // namespace ttq
