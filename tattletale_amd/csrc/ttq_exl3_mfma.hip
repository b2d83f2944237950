// Trellis-coded (EXL3-style) decode GEMV on the fp16 matrix cores, one launch:
//
//   y = svh o H( T * H(suh o x) ) + bias
//
// Work split.  A workgroup owns one Hadamard group of 128 output channels (8 tiles across) and one
// slice of the reduction dimension; its 8 wavefronts take one 16-channel tile column each.  The
// slices of a group hand their sums to the group's last slice through tagged words in a workspace (one
// store and one load each); the last slice adds them in a fixed order, rotates the 128 sums of
// each row and writes y.  With one slice there is no workspace traffic.
//
// Weights.  For one k-tile the 8 tiles of the group are contiguous in trellis[k_tile][n_tile][16*bits],
// so the workgroup copies whole runs of 256*bits bytes, 16 bytes per lane, into LDS: up to 32 k-tiles per
// pass, requested one pass ahead.  On the way in every dword's halves are swapped, which turns the
// string of 16-bit words (most significant bit first) into a string of big-endian dwords; every tile
// is followed by a copy of its first dword, because the string is cyclic.
//
// Decode.  v_mfma_f32_16x16x16_f16 wants from lane (j = lane % 16, q = lane / 16) the four weights
// k = 4q .. 4q+3 of channel j: the windows that start at bit (16j + 4q + e) * bits, e = 0..3.  The
// lane reads the two dwords that hold them, one funnel shift aligns the first window to bit 31, and
// the others are bit fields at constant offsets below it (two funnel shifts for 6..8 bits per weight).
// Per weight: one bit-field extract, one 32-bit multiply, one three-input bit operation, one fp16 add
// that writes its half of the A fragment directly.
//
// Activations.  Each slice rotates its own part of x: x o suh, the 128-group butterfly in registers,
// then a power-of-two scale per (row, group) that brings the group's largest magnitude to 2^14, and a
// split into two fp16 terms (value and remainder), which together carry 22 bits.  The B operand holds
// up to 8 activation rows as 16 columns (term 0, term 1 of each); the two columns are added at the end,
// and each group's matrix-core sum is scaled back in fp32 before it joins the running sum.
#include "ttq_exl3_common.h"

#include <mutex>
#include <unordered_map>

namespace ttq {

template <int BITS, int CB, typename XT>
__global__ void __launch_bounds__(kXmThreads)
gemv_exl3_mfma_kernel(const uint16_t* __restrict__ trellis, const uint16_t* __restrict__ suh,
                      const uint16_t* __restrict__ svh, const XT* __restrict__ x, void* __restrict__ y, int y_dtype,
                      const void* __restrict__ bias, int bias_dtype, int m, int n_out, int n_in, int slice_tiles,
                      unsigned long long* __restrict__ accum, int poll_limit) {
  using G = XmGeom<BITS>;
  __shared__ uint32_t slab[G::kSlabDw];
  __shared__ __attribute__((aligned(16))) _Float16 xs[2 * kXmTok * kXmColStride];
  __shared__ float inv_s[kXmChunkTiles / 8][2 * kXmTok];
  __shared__ __attribute__((aligned(16))) float yp[kXmTok * 128];
  __shared__ __attribute__((aligned(16))) float yq[(kXmKSplit - 1) * kXmTok * 128 + 4];   // the other wavefronts of a tile column

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = blockIdx.x, slice = blockIdx.y, nslices = gridDim.y;
  const int t0 = blockIdx.z * kXmTok;
  const int ntok = min(kXmTok, m - t0);
  const int nt_n = n_out >> 4, kt_n = n_in >> 4;
  const int kt_begin = slice * slice_tiles;
  const int kt_end = min(kt_n, kt_begin + slice_tiles);
  const int col = lane & 15, q = lane >> 4;

  XmLane<BITS> ln;
  ln.init(lane);

  // The tag of this launch's hand-off words: the workspace's generation count + 1 (read now, needed at the end).
  // accum[0] holds the generation, accum[1] the number of groups that have finished, the words start at accum + 8.
  uint32_t tag = 0;
  if (nslices > 1)
    tag = __hip_atomic_load(reinterpret_cast<const uint32_t*>(accum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;

  // ---- weights: global -> registers, one pass ahead
  const char* wbase = reinterpret_cast<const char*>(trellis) + (int64_t)grp * 8 * (32 * BITS);
  const int64_t row_bytes = (int64_t)nt_n * (32 * BITS);
  uint4 pre[G::kSets];
  // (a thread whose piece lies past the end of a short pass re-reads the last k-tile: no branch around the load)
  auto request = [&](int kt_first, int cnt) {
#pragma unroll
    for (int i = 0; i < G::kSets; i++) {
      const int p = tid + i * kXmThreads;
      const int ktl = p / G::kRunPieces, r = p - ktl * G::kRunPieces;
      pre[i] = *reinterpret_cast<const uint4*>(wbase + (int64_t)(kt_first + min(ktl, cnt - 1)) * row_bytes + r * 16);
    }
  };
  // piece set i of a pass (the i-th 16 bytes of every thread) into LDS
  auto stage = [&](int i, int cnt) {
    const int p = tid + i * kXmThreads;
    const int ktl = p / G::kRunPieces, r = p - ktl * G::kRunPieces;
    if (ktl < cnt) {
      const int nt = r / (2 * BITS), ci = r - nt * (2 * BITS);
      uint32_t* dst = slab + 1 + (ktl * 8 + nt) * G::kTileStride + 4 * ci;
      const uint32_t c0 = __builtin_amdgcn_alignbit(pre[i].x, pre[i].x, 16);
      dst[0] = c0;
      dst[1] = __builtin_amdgcn_alignbit(pre[i].y, pre[i].y, 16);
      dst[2] = __builtin_amdgcn_alignbit(pre[i].z, pre[i].z, 16);
      dst[3] = __builtin_amdgcn_alignbit(pre[i].w, pre[i].w, 16);
      if (ci == 0) dst[G::kTileDw] = c0;
    }
  };

  // ---- activations of a pass: (row, group) items of 32 lanes; an item's four values per lane are requested
  // early (before the weights of the first pass, one pass ahead after that) and rotated when the pass begins
  const int hw = tid >> 5, l32 = tid & 31;
  constexpr int kItemsPerThread = (kXmTok * 4 + kXmThreads / 32 - 1) / (kXmThreads / 32);
  XmRaw<XT> xv[kItemsPerThread];
  uint2 sv[kItemsPerThread];
  auto x_request = [&](int kt_first, int ngl) {
#pragma unroll
    for (int it = 0; it < kItemsPerThread; it++) {
      const int item = hw + it * (kXmThreads / 32), t = min(item >> 2, ntok - 1), gl = min(item & 3, ngl - 1);
      const int64_t k = (int64_t)kt_first * 16 + gl * 128 + 4 * l32;
      __builtin_memcpy(&sv[it], __builtin_assume_aligned(suh + k, 8), 8);
      xv[it].load(x + (int64_t)(t0 + t) * n_in + k);
    }
  };
  auto x_stage = [&](int ngl) {
#pragma unroll
    for (int it = 0; it < kItemsPerThread; it++) {
      const int item = hw + it * (kXmThreads / 32), t = item >> 2, gl = item & 3;
      if (item < kXmTok * 4 && t < ntok && gl < ngl) {
        float v[4];
        xv[it].get(v);
        v[0] *= f16_bits_to_f32((uint16_t)sv[it].x);
        v[1] *= f16_bits_to_f32((uint16_t)(sv[it].x >> 16));
        v[2] *= f16_bits_to_f32((uint16_t)sv[it].y);
        v[3] *= f16_bits_to_f32((uint16_t)(sv[it].y >> 16));
        fwht128_quad(v, lane);
        float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
        amax = fmaxf(amax, lane_xor<1>(amax, lane));
        amax = fmaxf(amax, lane_xor<2>(amax, lane));
        amax = fmaxf(amax, lane_xor<4>(amax, lane));
        amax = fmaxf(amax, lane_xor<8>(amax, lane));
        amax = fmaxf(amax, lane_xor<16>(amax, lane));
        // scale 2^(14 - exponent of amax); all-zero groups get the largest scale, which changes nothing
        int se = 268 - (int)((__float_as_uint(amax) >> 23) & 0xFF);
        se = se > 254 ? 254 : se;
        const float sc = __uint_as_float((uint32_t)se << 23);
        f16x4_t hi, lo;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float s = v[i] * sc;
          hi[i] = (_Float16)s;
          lo[i] = (_Float16)(s - (float)hi[i]);
        }
        const int kl = gl * 128 + 4 * l32;
        *reinterpret_cast<f16x4_t*>(xs + (2 * t) * kXmColStride + kl) = hi;
        *reinterpret_cast<f16x4_t*>(xs + (2 * t + 1) * kXmColStride + kl) = lo;
        if (l32 == 0) {
          // 1/sqrt(128) of the input rotation over the scale
          const float inv = 0.08838834764831845f * __uint_as_float((uint32_t)(254 - se) << 23);
          inv_s[gl][2 * t] = inv;
          inv_s[gl][2 * t + 1] = inv;
        }
      }
    }
  };

  {
    const int cnt0 = min(kXmChunkTiles, kt_end - kt_begin);
    x_request(kt_begin, cnt0 >> 3);
    __builtin_amdgcn_sched_barrier(0);     // the small loads stay in front of the weights: they are waited for first
    request(kt_begin, cnt0);
  }

  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int kt0 = kt_begin; kt0 < kt_end; kt0 += kXmChunkTiles) {
    const int cnt = min(kXmChunkTiles, kt_end - kt0);       // a multiple of 8
    const int ngl = cnt >> 3;
    if (kt0 != kt_begin) __syncthreads();                   // the previous pass has been read
    x_stage(ngl);
    // ---- decode and multiply: this wavefront's tile column and its share of every group's 8 k-tiles (one
    // Hadamard group per scale); the LDS reads of a group are issued while the group before it is decoded
    // (decoding a pass's first groups before its last pieces had landed was tried and gained nothing)
    const _Float16* xcol = xs + col * kXmColStride + 4 * q;
    const int tcol = wave & 7, kpart = wave >> 3;          // tile column, and which k-tiles of every group
    const uint32_t* wcol = slab + 1 + (kpart * kXmTilesPerWave * 8 + tcol) * G::kTileStride;
    const _Float16* xpart = xcol + kpart * kXmTilesPerWave * 16;
    constexpr int kWin = XmLane<BITS>::kWin;
    uint32_t cw[2][kXmTilesPerWave][kWin][2];
    f16x4_t bx[2][kXmTilesPerWave];
    float inv[2];
    auto fetch_group = [&](int gl, int buf) {
#pragma unroll
      for (int i = 0; i < kXmTilesPerWave; i++) {
        const int ktl = gl * 8 + i;
        ln.fetch(wcol + ktl * 8 * G::kTileStride, cw[buf][i]);
        bx[buf][i] = *reinterpret_cast<const f16x4_t*>(xpart + ktl * 16);
      }
      inv[buf] = inv_s[gl][col];
    };
    auto compute_group = [&](int buf) {
      f32x4_t d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < kXmTilesPerWave; i++)
        d = __builtin_amdgcn_mfma_f32_16x16x16f16(ln.template decode<CB>(cw[buf][i]), bx[buf][i], d, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; r++) acc[r] = fmaf_(d[r], inv[buf], acc[r]);
    };
#pragma unroll
    for (int i = 0; i < G::kSets; i++) stage(i, cnt);
    if (kt0 + kXmChunkTiles < kt_end) {
      const int cnt1 = min(kXmChunkTiles, kt_end - kt0 - kXmChunkTiles);
      x_request(kt0 + kXmChunkTiles, cnt1 >> 3);
      __builtin_amdgcn_sched_barrier(0);
      request(kt0 + kXmChunkTiles, cnt1);
    }
    __syncthreads();
    fetch_group(0, 0);
    for (int gl = 0; gl < ngl; gl += 2) {
      if (gl + 1 < ngl) fetch_group(gl + 1, 1);
      compute_group(0);
      if (gl + 1 < ngl) {
        if (gl + 2 < ngl) fetch_group(gl + 2, 0);
        compute_group(1);
      }
    }
  }

  // ---- the two terms of each row.  Then, in a sliced launch, every slice but the last hands its sums
  // to the last one straight from the registers, through tagged 64-bit words (the launch's tag in the high
  // half, the float in the low half) written and read with agent-scope accesses, which are coherent across
  // the chip without cache maintenance.  The last slice polls each word until this launch's tag is there
  // (a bounded number of times: rows it gave up on come out as NaN) and adds everything in a fixed order.
  // Nothing is cleared: the tag is the workspace's generation count + 1, and the group that finishes last
  // advances the count, so the words of this launch -- also those of a slice that arrives after its group
  // gave up on it -- can never pass for words of a later one.  The count lives in the workspace and not in
  // a kernel argument because a captured graph replays its arguments.  What remains: a slice that has not
  // even begun when its group gives up reads the advanced count and tags its words like the next launch
  // will; that takes a wavefront dispatch held back for poll_limit polls (tens of milliseconds by default).
#pragma unroll
  for (int r = 0; r < 4; r++) acc[r] += lane_xor<1>(acc[r], lane);
  const int tcol = wave & 7, kpart = wave >> 3;
  const bool owner = (col & 1) == 0 && (col >> 1) < ntok;      // this lane holds 4 channel sums of row col / 2
  constexpr int kPartWords = kXmTok * 128;                        // words per (slice, k part)
  unsigned long long* words = nullptr;
  if (nslices > 1) {
    words = accum + 8 + (((int64_t)blockIdx.z * gridDim.x + grp) * nslices) * (kXmKSplit * kPartWords);
    if (slice != nslices - 1) {
      if (owner) {
        unsigned long long* dst = words + ((int64_t)slice * kXmKSplit + kpart) * kPartWords + (col >> 1) * 128 + tcol * 16 + 4 * q;
#pragma unroll
        for (int r = 0; r < 4; r++)
          __hip_atomic_store(dst + r, ((unsigned long long)tag << 32) | __float_as_uint(acc[r]), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      }
      return;
    }
  }
  {
    float* dst = kpart == 0 ? yp : yq + (kpart - 1) * kPartWords;
    if (owner) *reinterpret_cast<float4*>(dst + (col >> 1) * 128 + tcol * 16 + 4 * q) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  }
  __syncthreads();
  constexpr int kHandoffBatch = 16;
  for (int e = tid; e < ntok * 128; e += kXmThreads) {
    // the other slices' words for this output (sixteen loads in flight before the first is looked at: the fourteen
    // words of a launch in eight slices in one round trip to the memory side),
    // then this workgroup's own sums
    float s = 0.f;
    bool late = false;
    const int nparts = (nslices - 1) * kXmKSplit;
    // The slices of a group finish their decode within a fraction of a microsecond of each other, and a word asked for
    // before it has reached the memory side costs a second round trip (about 0.9 us); 256 clocks of patience before
    // the first look make the first look the only one (4096 x 4096, one row: 9.1 -> 8.8 us; two to six units of 64
    // clocks measure the same).
    if (nparts > 0) __builtin_amdgcn_s_sleep(4);
    for (int p0 = 0; p0 < nparts; p0 += kHandoffBatch) {
      unsigned long long w[kHandoffBatch];
#pragma unroll
      for (int i = 0; i < kHandoffBatch; i++)
        w[i] = __hip_atomic_load(words + (int64_t)min(p0 + i, nparts - 1) * kPartWords + e, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int i = 0; i < kHandoffBatch; i++) {
        if (p0 + i < nparts) {
          unsigned long long* wp = words + (int64_t)(p0 + i) * kPartWords + e;
          for (int polls = 0; (uint32_t)(w[i] >> 32) != tag && polls < poll_limit; polls++) {
            __builtin_amdgcn_s_sleep(2);
            w[i] = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          late |= (uint32_t)(w[i] >> 32) != tag;
          s += __uint_as_float((uint32_t)w[i]);
        }
      }
    }
    s += yp[e];
#pragma unroll
    for (int k = 1; k < kXmKSplit; k++) s += yq[(k - 1) * kPartWords + e];
    yp[e] = late ? __uint_as_float(0x7FC00000u) : s;
  }
  // Thread 0 has now seen (or given up on) a word of every other slice of its group, so each of them has read
  // the generation count.  It counts its group in here and looks at the answer after the output phase: the group
  // that is counted last advances the generation.
  uint32_t counted = 0;
  if (nslices > 1 && tid == 0)
    counted = __hip_atomic_fetch_add(reinterpret_cast<uint32_t*>(accum) + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();

  // ---- output side: rotate the 128 sums of each row, svh, bias
  if (hw < ntok) {
    float v[4];
    const float4 t = *reinterpret_cast<const float4*>(yp + hw * 128 + 4 * l32);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    fwht128_quad(v, lane);
    const int n = grp * 128 + 4 * l32;
    uint2 sraw;
    __builtin_memcpy(&sraw, __builtin_assume_aligned(svh + n, 8), 8);
    const float svf[4] = {f16_bits_to_f32((uint16_t)sraw.x), f16_bits_to_f32((uint16_t)(sraw.x >> 16)),
                          f16_bits_to_f32((uint16_t)sraw.y), f16_bits_to_f32((uint16_t)(sraw.y >> 16))};
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      o[i] = v[i] * 0.08838834764831845f * svf[i];
      if (bias) o[i] += load_bias(bias, bias_dtype, n + i);
    }
    xm_store4(y, y_dtype, (int64_t)(t0 + hw) * n_out + n, o);
  }
  if (nslices > 1 && tid == 0 && counted == gridDim.x * gridDim.z - 1) {
    uint32_t* ctl = reinterpret_cast<uint32_t*>(accum);
    __hip_atomic_store(ctl + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ctl, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ------------------------------------------------------------------------------ launch
Exl3Plan exl3_mfma_plan(int64_t m, int64_t n_out, int64_t n_in) {
  Exl3Plan p;
  p.groups = (int)(n_out / 128);
  p.row_groups = (int)((m + kXmTok - 1) / kXmTok);
  const int kt_n = (int)(n_in / 16);
  const int64_t units = (int64_t)p.groups * p.row_groups;
  const int cus = device_num_cus();
  // enough slices to put a workgroup on every compute unit, each a whole number of Hadamard groups
  int64_t want = units >= cus ? 1 : cus / units;
  if (want > kt_n / 8) want = kt_n / 8;
  int tiles = (int)((kt_n + want - 1) / want);
  tiles = (tiles + 7) / 8 * 8;
  p.slice_tiles = tiles;
  p.slices = (kt_n + tiles - 1) / tiles;
  p.accum_words = p.slices > 1 ? 8 + units * p.slices * kXmKSplit * kXmTok * 128 : 0;   // 8 control words in front
  return p;
}

// How often the last slice of a group looks at a word that has not arrived before it gives the row up (NaN).
// A host-side setting so that the give-up path can be exercised without any kernel misbehaving.
static std::atomic<int> g_exl3_poll_limit{1 << 16};
int exl3_set_poll_limit(int limit) { return g_exl3_poll_limit.exchange(limit < 0 ? 0 : limit); }

template <int BITS, int CB, typename XT>
static hipError_t xm_launch(const Exl3Plan& p, const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                            const void* x, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                            int64_t n_out, int64_t n_in, unsigned long long* accum, hipStream_t s) {
  const dim3 grid((unsigned)p.groups, (unsigned)p.slices, (unsigned)p.row_groups), block(kXmThreads);
  hipLaunchKernelGGL((gemv_exl3_mfma_kernel<BITS, CB, XT>), grid, block, 0, s, trellis, suh, svh,
                     static_cast<const XT*>(x), y, y_dtype, bias, bias_dtype, (int)m, (int)n_out, (int)n_in, p.slice_tiles,
                     accum, g_exl3_poll_limit.load(std::memory_order_relaxed));
  return hipGetLastError();
}

template <int BITS, int CB>
static hipError_t xm_launch_x(const Exl3Plan& p, const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                              const void* x, int x_dtype, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                              int64_t n_out, int64_t n_in, unsigned long long* accum, hipStream_t s) {
  switch (x_dtype) {
    case kF32: return xm_launch<BITS, CB, float>(p, trellis, suh, svh, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, accum, s);
    case kF16: return xm_launch<BITS, CB, f16_tag>(p, trellis, suh, svh, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, accum, s);
    case kBF16: return xm_launch<BITS, CB, bf16_tag>(p, trellis, suh, svh, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, accum, s);
    default: return hipErrorInvalidValue;
  }
}

template <int BITS>
static hipError_t xm_launch_cb(const Exl3Plan& p, const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                               const void* x, int x_dtype, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                               int64_t n_out, int64_t n_in, int cb, unsigned long long* accum, hipStream_t s) {
  return cb == 0 ? xm_launch_x<BITS, 0>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, accum, s)
                 : xm_launch_x<BITS, 1>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, accum, s);
}

hipError_t launch_gemv_exl3_mfma(const Exl3Plan& p, const uint16_t* trellis, const uint16_t* suh,
                                 const uint16_t* svh, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int bits, int cb,
                                 unsigned long long* accum, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (p.slices > 1 && !accum) return hipErrorInvalidValue;
  switch (bits) {
    case 1: return xm_launch_cb<1>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 2: return xm_launch_cb<2>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 3: return xm_launch_cb<3>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 4: return xm_launch_cb<4>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 5: return xm_launch_cb<5>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 6: return xm_launch_cb<6>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 7: return xm_launch_cb<7>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    case 8: return xm_launch_cb<8>(p, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, cb, accum, s);
    default: return hipErrorInvalidValue;
  }
}

// ------------------------------------------------------------------------------ workspace
// Sliced launches exchange their sums through tagged 64-bit words behind eight control words (generation count,
// groups finished), all zero before the first launch.  A caller-owned workspace (ttq_workspace.hip) supplies them
// when one is bound; otherwise the library keeps one array per (device, stream): launches on one stream run in
// order and can share it, launches on different streams may overlap and get their own.  Sized for the largest
// plan: launches are sliced only while there are fewer (group, row group) units than compute units.
namespace {
std::mutex g_ws_mutex;
std::unordered_map<uint64_t, unsigned long long*> g_ws;
}  // namespace

// units * slices <= compute units
int64_t exl3_workspace_words() { return 8 + (int64_t)device_num_cus() * kXmKSplit * kXmTok * 128; }

hipError_t exl3_workspace(hipStream_t s, unsigned long long** accum) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  void* bound = nullptr;
  if (caller_workspace_region(kCwExl3Words, (size_t)exl3_workspace_words() * sizeof(unsigned long long), &bound, &e)) {
    *accum = static_cast<unsigned long long*>(bound);
    return e;
  }
  const uint64_t key = ((uint64_t)(uint32_t)dev << 48) ^ (uint64_t)reinterpret_cast<uintptr_t>(s);
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_ws.find(key);
  if (it == g_ws.end()) {
    const size_t bytes = (size_t)exl3_workspace_words() * sizeof(unsigned long long);
    void* p = nullptr;
    e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return e;
    e = hipMemsetAsync(p, 0, bytes, s);     // ordered before the launches that use it: they are all on this stream
    if (e != hipSuccess) {
      (void)hipFree(p);
      return e;
    }
    it = g_ws.emplace(key, static_cast<unsigned long long*>(p)).first;
  }
  *accum = it->second;
  return hipSuccess;
}

// ------------------------------------------------------------------------------ resident workspace
// The same words as a file-scope array in device memory, for the entry point that must not allocate:
// every GPU the library runs on holds its own copy from the moment the code object is loaded there
// until the process ends, zero-initialised; the launches only ever advance its generation count.
// The array's name is only a handle in host code; the address on a device comes from
// hipGetSymbolAddress, asked once per device with that device current.
constexpr int64_t kXmResidentWords = 8 + (int64_t)256 * kXmKSplit * kXmTok * 128;      // 4 MiB
static __device__ __align__(256) unsigned long long scratch[kXmResidentWords];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_resident_mutex;
unsigned long long* g_resident[kMaxDevices] = {};
}  // namespace

int64_t exl3_resident_words() { return kXmResidentWords; }

hipError_t exl3_resident_workspace(unsigned long long** accum) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_resident_mutex);
  if (!g_resident[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_resident[dev] = static_cast<unsigned long long*>(p);
  }
  *accum = g_resident[dev];
  return hipSuccess;
}

// Frees the library-owned arrays (ttq_release_workspaces: nothing that uses them may be in flight or captured).
hipError_t exl3_release_workspaces() {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  hipError_t first = hipSuccess;
  for (auto& kv : g_ws) {
    const hipError_t e = hipFree(kv.second);
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  g_ws.clear();
  return first;
}

}  // namespace ttq
