// Decode GEMV for Q4_K weights on gfx950: the weight stream goes HBM -> LDS as whole cache lines.
//
// Same operator and arithmetic as ttq_gemv_mfma.hip (F.linear with a single-token activation,
// workspace/libtorch/src/abi/neural_nets.nim:64-81; 15-bit block fixed point activations in two
// byte planes, v_mfma_i32_16x16x64_i8, fp32 scales in the canonical order).  What differs is how
// the packed weights reach the matrix cores.
//
// The MFMA wants, per lane, 16 bytes of one of 16 weight rows; requested like that every load
// instruction touches half a cache line of 16 different rows, the other half belongs to another
// instruction, and the stream runs at 4 TB/s.  A kernel that reads whole lines, eight lines per
// instruction, with the non-temporal hint, goes through the same bytes at 5.4 TB/s.  So here the
// requests and the operands are decoupled through LDS:
//   * a wavefront owns blocks of 16 rows x 8 super-blocks (1152 bytes = 9 whole lines per row,
//     18 KiB) and a private LDS buffer of that size;
//   * it requests a block with 18 global_load_lds_dwordx4 (no registers): request 2 l + o is line
//     l of the eight rows 8 o .. 8 o + 7.  Six go out at once, two more before every super-block:
//     a compute unit takes about 48 KiB of outstanding requests, and a wavefront that asks for
//     more waits inside the instruction instead of computing;
//   * the 16-byte chunks are XOR-swizzled inside their line on the way in (by choosing which
//     global chunk a lane fetches), so that the operand reads -- 16 rows, same position -- hit 16
//     different bank groups;
//   * requests complete in order, so super-block s (bytes 144 s .. 144 s + 143 of the rows,
//     lines s and s + 1) is ready once all but the youngest few have landed: the wavefront waits
//     on its own counter only, nine LDS reads and four MFMAs per super-block, and no barrier
//     until the row sums of the two halves of K meet.
#pragma once

#include <type_traits>

#include "ttq_gemv_mfma_common.h"

namespace ttq {

constexpr int kStWaves = 8;
constexpr int kStThreads = kStWaves * 64;
constexpr int kStBlockSb = 8;                             // super-blocks of a row per block
constexpr int kStSegBytes = kStBlockSb * 144;             // 1152: a row's share of a block
constexpr int kStLines = kStSegBytes / 128;               // 9
constexpr int kStHalfBytes = 8 * kStSegBytes;             // eight rows: [line 9][row 8][slot 8] x 16 bytes
constexpr int kStBlockBytes = 2 * kStHalfBytes;           // 18432
constexpr int kStBlockRequests = 2 * kStLines;            // 18
constexpr int kStUpFront = 6;                             // requests before the first super-block (even)
// With one or two blocks per workgroup only one or two wavefronts carry the whole stream, and six requests in
// flight each would leave it latency-bound: those launches ask for 16 of a block's 18 at once (the last
// request's slot holds the activations until they have been read back).  4096x4096: 4.53 -> 4.28 us.  Sharing
// the landed super-blocks among all 8 wavefronts after a wait-for-all and a barrier was measured too: slower
// (4.54 us; 6144x4096 4.77 -> 6.03 us), the pipelined consumption by the owners wins.
constexpr int kStUpFrontFew = 16;
// With at most two blocks per workgroup (one row group of rows of 2048 or 4096 values: the attention output
// projection 4096x4096) four wavefronts share a block instead: wavefront 4 b + p takes super-blocks 2 p and 2 p + 1 of
// block b.  The block lands in one buffer (that of wavefront 4 b), every line requested once: wavefront p asks for
// lines 2 p + 1 and 2 p + 2 of both row halves (p = 0 also for line 0), multiplies super-block 2 p + 1, which lies in
// its own lines, as soon as they have landed, and super-block 2 p, which begins in its neighbour's last line, after
// a barrier that every wavefront reaches with its own lines landed.  After a stream of little more than a
// microsecond eight wavefronts multiply two super-blocks each instead of two multiplying eight.  The raw activations
// land in the buffer of wavefront 1, which holds no block in this form.  (kStQuad as the UP argument.)
constexpr int kStQuad = -1;
constexpr int kStMaxSb = 16;                              // n_in <= 4096: one staging pass, 8 KiB table
constexpr int kStMaxBlocks = 80;                          // blocks of a workgroup (their row sums wait in LDS)

typedef const __attribute__((address_space(1))) void* st_gptr_t;
typedef __attribute__((address_space(3))) void* st_lptr_t;
typedef uint32_t st_u32x4 __attribute__((ext_vector_type(4)));

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void st_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}

// Barrier that does not drain the outstanding global_load_lds requests (a __syncthreads() would).
__device__ __forceinline__ void st_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A 16-byte LDS read the compiler does not see as one: it cannot tell it from the asynchronous
// writes of the requests still in flight and would wait for all of those first.
__device__ __forceinline__ st_u32x4 st_read1(uint32_t a) {
  st_u32x4 v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(a) : "memory");
  return v;
}

// XT: bf16 or fp16 activations.  STAGE 0 is the GEMV; STAGE 1 leaves out the arithmetic (requests,
// waits, LDS reads and the activation prologue stay) and exists for the roofline ladder of bench.py.
// FUSE: the weight holds gate rows [0, n_out) followed by up rows [n_out, 2 n_out), as GatedMLP builds it
// (workspace/transformers/src/layers/mlp.nim:39), and the kernel writes silu(gate . x) * (up . x), the
// silu_and_mul of workspace/transformers/src/kernels/activations.nim:14-38: a workgroup takes the gate row
// groups of its outputs, then the up row groups of the same outputs, and pairs their sums at the end.
// n_out and rows_per_wg count outputs.
// NORM: every workgroup first normalizes the activation row itself: t = x + residual rounded to the activation
// type, normalized = t * rsqrt(mean(t^2) + eps) * gamma in fp32, rounded once to the activation type; the GEMV
// consumes exactly those rounded values, and workgroup 0 writes t and the normalized row out.  Residual and
// gamma arrive like the activations, as LDS requests into the slots of the block's last requests.
template <typename XT, typename YT, int STAGE, bool FUSE = false, int UP = kStUpFront, bool NORM = false>
__global__ void __launch_bounds__(kStThreads)
gemv_q4k_stream_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                       const void* __restrict__ bias, int bias_dtype, int n_out, int nsb, int rows_per_wg,
                       GemvNormArgs na) {
  static_assert(!NORM || UP + 3 <= kStBlockRequests, "three slots stay free for x, residual and gamma");
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kStWaves * kStBlockBytes];
  __shared__ __attribute__((aligned(16))) v4i_t xa[kStMaxSb * 32 + 1];   // plane table + one zero entry
  __shared__ __attribute__((aligned(16))) float tab[kStMaxSb * 32];
  __shared__ float part[kStMaxBlocks][16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nsb * 256;
  const int nks_log2 = nsb >> 4;                          // nsb is 8 or 16: one or two blocks per row group
  const uint16_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const uint32_t rb = (uint32_t)nsb * 144u;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int last = wg_row_end - 1;
  const int ngroups = (wg_row_end - wg_row0 + 15) >> 4;                  // row groups of 16 outputs
  const int nblocks = ((FUSE ? 2 : 1) * ngroups) << nks_log2;            // <= kStMaxBlocks (the launcher sees to it)
  uint8_t* mybuf = wbuf + wave * kStBlockBytes;

  // ---- activations first, also as an LDS request (a register load among the weight requests
  // would make the compiler wait for every one of them at its first use): thread t stages
  // x[8 t .. 8 t + 7].  It is the oldest request of its wavefront and lands where the block's last
  // request will: that one is made long after the activations have been read back.
  const int k0 = 8 * tid;
  const bool xok = k0 < n_in;                             // whole wavefronts: n_in is a multiple of 512
  constexpr bool kQuad = UP == kStQuad;
  static_assert(!kQuad || (!FUSE && !NORM), "four wavefronts per block: the plain form only");
  uint8_t* xland = kQuad ? wbuf + kStBlockBytes + wave * 1024 : mybuf + kStHalfBytes + (kStLines - 1) * 1024;
  if (xok) __builtin_amdgcn_global_load_lds((st_gptr_t)(xm + k0), (st_lptr_t)xland, 16, 0, 0);
  uint8_t* rland = mybuf + (kStLines - 1) * 1024;                      // request 16's slot
  uint8_t* gland = mybuf + kStHalfBytes + (kStLines - 2) * 1024;       // request 15's slot
  if constexpr (NORM) {
    if (xok) {
      if (na.residual != nullptr)
        __builtin_amdgcn_global_load_lds((st_gptr_t)(na.residual + (int64_t)blockIdx.y * n_in + k0), (st_lptr_t)rland, 16, 0, 0);
      __builtin_amdgcn_global_load_lds((st_gptr_t)(na.gamma + k0), (st_lptr_t)gland, 16, 0, 0);
    }
  }
  // a compute unit serves its requests in the order they were made: every wavefront's activation
  // request is queued before any weight request of the workgroup
  asm volatile("s_barrier" ::: "memory");

  // ---- requests of a block.  Lane l fetches, of line `line` of row 8 o + l / 8, the chunk
  // (l % 8) ^ key(row), key = (row / 2) % 8 with row counted inside the block: rows one apart sit in
  // different halves of the 256-byte bank period, rows of the same parity differ in key.
  uint32_t lane_off[2];
  auto set_block = [&](int blk) {
    const int rg = blk >> nks_log2, ks = blk & ((1 << nks_log2) - 1);
    const int r8 = lane >> 3;
#pragma unroll
    for (int o = 0; o < 2; o++) {
      const int row16 = 8 * o + r8;
      // past the end: the last row again, never used
      int row;
      if (FUSE) {
        const int up = rg >= ngroups ? 1 : 0;
        row = up * n_out + min(wg_row0 + (rg - up * ngroups) * 16 + row16, last);
      } else {
        row = min(wg_row0 + rg * 16 + row16, last);
      }
      lane_off[o] = (uint32_t)row * rb + (uint32_t)(ks * kStSegBytes) + (uint32_t)(((lane & 7) ^ ((row16 >> 1) & 7)) * 16);
    }
  };
  uint8_t* blockbuf = kQuad ? wbuf + (wave >> 2) * (4 * kStBlockBytes) : mybuf;
  auto request = [&](int i) {
    const int line = i >> 1, o = i & 1;
    // non-temporal: every line is used once
    __builtin_amdgcn_global_load_lds((st_gptr_t)(w + (size_t)(lane_off[o] + (uint32_t)(line * 128))),
                                     (st_lptr_t)(blockbuf + o * kStHalfBytes + line * 1024), 16, 0, 2);
  };
  int blk = kQuad ? wave >> 2 : wave;
  const int quad_p = wave & 3;                            // (kQuad) which quarter of the block
  const bool have_block = blk < nblocks;
  if (have_block) {
    set_block(blk);
    if constexpr (kQuad) {
      if (quad_p == 0) {
        request(0);
        request(1);
      }
#pragma unroll
      for (int i = 2; i < 6; i++) request(4 * quad_p + i);
    } else {
#pragma unroll
      for (int i = 0; i < UP; i++) request(i);
    }
  }

  // ---- the raw activations back into registers
  float xf[8];
  if (xok) {
    if (!have_block) st_wait_vmcnt<0>();
    else if (kQuad && quad_p == 0) st_wait_vmcnt<6>();
    else st_wait_vmcnt<(kQuad ? 4 : UP)>();
    const st_u32x4 r = st_read1((uint32_t)(size_t)(st_lptr_t)(xland) + (uint32_t)(lane * 16));
    widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), xf);
  }
  if constexpr (NORM) {
    float ss = 0.f, gf[8];
    if (xok) {
      if (na.residual != nullptr) {
        const st_u32x4 rr = st_read1((uint32_t)(size_t)(st_lptr_t)(rland) + (uint32_t)(lane * 16));
        float rf[8];
        widen8<XT>(make_uint4(rr[0], rr[1], rr[2], rr[3]), rf);
#pragma unroll
        for (int i = 0; i < 8; i++) xf[i] += rf[i];
        const uint4 t = narrow8<XT>(xf);          // the new residual, as the reference's add rounds it
        if (blockIdx.x == 0 && na.new_residual != nullptr)
          *reinterpret_cast<uint4*>(na.new_residual + (int64_t)blockIdx.y * n_in + k0) = t;
      }
      const st_u32x4 gr = st_read1((uint32_t)(size_t)(st_lptr_t)(gland) + (uint32_t)(lane * 16));
      widen8<XT>(make_uint4(gr[0], gr[1], gr[2], gr[3]), gf);
#pragma unroll
      for (int i = 0; i < 8; i++) ss += xf[i] * xf[i];
    }
    ss = wave_sum(ss);
    if (lane == 0) part[0][wave] = ss;
    st_barrier();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < kStWaves; i++) total += part[0][i];
    const float rs = 1.f / sqrtf(total / (float)n_in + na.eps);
    if (xok) {
#pragma unroll
      for (int i = 0; i < 8; i++) xf[i] = (xf[i] * rs) * gf[i];
      const uint4 t = narrow8<XT>(xf);
      if (blockIdx.x == 0 && na.normed != nullptr)
        *reinterpret_cast<uint4*>(na.normed + (int64_t)blockIdx.y * n_in + k0) = t;
    }
  }

  // ---- quantize the activations into the two byte planes (compact table: entry (b, j, t, h) =
  // plane t of x[256 b + 32 j + 16 h ..], 16 bytes)
  if (tid < 4) reinterpret_cast<uint32_t*>(&xa[nsb * 32])[tid] = 0u;
  if (xok) {
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
    const uint32_t ec = eb < 18u ? 18u : eb;              // 2^(E-13) / 16 stays a normal number
    const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
    // non-finite activations poison the sub-block instead of being clipped
    const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
    int hi[8], lo[8], vsum = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int v = (int)rintf(xf[i] * mul);
      hi[i] = (v + 128) >> 8;
      lo[i] = v;                     // only the low byte is used
      vsum += v;
    }
    vsum += __builtin_amdgcn_update_dpp(vsum, vsum, 0xB1, 0xF, 0xF, false);
    vsum += __builtin_amdgcn_update_dpp(vsum, vsum, 0x4E, 0xF, 0xF, false);
    const int b = k0 >> 8, j = (k0 >> 5) & 7, h = (k0 >> 4) & 1, half8 = (k0 >> 3) & 1;
    const int e_hi = (b * 32 + 4 * j + h) * 2 + half8;
    uint2* xa8 = reinterpret_cast<uint2*>(&xa[0]);
    xa8[e_hi] = make_uint2(pack_low_bytes(hi[0], hi[1], hi[2], hi[3]), pack_low_bytes(hi[4], hi[5], hi[6], hi[7]));
    xa8[e_hi + 4] = make_uint2(pack_low_bytes(lo[0], lo[1], lo[2], lo[3]), pack_low_bytes(lo[4], lo[5], lo[6], lo[7]));
    // per (super-block, pair of sub-blocks 2g, 2g+1): {2^(E-13) of 2g, 2^(E-13) / 16 of 2g+1, sum(x) of
    // both, 128 * sum(v) of 2g+1}: the odd sub-block's nibbles reach the MFMA as 16 * (q - 8)
    if ((tid & 3) == 0) {
      float* e = tab + (b * 4 + (j >> 1)) * 8;
      e[j & 1] = (j & 1) ? f * 0.0625f : f;
      e[2 + (j & 1)] = sum;
      if (j & 1) reinterpret_cast<int*>(e)[4] = 128 * vsum;
    }
  }

  // ---- per-lane constants of the main loop
  // Scales and mins of the lane's two sub-blocks (2g, 2g+1) as bytes 0 and 1 of a dword:
  //   sub-blocks 0-3: (bytes 0-3 | 4-7 of the field) & 63;  sub-blocks 4-7: low | high nibble of bytes
  //   8-11, with bits 6-7 of bytes 0-3 | 4-7 on top.  One expression with per-lane masks.
  const bool upper = g >= 2;
  const uint32_t m_lo = upper ? 0x0F0F0F0Fu : 0x3F3F3F3Fu, m_top = upper ? 0x30303030u : 0u;
  const uint32_t pair_shift = 16u * (uint32_t)(g & 1);
  constexpr uint32_t N4 = 0x0F0F0F0Fu;
  // A-operand table addresses (compact layout of ttq_gemv_mfma.hip): a lane has at most one
  // non-zero MFMA out of the four; the others read the zero entry with stride 0.  The block's
  // half of K (ks) is added per block.
  const uint32_t xa_base = (uint32_t)(size_t)(st_lptr_t)(&xa[0]);
  uint32_t a_addr0[4], a_step[4];
  {
    const int mrow = lane & 15, ga = lane >> 4, j = mrow >> 1;
    const bool valid = (ga >> 1) == ((j & 3) >> 1);
    const int qstar = 2 * (j >> 2) + (j & 1);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const bool mine = valid && q == qstar;
      a_addr0[q] = xa_base + 16u * (mine ? (uint32_t)(mrow * 2 + (ga & 1)) : (uint32_t)nsb * 32u);
      a_step[q] = mine ? 512u : 0u;
    }
  }
  const uint32_t tab_addr0 = (uint32_t)(size_t)(st_lptr_t)(&tab[0]) + (uint32_t)(g * 32);
  // operand reads: row n of the block, chunk 9 s + c of its 72, c = 0 (header), 1 + g, 5 + g:
  // line s + (s + c) / 8, slot ((s + c) % 8) ^ key
  const uint32_t key = (uint32_t)(n >> 1) & 7u;
  const uint32_t rowbase = (uint32_t)(size_t)(st_lptr_t)(blockbuf) + (uint32_t)((n >> 3) * kStHalfBytes + (n & 7) * 128);

  st_barrier();                         // the plane table is complete

  // Everything a super-block needs from LDS, read by one asm statement (the compiler would put a
  // wait for every outstanding weight request in front of a read it can see) and waited for by
  // another, one super-block later: lgkmcnt counts the nine reads issued in between.
  struct Regs { st_u32x4 hdr, c0, c1, a0, a1, a2, a3, cst; uint32_t kodd; };
  uint32_t a_addr[4], tab_addr = tab_addr0;
  auto topup = [&](auto sc) {
    constexpr int s = decltype(sc)::value;
    if constexpr (!kQuad && UP + 2 * s < kStBlockRequests) {
      request(UP + 2 * s);
      request(UP + 2 * s + 1);
    }
  };
  auto issue = [&](auto sc, Regs& r) {
    constexpr int s = decltype(sc)::value;
    // super-block s needs requests 0 .. 2 s + 3 (its two top-up requests have been made by now)
    if constexpr (kQuad) {
      // (the caller has waited: its own lines have landed, and after the barrier everybody's)
    } else {
      constexpr int kIssued = UP + 2 * (s + 1) < kStBlockRequests ? UP + 2 * (s + 1) : kStBlockRequests;
      st_wait_vmcnt<kIssued - (2 * s + 4)>();
    }
    const uint32_t ta = tab_addr;
    // (s + c) ^ key, c = 1 + g or 5 + g: bits 0-2 are the slot, bit 3 says "next line"
    const uint32_t e0 = ((1u + (uint32_t)g + (uint32_t)s) ^ key), e1 = ((5u + (uint32_t)g + (uint32_t)s) ^ key);
    const uint32_t a_h = rowbase + ((key ^ (uint32_t)s) << 4);
    const uint32_t a_0 = rowbase + ((e0 & 8u) << 7) + ((e0 & 7u) << 4);
    const uint32_t a_1 = rowbase + ((e1 & 8u) << 7) + ((e1 & 7u) << 4);
    const uint32_t x0 = a_addr[0] + (uint32_t)s * a_step[0], x1 = a_addr[1] + (uint32_t)s * a_step[1];
    const uint32_t x2 = a_addr[2] + (uint32_t)s * a_step[2], x3 = a_addr[3] + (uint32_t)s * a_step[3];
    asm volatile(
        "ds_read_b128 %0, %9 offset:%16\n\t"
        "ds_read_b128 %1, %10 offset:%16\n\t"
        "ds_read_b128 %2, %11 offset:%16\n\t"
        "ds_read_b128 %3, %12\n\t"
        "ds_read_b128 %4, %13\n\t"
        "ds_read_b128 %5, %14\n\t"
        "ds_read_b128 %6, %15\n\t"
        "ds_read_b128 %7, %17 offset:%18\n\t"
        "ds_read_b32 %8, %17 offset:%19"
        : "=&v"(r.hdr), "=&v"(r.c0), "=&v"(r.c1), "=&v"(r.a0), "=&v"(r.a1), "=&v"(r.a2), "=&v"(r.a3), "=&v"(r.cst),
          "=&v"(r.kodd)
        : "v"(a_h), "v"(a_0), "v"(a_1), "v"(x0), "v"(x1), "v"(x2), "v"(x3), "n"(s * 1024), "v"(ta),
          "n"(s * 128), "n"(s * 128 + 16)
        : "memory");
  };
  auto settle = [&](auto pending, Regs& r) {
    constexpr int P = decltype(pending)::value;
    asm volatile("s_waitcnt lgkmcnt(%9)"
                 : "+v"(r.hdr), "+v"(r.c0), "+v"(r.c1), "+v"(r.a0), "+v"(r.a1), "+v"(r.a2), "+v"(r.a3), "+v"(r.cst),
                   "+v"(r.kodd)
                 : "n"(P)
                 : "memory");
  };
  float acc = 0.f;
  auto compute = [&](const Regs& r) {
    if constexpr (STAGE != 0) return;
    v4i_t L0, H0, L1, H1, a0, a1, a2, a3;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // low nibbles as they are; high nibbles as the signed bytes 16 * (q - 8)
      L0[i] = (int)(r.c0[i] & N4); H0[i] = (int)((r.c0[i] & 0xF0F0F0F0u) ^ 0x80808080u);
      L1[i] = (int)(r.c1[i] & N4); H1[i] = (int)((r.c1[i] & 0xF0F0F0F0u) ^ 0x80808080u);
      a0[i] = (int)r.a0[i]; a1[i] = (int)r.a1[i]; a2[i] = (int)r.a2[i]; a3[i] = (int)r.a3[i];
    }
    // two independent chains; their non-zero rows are disjoint (sub-blocks 0-3 and 4-7)
    const v4i_t zero = {0, 0, 0, 0};
    v4i_t Ca = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, L0, zero, 0, 0, 0);
    v4i_t Cb = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, L1, zero, 0, 0, 0);
    Ca = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, H0, Ca, 0, 0, 0);
    Cb = __builtin_amdgcn_mfma_i32_16x16x64_i8(a3, H1, Cb, 0, 0, 0);
    const v4i_t C = Ca + Cb;
    const float d = f16_bits_to_f32((uint16_t)(r.hdr[0] & 0xFFFFu));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr[0] >> 16));
    const uint32_t xs = upper ? r.hdr[3] : r.hdr[1];
    const uint32_t xm4 = upper ? (r.hdr[3] >> 4) : r.hdr[2];
    const uint32_t sc4 = ((xs & m_lo) | ((r.hdr[1] >> 2) & m_top)) >> pair_shift;
    const uint32_t mn4 = ((xm4 & m_lo) | ((r.hdr[2] >> 2) & m_top)) >> pair_shift;
    const float sc1 = (float)(sc4 & 0xFFu), sc2 = (float)((sc4 >> 8) & 0xFFu);
    const float mn1 = (float)(mn4 & 0xFFu), mn2 = (float)((mn4 >> 8) & 0xFFu);
    // exact integers scaled by a power of two: sum(q * x) of the sub-block
    const float q1 = (float)(C[0] * 256 + C[1]) * __uint_as_float(r.cst[0]);
    const float q2 = (float)(C[2] * 256 + C[3] + (int)r.kodd) * __uint_as_float(r.cst[1]);
    // (d * sc) * q - (dmin * m) * sum(x): with a unit-vector activation each fused multiply-add
    // rounds exactly where the canonical dequantizer does
    acc = fmaf_(d * sc1, q1, acc);
    acc = fmaf_(-(dmin * mn1), __uint_as_float(r.cst[2]), acc);
    acc = fmaf_(d * sc2, q2, acc);
    acc = fmaf_(-(dmin * mn2), __uint_as_float(r.cst[3]), acc);
    // pins the arithmetic here: left alone the compiler moves it behind every wait of the block
    asm volatile("" : "+v"(acc));
  };

  // ---- four wavefronts per block: this one's two super-blocks
  if constexpr (kQuad) {
    if (have_block) {
      const int ks = blk & ((1 << nks_log2) - 1);
#pragma unroll
      for (int q = 0; q < 4; q++) a_addr[q] = a_addr0[q] + (uint32_t)ks * (kStBlockSb * a_step[q]);
      tab_addr = tab_addr0 + (uint32_t)(ks * kStBlockSb * 128);
      Regs ra, rb2;
      st_wait_vmcnt<0>();                  // this wavefront's lines
      auto two = [&](auto pc) {
        constexpr int p2 = 2 * decltype(pc)::value;
        issue(std::integral_constant<int, p2 + 1>{}, ra);
        st_barrier();                      // every wavefront's lines (and ra's reads)
        issue(std::integral_constant<int, p2>{}, rb2);
        settle(std::integral_constant<int, 9>{}, ra);
        compute(ra);
        settle(std::integral_constant<int, 0>{}, rb2);
        compute(rb2);
      };
      switch (quad_p) {
        case 0: two(std::integral_constant<int, 0>{}); break;
        case 1: two(std::integral_constant<int, 1>{}); break;
        case 2: two(std::integral_constant<int, 2>{}); break;
        default: two(std::integral_constant<int, 3>{}); break;
      }
      acc = add_xor16(acc);
      acc = add_xor32(acc);
      if (lane < 16) part[wave][lane] = acc;
    } else {
      st_barrier();
    }
    __syncthreads();
    // one row group: its (block, quarter) sums in order
    if (tid < 16) {
      float v = 0.f;
      for (int k = 0; k < 4 * nblocks; k++) v += part[k][tid];
      const int row = wg_row0 + tid;
      if (row < wg_row_end) YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
    }
    return;
  }

  // ---- the wavefront's blocks: wave, wave + 8, ...  A block starts with nothing outstanding.
  auto run_block = [&](const int blk) {
    const int ks = blk & ((1 << nks_log2) - 1);
#pragma unroll
    for (int q = 0; q < 4; q++) a_addr[q] = a_addr0[q] + (uint32_t)ks * (kStBlockSb * a_step[q]);
    tab_addr = tab_addr0 + (uint32_t)(ks * kStBlockSb * 128);
    acc = 0.f;
    Regs ra, rb2;
    using I0 = std::integral_constant<int, 0>;
    if constexpr (UP == kStUpFront) {
      // per super-block: its top-up requests, then the arithmetic of the one before (whose operands were read a step
      // ago), and only then the wait for its own bytes -- so that when the block's last bytes land, one super-block
      // of arithmetic is left, not two
      topup(std::integral_constant<int, 0>{}); issue(std::integral_constant<int, 0>{}, ra);
      topup(std::integral_constant<int, 1>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 1>{}, rb2);
      topup(std::integral_constant<int, 2>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 2>{}, ra);
      topup(std::integral_constant<int, 3>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 3>{}, rb2);
      topup(std::integral_constant<int, 4>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 4>{}, ra);
      topup(std::integral_constant<int, 5>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 5>{}, rb2);
      topup(std::integral_constant<int, 6>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 6>{}, ra);
      topup(std::integral_constant<int, 7>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 7>{}, rb2);
    } else {
      // few blocks per workgroup: the bytes arrive in one burst and the wavefronts that own them multiply eight
      // super-blocks back to back, so the operand reads of a super-block overlap the arithmetic of the one before
      using I9 = std::integral_constant<int, 9>;
      topup(std::integral_constant<int, 0>{}); issue(std::integral_constant<int, 0>{}, ra);
      topup(std::integral_constant<int, 1>{}); issue(std::integral_constant<int, 1>{}, rb2); settle(I9{}, ra); compute(ra);
      topup(std::integral_constant<int, 2>{}); issue(std::integral_constant<int, 2>{}, ra); settle(I9{}, rb2); compute(rb2);
      topup(std::integral_constant<int, 3>{}); issue(std::integral_constant<int, 3>{}, rb2); settle(I9{}, ra); compute(ra);
      topup(std::integral_constant<int, 4>{}); issue(std::integral_constant<int, 4>{}, ra); settle(I9{}, rb2); compute(rb2);
      topup(std::integral_constant<int, 5>{}); issue(std::integral_constant<int, 5>{}, rb2); settle(I9{}, ra); compute(ra);
      topup(std::integral_constant<int, 6>{}); issue(std::integral_constant<int, 6>{}, ra); settle(I9{}, rb2); compute(rb2);
      topup(std::integral_constant<int, 7>{}); issue(std::integral_constant<int, 7>{}, rb2); settle(I9{}, ra); compute(ra);
    }
    settle(I0{}, rb2);
    // every request of the block has landed and been read: the next block may use the buffer
    const int next = blk + kStWaves;
    if (next < nblocks) {
      set_block(next);
#pragma unroll
      for (int i = 0; i < UP; i++) request(i);
    }
    compute(rb2);
    // the four k-groups of a row
    acc = add_xor16(acc);
    acc = add_xor32(acc);
    if (lane < 16) part[blk][lane] = acc;
  };
  // (the first block apart from the loop: the compiler schedules the straight-line copy better)
  if (blk < nblocks) {
    run_block(blk);
    blk += kStWaves;
  }
  for (; blk < nblocks; blk += kStWaves) run_block(blk);
  // every request has landed (plain loads and barriers are safe again); the blocks of a row group add up
  __syncthreads();
  for (int t = tid; t < ngroups * 16; t += kStThreads) {
    const int grp = t >> 4, nn = t & 15;
    float v = part[grp << nks_log2][nn];
    if (nks_log2) v += part[(grp << 1) + 1][nn];
    const int row = wg_row0 + t;
    if (FUSE) {
      float u = part[(ngroups + grp) << nks_log2][nn];
      if (nks_log2) u += part[((ngroups + grp) << 1) + 1][nn];
      if (row < wg_row_end) YElem<YT>::store_through(ym, row, (v / (1.f + expf(-v))) * u);
    } else {
      if (row < wg_row_end) YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
    }
  }
}

// Rows are dealt to the compute units in equal shares, as in the register-streamed kernel.
inline int st_rows_per_wg(int64_t n_out, int* num_wg_out) {
  int num_wg = device_num_cus();
  const int64_t groups = (n_out + 15) / 16;
  if (num_wg > groups) num_wg = (int)groups;
  const int rows_per_wg = (int)((n_out + num_wg - 1) / num_wg);
  if (num_wg_out) *num_wg_out = (int)((n_out + rows_per_wg - 1) / rows_per_wg);
  return rows_per_wg;
}

template <typename XT, typename YT, int STAGE, bool FUSE = false, bool NORM = false>
inline hipError_t st_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m,
                               int64_t n_out, int64_t n_in, hipStream_t s, GemvNormArgs na = GemvNormArgs{}) {
  int num_wg = 0;
  const int rows_per_wg = st_rows_per_wg(n_out, &num_wg);
  const dim3 grid((unsigned)num_wg, (unsigned)m), block(kStThreads);
  const int blocks = (FUSE ? 2 : 1) * ((rows_per_wg + 15) / 16) * (int)(n_in / 2048);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)(n_in / 256), rows_per_wg, na);
  };
  // (the normalizing form keeps three request slots free for x, residual and gamma)
  if constexpr (!FUSE && !NORM) {
    if (blocks <= 2 && rows_per_wg <= 16) {
      go(gemv_q4k_stream_kernel<XT, YT, STAGE, false, kStQuad, false>);
      return hipGetLastError();
    }
  }
  if (blocks <= 2 && !NORM) go(gemv_q4k_stream_kernel<XT, YT, STAGE, FUSE, NORM ? 12 : kStUpFrontFew, NORM>);
  else if (blocks <= 4) go(gemv_q4k_stream_kernel<XT, YT, STAGE, FUSE, 12, NORM>);
  else go(gemv_q4k_stream_kernel<XT, YT, STAGE, FUSE, kStUpFront, NORM>);
  return hipGetLastError();
}

}  // namespace ttq
