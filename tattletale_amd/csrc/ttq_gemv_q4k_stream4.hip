// Decode GEMV for Q4_K weights and two to four activation rows at once (speculative decoding, small batches):
// F.linear with a handful of tokens, workspace/libtorch/src/abi/neural_nets.nim:64-81.
//
// The single-row kernel of ttq_gemv_q4k_stream.h streams the packed weights HBM -> LDS as whole cache lines and
// multiplies them on the int8 matrix cores against an activation table whose 16 rows are (sub-block, byte plane)
// selectors: each of a super-block's four v_mfma_i32_16x16x64_i8 covers two sub-blocks, so only four of its 16
// rows carry data.  Here the other twelve carry three more tokens: row (token, sub-block of the pair, plane).
// Four tokens then cost the same four matrix instructions per super-block as one, the weights are streamed and
// unpacked once, and only the scale arithmetic behind the matrix cores is per token -- which falls to the lane
// group that owns the token: lane (n, g) of the accumulator holds, for weight row n and token g, the two
// sub-blocks' high- and low-plane sums.  It applies the sub-block scales of row n (all eight decoded by every
// lane), the token's block exponents and sums of x (five 16-byte LDS reads per super-block), and keeps the running
// sum of (row n, token g) in one register: no cross-lane reduction at all.
//
// What differs from the single-row kernel besides that: four plane tables (32 KiB) do not fit beside eight
// 18 KiB stream buffers, and fewer wavefronts than blocks leave a second, latency-bound round (8 blocks on 6
// wavefronts: +1.4 us).  A wavefront's buffer is therefore a ring of seven of a block's nine lines (14 KiB):
// line l lives in slot l % 7, lines 7 and 8 are requested into the slots of lines 0 and 1 once the first two
// super-blocks have been read (super-block s needs lines s and s + 1 only), and everything that selects a slot
// is still a compile-time constant per super-block.  The activations of all tokens arrive as four LDS requests
// per wavefront into slots the stream needs only later, and every wavefront quantizes what it fetched itself.
#include "ttq_gemv_q4k_stream.h"

namespace ttq {

namespace {

constexpr int kS4Waves = 8;
constexpr int kS4Threads = kS4Waves * 64;
constexpr int kS4Tok = 4;                      // activation rows per launch
constexpr int kS4Up = 6;                       // weight requests in flight per wavefront (48 KiB per compute unit)
constexpr int kS4UpFirst = 4;                  // of them, before the activations are quantized
constexpr int kS4RingLines = 7;                // of a block's 9 lines (16 rows x 128 bytes each: 2 KiB)
constexpr int kS4HalfBytes = kS4RingLines * 1024;          // eight rows: [slot 7][row 8][chunk 8] x 16 bytes
constexpr int kS4BufBytes = 2 * kS4HalfBytes;              // 14336
constexpr int kS4XPasses = 4;                  // activation requests per wavefront: 4 x 512 chunks of 8 values = 4 x 4096 / 8
constexpr int kS4XLine0 = 4;                   // they land in the slots of lines 4 and 5
constexpr int kS4MaxSb = 16;                   // n_in <= 4096
// Sums that wait in LDS for the end of the kernel: one per block of a workgroup, or -- when a workgroup has more
// blocks than this and rows of 4096 values -- one per row group: a wavefront then takes both blocks of a group,
// one after the other, and adds them in its accumulator.
constexpr int kS4MaxPart = 40;
constexpr int kS4CstDw = 20;                   // per (token, super-block): f[8], sum[8], kodd[4]
static_assert(kS4XPasses * kS4Threads * 8 >= kS4Tok * kS4MaxSb * 256, "every activation has a thread");
static_assert(kS4XLine0 + (kS4XPasses + 1) / 2 <= kS4RingLines, "the landing slots exist");
static_assert(2 * kS4XLine0 >= kS4Up + 2, "the landing slots are beyond the requests made before the tables are complete");
// the top-up of super-block s asks for line kS4Up / 2 + s, into the slot of line kS4Up / 2 + s - 7, whose last
// reader is the super-block of that number: its reads must have completed, i.e. it must be s - 2 or earlier
static_assert(kS4Up / 2 - kS4RingLines <= -2, "a top-up never overwrites a line that is still to be read");
constexpr int s4_slot(int line) { return line % kS4RingLines; }

// FUSE: the weight holds gate rows [0, n_out) followed by up rows [n_out, 2 n_out), as GatedMLP builds it
// (workspace/transformers/src/layers/mlp.nim:39), and the kernel writes silu(gate . x) * (up . x), the silu_and_mul
// of workspace/transformers/src/kernels/activations.nim:14-38: a workgroup takes the gate row groups of its
// outputs, then the up row groups of the same outputs, and pairs their sums at the end.  n_out and rows_per_wg
// count outputs.
template <typename XT, typename YT, bool FUSE>
__global__ void __launch_bounds__(kS4Threads)
gemv_q4k_stream4_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                        const void* __restrict__ bias, int bias_dtype, int m, int n_out, int nsb, int rows_per_wg) {
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kS4Waves * kS4BufBytes];
  __shared__ __attribute__((aligned(16))) v4i_t xa[kS4Tok * kS4MaxSb * 32 + 1];      // plane tables + one zero entry
  __shared__ __attribute__((aligned(16))) uint32_t cst[kS4Tok * kS4MaxSb * kS4CstDw];
  __shared__ float part[kS4MaxPart][64];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nsb * 256;
  const int nks_log2 = nsb >> 4;                          // nsb is 8 or 16: one or two blocks per row group
  const uint32_t rb = (uint32_t)nsb * 144u;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int last = wg_row_end - 1;
  const int ngroups = (wg_row_end - wg_row0 + 15) >> 4;
  const int nblocks = ((FUSE ? 2 : 1) * ngroups) << nks_log2;
  // (the launcher sees to it that the blocks, or else the row groups, number kS4MaxPart at most)
  const bool pair = nblocks > kS4MaxPart;
  uint8_t* mybuf = wbuf + wave * kS4BufBytes;
  const int zero_entry = kS4Tok * kS4MaxSb * 32;

  // ---- activations: chunk c = 8 values, c = token * (n_in / 8) + k / 8.  Pass p of thread tid is chunk
  // p * 512 + tid; a wavefront's pass is one LDS request (64 chunks = 1 KiB) into its own buffer -- the slots of
  // lines 4 and 5, both halves, which the stream asks for from the second super-block's top-up on, i.e. after
  // the tables are complete.  Chunks past the end re-read the last one: the request count stays fixed.
  const int chunks_per_tok = nsb * 32;
  const int total_chunks = m * chunks_per_tok;
  auto land = [&](int p) { return mybuf + (p & 1) * kS4HalfBytes + s4_slot(kS4XLine0 + (p >> 1)) * 1024; };
#pragma unroll
  for (int p = 0; p < kS4XPasses; p++) {
    const int c = min(p * kS4Threads + tid, total_chunks - 1);
    const int tok = c / chunks_per_tok, kc = c - tok * chunks_per_tok;
    __builtin_amdgcn_global_load_lds((st_gptr_t)(x + (int64_t)tok * n_in + kc * 8), (st_lptr_t)land(p), 16, 0, 0);
  }

  // ---- requests of a block: as in the single-row kernel
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
  auto request = [&](int i) {
    const int line = i >> 1, o = i & 1;
    __builtin_amdgcn_global_load_lds((st_gptr_t)(w + (size_t)(lane_off[o] + (uint32_t)(line * 128))),
                                     (st_lptr_t)(mybuf + o * kS4HalfBytes + s4_slot(line) * 1024), 16, 0, 2);
  };
  // the wavefront's blocks: wave, wave + 8, ..., or both blocks of row groups wave, wave + 8, ...
  const int blk0 = pair ? 2 * wave : wave;
  const bool have_block = blk0 < nblocks;
  if (have_block) {
    set_block(blk0);
#pragma unroll
    for (int i = 0; i < kS4UpFirst; i++) request(i);
    st_wait_vmcnt<kS4UpFirst>();
  } else {
    st_wait_vmcnt<0>();
  }

  // ---- quantize what this wavefront fetched: block fixed point per 32 values, two byte planes (entry
  // (token, b, j, t, h) = plane t of x[token][256 b + 32 j + 16 h ..], 16 bytes), and per (token, super-block)
  // the constants of the scale arithmetic: {2^(E-13) of the even, 2^(E-13) / 16 of the odd sub-blocks} (the odd
  // sub-blocks' nibbles reach the matrix cores as 16 * (q - 8)), {sum(x)}, {128 * sum(v) of the odd ones}
  if (tid < 4) reinterpret_cast<uint32_t*>(&xa[zero_entry])[tid] = 0u;
#pragma unroll
  for (int p = 0; p < kS4XPasses; p++) {
    const int c = p * kS4Threads + tid;
    if (c < total_chunks) {                     // whole quads: the chunk counts are multiples of four
      const int tok = c / chunks_per_tok, kc = c - tok * chunks_per_tok;
      const st_u32x4 r = st_read1((uint32_t)(size_t)(st_lptr_t)(land(p)) + (uint32_t)(lane * 16));
      float xf[8];
      widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), xf);
      uint32_t amax = amax_bits(xf);
      // the four threads of a sub-block are an aligned quad
      amax = umax(amax, dpp_quad_u32<0xB1>(amax));
      amax = umax(amax, dpp_quad_u32<0x4E>(amax));
      const uint32_t eb = amax >> 23;                       // biased exponent of max |x|; 255 for Inf and NaN
      const uint32_t ec = eb < 18u ? 18u : eb;              // 2^(E-13) / 16 stays a normal number
      const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
      // non-finite activations poison the sub-block instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
      // v = rint(x * 2^(13-E)) read off the low bits of x * 2^(13-E) + 1.5 * 2^23
      uint32_t vb[8], vacc = 0u;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        vb[i] = __float_as_uint(fmaf_(xf[i], mul, __uint_as_float(kRoundMagicBits)));
        vacc += vb[i];
      }
      int vsum = (int)(vacc - 8u * kRoundMagicBits);
      vsum += __builtin_amdgcn_update_dpp(vsum, vsum, 0xB1, 0xF, 0xF, false);
      vsum += __builtin_amdgcn_update_dpp(vsum, vsum, 0x4E, 0xF, 0xF, false);
      // sum(x) as the fixed-point values give it: a row sum is the dot product with the quantized activations
      const float sum = (float)vsum * f;
      const int k0 = kc * 8;
      const int b = k0 >> 8, j = (k0 >> 5) & 7, h = (k0 >> 4) & 1, half8 = (k0 >> 3) & 1;
      const int e_hi = ((tok * nsb + b) * 32 + 4 * j + h) * 2 + half8;
      uint2* xa8 = reinterpret_cast<uint2*>(&xa[0]);
      xa8[e_hi] = make_uint2(pack_bytes1(vb[0] + 128u, vb[1] + 128u, vb[2] + 128u, vb[3] + 128u),
                             pack_bytes1(vb[4] + 128u, vb[5] + 128u, vb[6] + 128u, vb[7] + 128u));
      xa8[e_hi + 4] = make_uint2(pack_low_bytes((int)vb[0], (int)vb[1], (int)vb[2], (int)vb[3]),
                                 pack_low_bytes((int)vb[4], (int)vb[5], (int)vb[6], (int)vb[7]));
      if ((tid & 3) == 0) {
        uint32_t* e = cst + (tok * nsb + b) * kS4CstDw;
        e[j] = __float_as_uint((j & 1) ? f * 0.0625f : f);
        e[8 + j] = __float_as_uint(sum);
        if (j & 1) e[16 + (j >> 1)] = (uint32_t)(128 * vsum);
      }
    }
  }
  if (have_block) {
#pragma unroll
    for (int i = kS4UpFirst; i < kS4Up; i++) request(i);
  }

  // ---- per-lane constants of the main loop
  // matrix instruction u covers sub-blocks ja = (u & 1) + 4 (u >> 1) (k chunks of lane groups 0, 1) and ja + 2
  // (lane groups 2, 3); A row = (token, which of the two, plane); a lane supplies the 16 bytes of its row at its
  // k chunk, which are zero unless the chunk belongs to the row's sub-block (and the token exists)
  const uint32_t xa_base = (uint32_t)(size_t)(st_lptr_t)(&xa[0]);
  uint32_t a_addr0[4], a_step;
  {
    const int mrow = lane & 15, ga = lane >> 4;
    const int tok = mrow >> 2, jj = (mrow >> 1) & 1, t = mrow & 1, h = ga & 1;
    const bool mine = (ga >> 1) == jj && tok < m;
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int j = (u & 1) + 4 * (u >> 1) + 2 * jj;
      a_addr0[u] = xa_base + 16u * (uint32_t)(mine ? tok * nsb * 32 + 4 * j + 2 * t + h : zero_entry);
    }
    a_step = mine ? 512u : 0u;
  }
  // the constants of token g
  const uint32_t cst_addr0 = (uint32_t)(size_t)(st_lptr_t)(&cst[0]) + (uint32_t)(g * nsb * kS4CstDw * 4);
  const uint32_t key = (uint32_t)(n >> 1) & 7u;
  const uint32_t rowbase = (uint32_t)(size_t)(st_lptr_t)(mybuf) + (uint32_t)((n >> 3) * kS4HalfBytes + (n & 7) * 128);
  constexpr uint32_t N4 = 0x0F0F0F0Fu;

  st_barrier();                         // the tables are complete

  struct Regs { st_u32x4 hdr, c0, c1, a0, a1, a2, a3, f0, f1, s0, s1, kd; };
  uint32_t a_addr[4], cst_addr = cst_addr0;
  auto topup = [&](auto upc, auto sc) {
    constexpr int UP = decltype(upc)::value, s = decltype(sc)::value;
    if constexpr (UP + 2 * s < kStBlockRequests) {
      request(UP + 2 * s);
      request(UP + 2 * s + 1);
    }
  };
  auto issue = [&](auto upc, auto sc, Regs& r) {
    constexpr int UP = decltype(upc)::value, s = decltype(sc)::value;
    // super-block s needs requests 0 .. 2 s + 3 (its two top-up requests have been made by now)
    constexpr int kIssued = UP + 2 * (s + 1) < kStBlockRequests ? UP + 2 * (s + 1) : kStBlockRequests;
    st_wait_vmcnt<kIssued - (2 * s + 4)>();
    // chunk 9 s + c of the row's 72 (c = 0: header, 1 + g, 5 + g): line s + (s + c) / 8, position ((s + c) % 8) ^ key.
    // Line s is in slot s % 7, the next line kNext bytes further on (back, where the ring wraps).
    constexpr int kNext = (s4_slot(s + 1) - s4_slot(s)) * 1024;
    const uint32_t e0 = ((1u + (uint32_t)g + (uint32_t)s) ^ key), e1 = ((5u + (uint32_t)g + (uint32_t)s) ^ key);
    const uint32_t a_h = rowbase + ((key ^ (uint32_t)s) << 4);
    const uint32_t a_0 = rowbase + ((e0 & 8u) ? (uint32_t)kNext : 0u) + ((e0 & 7u) << 4);
    const uint32_t a_1 = rowbase + ((e1 & 8u) ? (uint32_t)kNext : 0u) + ((e1 & 7u) << 4);
    const uint32_t x0 = a_addr[0] + (uint32_t)s * a_step, x1 = a_addr[1] + (uint32_t)s * a_step;
    const uint32_t x2 = a_addr[2] + (uint32_t)s * a_step, x3 = a_addr[3] + (uint32_t)s * a_step;
    const uint32_t ca = cst_addr;
    asm volatile(
        "ds_read_b128 %0, %12 offset:%19\n\t"
        "ds_read_b128 %1, %13 offset:%19\n\t"
        "ds_read_b128 %2, %14 offset:%19\n\t"
        "ds_read_b128 %3, %15\n\t"
        "ds_read_b128 %4, %16\n\t"
        "ds_read_b128 %5, %17\n\t"
        "ds_read_b128 %6, %18\n\t"
        "ds_read_b128 %7, %20 offset:%21\n\t"
        "ds_read_b128 %8, %20 offset:%22\n\t"
        "ds_read_b128 %9, %20 offset:%23\n\t"
        "ds_read_b128 %10, %20 offset:%24\n\t"
        "ds_read_b128 %11, %20 offset:%25"
        : "=&v"(r.hdr), "=&v"(r.c0), "=&v"(r.c1), "=&v"(r.a0), "=&v"(r.a1), "=&v"(r.a2), "=&v"(r.a3), "=&v"(r.f0),
          "=&v"(r.f1), "=&v"(r.s0), "=&v"(r.s1), "=&v"(r.kd)
        : "v"(a_h), "v"(a_0), "v"(a_1), "v"(x0), "v"(x1), "v"(x2), "v"(x3), "n"(s4_slot(s) * 1024), "v"(ca),
          "n"(s * kS4CstDw * 4), "n"(s * kS4CstDw * 4 + 16), "n"(s * kS4CstDw * 4 + 32), "n"(s * kS4CstDw * 4 + 48),
          "n"(s * kS4CstDw * 4 + 64)
        : "memory");
  };
  auto settle = [&](Regs& r) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(r.hdr), "+v"(r.c0), "+v"(r.c1), "+v"(r.a0), "+v"(r.a1), "+v"(r.a2), "+v"(r.a3), "+v"(r.f0),
                   "+v"(r.f1), "+v"(r.s0), "+v"(r.s1), "+v"(r.kd)
                 :
                 : "memory");
  };
  float acc = 0.f;
  auto compute = [&](const Regs& r) {
    v4i_t L0, H0, L1, H1, a0, a1, a2, a3;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // low nibbles as they are; high nibbles as the signed bytes 16 * (q - 8)
      L0[i] = (int)(r.c0[i] & N4); H0[i] = (int)((r.c0[i] & 0xF0F0F0F0u) ^ 0x80808080u);
      L1[i] = (int)(r.c1[i] & N4); H1[i] = (int)((r.c1[i] & 0xF0F0F0F0u) ^ 0x80808080u);
      a0[i] = (int)r.a0[i]; a1[i] = (int)r.a1[i]; a2[i] = (int)r.a2[i]; a3[i] = (int)r.a3[i];
    }
    const v4i_t zero = {0, 0, 0, 0};
    const v4i_t C0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, L0, zero, 0, 0, 0);   // sub-blocks 0, 2
    const v4i_t C1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, H0, zero, 0, 0, 0);   // 1, 3
    const v4i_t C2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, L1, zero, 0, 0, 0);   // 4, 6
    const v4i_t C3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a3, H1, zero, 0, 0, 0);   // 5, 7
    // the row's eight scales and mins (6 bits each): 0-3 in bytes 0-3 | 4-7 of the field, 4-7 as the low | high
    // nibbles of bytes 8-11 with bits 6-7 of bytes 0-3 | 4-7 on top
    const float d = f16_bits_to_f32((uint16_t)(r.hdr[0] & 0xFFFFu));
    const float dmin = f16_bits_to_f32((uint16_t)(r.hdr[0] >> 16));
    const uint32_t sc_lo = r.hdr[1] & 0x3F3F3F3Fu, mn_lo = r.hdr[2] & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (r.hdr[3] & N4) | ((r.hdr[1] >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((r.hdr[3] >> 4) & N4) | ((r.hdr[2] >> 2) & 0x30303030u);
    float dsc[8], ndm[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      dsc[j] = d * (float)((sc_lo >> (8 * j)) & 0xFFu);
      dsc[4 + j] = d * (float)((sc_hi >> (8 * j)) & 0xFFu);
      ndm[j] = -(dmin * (float)((mn_lo >> (8 * j)) & 0xFFu));
      ndm[4 + j] = -(dmin * (float)((mn_hi >> (8 * j)) & 0xFFu));
    }
    // lane (n, g): rows 4 g .. 4 g + 3 of each accumulator = token g: {first sub-block: high, low plane; second
    // sub-block: high, low plane}.  sum(q x) of a sub-block is an exact integer scaled by a power of two; then
    // (d * sc) * q - (dmin * m) * sum(x), each fused multiply-add rounding where the canonical dequantizer does
    auto tail = [&](const v4i_t& C, int ja, float fa, float fb, float sa, float sb, int ka, int kb) {
      const float qa = (float)(C[0] * 256 + C[1] + ka) * fa;
      const float qb = (float)(C[2] * 256 + C[3] + kb) * fb;
      acc = fmaf_(dsc[ja], qa, acc);
      acc = fmaf_(ndm[ja], sa, acc);
      acc = fmaf_(dsc[ja + 2], qb, acc);
      acc = fmaf_(ndm[ja + 2], sb, acc);
    };
    auto F = [](uint32_t v) { return __uint_as_float(v); };
    tail(C0, 0, F(r.f0[0]), F(r.f0[2]), F(r.s0[0]), F(r.s0[2]), 0, 0);
    tail(C1, 1, F(r.f0[1]), F(r.f0[3]), F(r.s0[1]), F(r.s0[3]), (int)r.kd[0], (int)r.kd[1]);
    tail(C2, 4, F(r.f1[0]), F(r.f1[2]), F(r.s1[0]), F(r.s1[2]), 0, 0);
    tail(C3, 5, F(r.f1[1]), F(r.f1[3]), F(r.s1[1]), F(r.s1[3]), (int)r.kd[2], (int)r.kd[3]);
    asm volatile("" : "+v"(acc));       // keeps the arithmetic between the waits it was written between
  };

  // ---- a block starts with UP requests outstanding.  next: the wavefront's block after it; reset: a new sum
  // starts here; store >= 0: the sum is complete and goes there
  auto run_block = [&](auto upc, const int b_, const int next, const bool reset, const int store) {
    constexpr int UP = decltype(upc)::value;
    using U = std::integral_constant<int, UP>;
    const int ks = b_ & ((1 << nks_log2) - 1);
#pragma unroll
    for (int u = 0; u < 4; u++) a_addr[u] = a_addr0[u] + (uint32_t)ks * (kStBlockSb * a_step);
    cst_addr = cst_addr0 + (uint32_t)(ks * kStBlockSb * kS4CstDw * 4);
    if (reset) acc = 0.f;
    Regs ra, rb2;
    topup(U{}, std::integral_constant<int, 0>{}); issue(U{}, std::integral_constant<int, 0>{}, ra);
    topup(U{}, std::integral_constant<int, 1>{}); settle(ra); compute(ra); issue(U{}, std::integral_constant<int, 1>{}, rb2);
    topup(U{}, std::integral_constant<int, 2>{}); settle(rb2); compute(rb2); issue(U{}, std::integral_constant<int, 2>{}, ra);
    topup(U{}, std::integral_constant<int, 3>{}); settle(ra); compute(ra); issue(U{}, std::integral_constant<int, 3>{}, rb2);
    topup(U{}, std::integral_constant<int, 4>{}); settle(rb2); compute(rb2); issue(U{}, std::integral_constant<int, 4>{}, ra);
    topup(U{}, std::integral_constant<int, 5>{}); settle(ra); compute(ra); issue(U{}, std::integral_constant<int, 5>{}, rb2);
    topup(U{}, std::integral_constant<int, 6>{}); settle(rb2); compute(rb2); issue(U{}, std::integral_constant<int, 6>{}, ra);
    topup(U{}, std::integral_constant<int, 7>{}); settle(ra); compute(ra); issue(U{}, std::integral_constant<int, 7>{}, rb2);
    settle(rb2);
    // every request of the block has landed and been read: the next block may use the buffer
    if (next < nblocks) {
      set_block(next);
#pragma unroll
      for (int i = 0; i < kS4Up; i++) request(i);
    }
    compute(rb2);
    if (store >= 0) part[store][lane] = acc;               // (row n, token g): nothing to reduce across lanes
  };
  for (int i = 0;; i++) {
    int b_, next, store;
    bool reset;
    if (pair) {
      const int rgi = wave + kS4Waves * (i >> 1), second = i & 1;
      b_ = 2 * rgi + second;
      next = second ? 2 * (rgi + kS4Waves) : b_ + 1;
      reset = !second;
      store = second ? rgi : -1;
    } else {
      b_ = wave + kS4Waves * i;
      next = b_ + kS4Waves;
      reset = true;
      store = b_;
    }
    if (b_ >= nblocks) break;
    run_block(std::integral_constant<int, kS4Up>{}, b_, next, reset, store);
  }

  // every request has landed; the blocks of a row group add up
  __syncthreads();
  const int wg_rows16 = ngroups * 16;
  for (int t = tid; t < wg_rows16 * m; t += kS4Threads) {
    const int tok = t / wg_rows16, r = t - tok * wg_rows16;
    const int grp = r >> 4, nn = r & 15;
    float v = part[pair ? grp : grp << nks_log2][tok * 16 + nn];
    if (nks_log2 && !pair) v += part[(grp << 1) + 1][tok * 16 + nn];
    const int row = wg_row0 + r;
    if (FUSE) {
      float u = part[pair ? ngroups + grp : (ngroups + grp) << nks_log2][tok * 16 + nn];
      if (nks_log2 && !pair) u += part[((ngroups + grp) << 1) + 1][tok * 16 + nn];
      if (row < wg_row_end) YElem<YT>::store(y, (int64_t)tok * n_out + row, (v / (1.f + expf(-v))) * u);
    } else {
      if (row < wg_row_end) YElem<YT>::store(y, (int64_t)tok * n_out + row, v + load_bias(bias, bias_dtype, row));
    }
  }
}

struct S4Plan { bool ok; int num_wg, rows_per_wg; };

// n_out counts outputs; a fused launch has twice as many weight rows and blocks
S4Plan s4_plan(int64_t m, int64_t n_out, int64_t n_in, bool fuse) {
  S4Plan p{};
  const int64_t parts = fuse ? 2 : 1;
  if (m < 2 || m > kS4Tok || (n_in != 4096 && n_in != 2048)) return p;
  if (parts * n_out < 16 * (int64_t)device_num_cus() || parts * n_out * (n_in / 256) * 144 >= ((int64_t)1 << 32)) return p;
  if (fuse && n_out % 8 != 0) return p;
  p.rows_per_wg = st_rows_per_wg(n_out, &p.num_wg);
  // the sums of a workgroup's blocks, or for rows of 4096 values else those of its row groups, fit LDS
  const int64_t groups = parts * ((p.rows_per_wg + 15) / 16);
  if (groups * (n_in / 2048) > kS4MaxPart && !(n_in == 4096 && groups <= kS4MaxPart)) return p;
  p.ok = true;
  return p;
}

template <typename XT, typename YT, bool FUSE>
hipError_t s4_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m,
                        int64_t n_out, int64_t n_in, hipStream_t s) {
  const S4Plan p = s4_plan(m, n_out, n_in, FUSE);
  if (!p.ok) return hipErrorInvalidValue;
  hipLaunchKernelGGL((gemv_q4k_stream4_kernel<XT, YT, FUSE>), dim3((unsigned)p.num_wg), dim3(kS4Threads), 0, s,
                     static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x), static_cast<YT*>(y), bias,
                     bias_dtype, (int)m, (int)n_out, (int)(n_in / 256), p.rows_per_wg);
  return hipGetLastError();
}

template <typename XT, bool FUSE>
hipError_t s4_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                       int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return s4_launch_xy<XT, float, FUSE>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return s4_launch_xy<XT, f16_tag, FUSE>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return s4_launch_xy<XT, bf16_tag, FUSE>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool gemv_q4k_stream4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in) {
  static const int disabled = dev_knob("TTQ_GEMV_NO_STREAM4", 0);
  if (disabled || format != kQ4_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  return s4_plan(m, n_out, n_in, false).ok;
}

hipError_t launch_gemv_q4k_stream4(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                   int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return s4_launch_x<bf16_tag, false>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return s4_launch_x<f16_tag, false>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

// The gate || up form: n_ff outputs from 2 n_ff weight rows, two to four activation rows.
bool gemv_q4k_stream4_fused_supported(int x_dtype, int64_t m, int64_t n_ff, int64_t n_in) {
  if (!(x_dtype == kBF16 || x_dtype == kF16)) return false;
  return s4_plan(m, n_ff, n_in, true).ok;
}

hipError_t launch_gemv_q4k_stream4_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                         int64_t n_ff, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return s4_launch_x<bf16_tag, true>(w, x, y, y_dtype, nullptr, 0, m, n_ff, n_in, s);
  if (x_dtype == kF16) return s4_launch_x<f16_tag, true>(w, x, y, y_dtype, nullptr, 0, m, n_ff, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
