// Decode GEMV for Q6_K weights and two or more activation rows at once (a few sequences, or the tokens a
// speculative step verifies) on gfx950: one pass over the weight stream of the single-row kernel
// (ttq_gemv_q6k_stream.h) serves two or four of them; more rows take more passes.
//
// Operator: F.linear with a (2.., n_in) activation (workspace/libtorch/src/abi/neural_nets.nim:64-81) over a weight
// of GGUF Q6_K blocks.
//
// The stream is the single-row kernel's: rounds of eight blocks of one group of 16 rows land in LDS buffers as 28
// requests of 1 KiB, every block moved to a 16-byte boundary and the rows rotated against each other; every
// wavefront multiplies one block of the round.  What changes is the activation operand.  The single-row kernel
// spends the 16 rows of a v_mfma_i32_16x16x64_i8 on (k-set, plane, sub-block) and adds the two k-sets of a unit into
// one accumulator.  Here a row is (token of a pair, plane, sub-block): each of a unit's two MFMAs covers one k-set
// for two tokens, and a second pair of tokens takes two MFMAs more.  Accumulator lane (n, g) then holds the four
// sub-block sums of weight row n, token g / 2 of the pair, plane g % 2 -- the four that the k-set's four scale bytes
// weigh -- so the weights are unpacked once for all tokens and only the short scale arithmetic is per token.
//
// The partial sums of the eight wavefronts (the K split of a round) of up to 56 groups and four tokens would not fit
// LDS beside the tokens' plane tables, so they are added up on the way: at the end of a group every wavefront leaves
// its sums in one of two small exchange areas, and at the end of the next group -- two or more barriers later -- one
// wavefront (they take turns) adds the eight in a fixed order into the group's totals.
//
// Rows of 2048 or 4096 values: a wavefront's place in a group's rounds never changes, so its activation operands
// live in registers.  Longer rows read them from LDS every unit; with four tokens their tables do not fit for a
// whole row, and K is streamed in parts of 8192 values, each with tables of its own, one part on top of the other
// in the totals.
#include "ttq_gemv_q6k_stream.h"

namespace ttq {

namespace {

typedef uint32_t sm_u32x2 __attribute__((ext_vector_type(2)));

// TOK: activation rows of a pass (2 or 4); the other parameters as in the single-row kernel's shapes.
// RPG: rounds per group (rows of 2048 RPG values) when the kernel is built for one row length, else 0.
// KP: into how many parts of NBMAX blocks a row may fall; the parts are streamed one after the other, each with
// its own plane tables (four tokens' tables of a row of 14336 values would not fit LDS).
// SETS: real rows of a streamed row whose sums a wavefront can keep apart (unevenly folded rows: up to four).
template <int TOK_, int NBMAX_, int BUFS_, int WGS_, int MAXG_, int RPG_, int KP_ = 1, int SETS_ = 1>
struct Q6Multi {
  static constexpr int TOK = TOK_, NBMAX = NBMAX_, BUFS = BUFS_, WGS = WGS_, MAXG = MAXG_, RPG = RPG_, KP = KP_;
  static constexpr int SETS = SETS_;
  static_assert(RPG == 0 || (NBMAX == 8 * RPG && KP == 1), "a fixed row length is the table's");
};
// rows of 2048 RPG values (RPG 1 or 2), many of them, two tokens: two workgroups per compute unit
template <int RPG> using Q6M2Head = Q6Multi<2, 8 * RPG, 2, 2, 20, RPG>;
template <int RPG> using Q6M2One = Q6Multi<2, 8 * RPG, 3, 1, 56, RPG>;    // rows of 2048 RPG values, two tokens
template <int RPG> using Q6M4One = Q6Multi<4, 8 * RPG, 3, 1, 56, RPG>;    // rows of 2048 RPG values, four tokens
using Q6M2Wide = Q6Multi<2, 56, 3, 1, 24, 0, 1, 4>;                       // rows of up to 14336, two tokens
using Q6M4Wide = Q6Multi<4, 32, 3, 1, 6, 0, 2>;                           // rows of up to 14336, four tokens, K in two parts

template <typename XT, typename YT, typename CFG>
__global__ void __launch_bounds__(kQ6Threads) __attribute__((amdgpu_waves_per_eu(2 * CFG::WGS, 2 * CFG::WGS)))
gemv_q6k_multi_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                      const void* __restrict__ bias, int bias_dtype, int m, int n_out, int nb_arg, int groups_per_wg,
                      int groups_rem, int fold_log2, int fold_nb) {
  constexpr int TOK = CFG::TOK, kBufs = CFG::BUFS, kPairs = TOK / 2, RPG = CFG::RPG, KP = CFG::KP;
  const int nb = RPG > 0 ? 8 * RPG : nb_arg;              // blocks of a row: NBMAX KP at most
  static_assert(TOK == 2 || TOK == 4, "tokens come in pairs");
  static_assert(kBufs >= 2 && kBufs <= 3, "the waits below count up to two later rounds");
  // a token's plane table: kXaHead bytes of zeros, then (16 values, plane) entries of 16 bytes.  Consecutive tables
  // are 64 bytes apart in the bank pattern (256 bytes), so that the four entries a 16-lane group reads for one
  // sub-block -- two tokens, two planes -- and the zeros of its other lanes are five different 16-byte columns.
  constexpr int kXaHead = 512;
  constexpr int kXaTok = kXaHead + CFG::NBMAX * 512 + 64;
  // a token's scales of the integer sums: (unit, plane, k-set) floats
  constexpr int kFacTok = CFG::NBMAX * 32;
  constexpr int SETS = CFG::SETS;
  constexpr int kStageWave = SETS * TOK * 64;                // bytes of a wavefront's sums in an exchange area
  constexpr int kStageHalf = kQ6Waves * kStageWave;          // bytes of one exchange area
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kBufs * kQ6BufBytes];
  __shared__ __attribute__((aligned(16))) uint8_t xa[TOK * kXaTok];
  __shared__ __attribute__((aligned(16))) float fac[TOK * CFG::NBMAX * 8];
  __shared__ __attribute__((aligned(16))) float stage[2][kQ6Waves][SETS][TOK][16];
  __shared__ __attribute__((aligned(16))) float total[CFG::MAXG][TOK][16];
  // The raw activations land where their planes will be: 16 values are 32 bytes either way, and the two threads
  // that turn them into two entries of 16 bytes are neighbours in one wavefront, which has read before it writes.
  // So the stream buffers are free from the start.  (The tables are written from inline asm like everything else
  // that requests land in: the compiler would wait for every request in flight first.)

  const int n_in = nb * 256;
  // Folded rows (fold_log2 > 0, as in the single-row kernel): 2^fold_log2 consecutive real rows of 2048 >> fold_log2
  // values are streamed as one row of eight blocks against the activations repeated; n_out counts streamed rows.
  // fold_nb > 0: real rows of fold_nb blocks, not a divisor of eight; a round's blocks belong to different real rows
  // from round to round, so a wavefront keeps one sum per real row of the streamed row (SETS of them at most) and
  // hands all of them over at the end of the group (single part of K only).
  const int x_len = n_in >> fold_log2;
  const int x_mask = fold_log2 ? x_len - 1 : -1;          // (fold_nb == 0: a folded length is a power of two)
  const bool per_round = fold_nb != 0;
  const uint32_t row_bytes = (uint32_t)nb * 210u;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int m0 = (int)blockIdx.y * TOK;                   // rows past the last one repeat it and are not stored
  const int bx = blockIdx.x;
  const int grp0 = bx * groups_per_wg + min(bx, groups_rem);
  const int ng = groups_per_wg + (bx < groups_rem ? 1 : 0);            // 1 .. CFG::MAXG

  // ---- requests of a round, exactly as in the single-row kernel: request q = wave + 8 i fills LDS chunks
  // 64 q .. 64 q + 63 of the buffer; chunk position 112 n + (c + n) % 112 holds chunk c of row n's eight slots
  uint32_t src_off[kQ6ReqMax];
#pragma unroll
  for (int i = 0; i < kQ6ReqMax; i++) {
    const int p = min(64 * (wave + kQ6Waves * i) + lane, 16 * kQ6RowChunks - 1);
    const int row = p / kQ6RowChunks, pos = p - row * kQ6RowChunks;
    const int c = pos >= row ? pos - row : pos - row + kQ6RowChunks;
    const int b = c / kQ6SlotChunks, j = c - b * kQ6SlotChunks;
    src_off[i] = (uint32_t)row * row_bytes + (uint32_t)(b * 210 - 2 * (b & 1) + (j < kQ6SlotChunks - 1 ? 16 * j : kQ6TailAt));
  }
  const bool full = wave < kQ6FullWaves;
  // all but the youngest `rounds_after` rounds of requests of this wavefront have landed
  auto wait_rounds = [&](auto rounds_after) {
    constexpr int A = decltype(rounds_after)::value;
    if (full) sm_wait_vmcnt<A * kQ6ReqMax>();
    else sm_wait_vmcnt<A * (kQ6ReqMax - 1)>();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;

  // ---- the parts of K (one, unless the configuration says otherwise): blocks kb0 .. kb0 + nbp - 1 of every row
  for (int kp = 0, kb0 = 0; kp < KP && kb0 < nb; kp++, kb0 += CFG::NBMAX) {
  const int nbp = min(nb - kb0, CFG::NBMAX);
  const int n_in_p = nbp * 256;
  const int rpg = nbp >> 3;                               // rounds per group
  const int nrounds = rpg * ng;

  // ---- the activations, as LDS requests: thread t fetches values 8 t + 4096 i .. + 7 of every token's part
  constexpr int kXPasses = (CFG::NBMAX * 256 + 8 * kQ6Threads - 1) / (8 * kQ6Threads);
#pragma unroll
  for (int t = 0; t < TOK; t++) {
    const uint16_t* xt = x + (int64_t)min(m0 + t, m - 1) * x_len + kb0 * 256;
#pragma unroll
    for (int i = 0; i < kXPasses; i++) {
      const int k0 = 8 * tid + i * (8 * kQ6Threads);
      if (k0 < n_in_p)                                    // whole wavefronts: the part is a multiple of 512
        __builtin_amdgcn_global_load_lds((sm_gptr_t)(xt + (per_round ? k0 % x_len : (k0 & x_mask))),
                                         (sm_lptr_t)(xa + t * kXaTok + kXaHead + i * (16 * kQ6Threads) + wave * 1024),
                                         16, 0, 0);
    }
  }
  // a compute unit serves its requests in the order they were made: every wavefront's activation requests are
  // queued before any weight request of the workgroup
  asm volatile("s_barrier" ::: "memory");

  // byte offset of the next round to request
  uint32_t req_src = (uint32_t)min(grp0, n_out / 16 - 1) * 16u * row_bytes + (uint32_t)kb0 * 210u;
  int req_kr = 0, req_buf = 0;
  auto request_next = [&]() {
    const uint8_t* src = w + (size_t)req_src;
    uint8_t* dst = wbuf + req_buf * kQ6BufBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kQ6ReqMax - 1; i++)
      __builtin_amdgcn_global_load_lds((sm_gptr_t)(src + src_off[i]), (sm_lptr_t)(dst + i * (kQ6Waves * 1024)), 16, 0, 2);
    if (full)
      __builtin_amdgcn_global_load_lds((sm_gptr_t)(src + src_off[kQ6ReqMax - 1]),
                                       (sm_lptr_t)(dst + (kQ6ReqMax - 1) * (kQ6Waves * 1024)), 16, 0, 2);
    req_buf = req_buf == kBufs - 1 ? 0 : req_buf + 1;
    req_kr++;
    req_src += kQ6RoundBlocks * 210;
    if (req_kr == rpg) {                  // the same part of the next group's rows
      req_kr = 0;
      req_src += 16u * row_bytes - (uint32_t)rpg * (kQ6RoundBlocks * 210);
    }
  };
  // One round now, the others once the tables are built: a compute unit takes about 64 KiB of outstanding requests,
  // and a wavefront that asks for more sits in the request -- with the activations still unprocessed behind it.
  request_next();
  wait_rounds(I1{});
  // Long rows: the activations have landed, and their share of what the compute unit has in flight goes to a
  // second round (measured on short rows, whose activations are a quarter of a round: slower by 0.2 - 0.4 us).
  constexpr int kEarlyRounds = RPG == 0 && kBufs > 2 ? 2 : 1;
  if (kEarlyRounds > 1 && 1 < nrounds) request_next();

  // ---- the raw activations back into registers (each wavefront reads what it asked for), then into byte planes
  if (tid < 128) {
#pragma unroll
    for (int t = 0; t < TOK; t++) sm_write_b32(sm_lds(xa) + (uint32_t)(t * kXaTok + 4 * tid), 0u);
  }
#pragma unroll
  for (int t = 0; t < TOK; t++) {
#pragma unroll
    for (int i = 0; i < kXPasses; i++) {
      const int k0 = 8 * tid + i * (8 * kQ6Threads);
      if (k0 >= n_in_p) break;
      float xf[8];
      const uint32_t tab = sm_lds(xa) + (uint32_t)(t * kXaTok + kXaHead);
      const sm_u32x4 r = sm_read16(tab + (uint32_t)(i * (16 * kQ6Threads) + tid * 16));
      widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), xf);
      uint32_t amax = amax_bits(xf);
      // the eight threads of 64 values are an aligned octet
      amax = umax(amax, dpp_quad_u32<0xB1>(amax));
      amax = umax(amax, dpp_quad_u32<0x4E>(amax));
      amax = umax(amax, dpp_other_quad_u32(amax));
      const uint32_t eb = amax >> 23;                        // biased exponent of max |x|; 255 for Inf and NaN
      const uint32_t ec = eb < 18u ? 18u : eb;               // 2^(E-13) / 4 stays a normal number
      const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
      // non-finite activations poison their 64 values instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
      // v = rint(x * 2^(13-E)) read off the low bits of x * 2^(13-E) + 1.5 * 2^23; the planes are byte 1 of
      // v + 128 (the high one: (v + 128) >> 8) and byte 0 of v (the low one, a signed byte)
      uint32_t vb[8];
#pragma unroll
      for (int j = 0; j < 8; j++) vb[j] = __float_as_uint(fmaf_(xf[j], mul, __uint_as_float(kRoundMagicBits)));
      // entry (k / 16, plane), 16 bytes; this thread's eight values are one half of it
      const uint32_t e = tab + (uint32_t)((k0 >> 4) * 32 + ((k0 >> 3) & 1) * 8);
      sm_write_b64(e, pack_bytes1(vb[0] + 128u, vb[1] + 128u, vb[2] + 128u, vb[3] + 128u),
                   pack_bytes1(vb[4] + 128u, vb[5] + 128u, vb[6] + 128u, vb[7] + 128u));
      sm_write_b64(e + 16u, pack_low_bytes((int)vb[0], (int)vb[1], (int)vb[2], (int)vb[3]),
                   pack_low_bytes((int)vb[4], (int)vb[5], (int)vb[6], (int)vb[7]));
      // the weights arrive as 4 * (q - 32): a quarter of the scale; the high plane counts 256
      if ((tid & 7) == 0) {
        const int k64 = k0 >> 6;       // unit k64 / 2, k-set k64 % 2
        float* ft = &fac[t * (CFG::NBMAX * 8) + (k64 >> 1) * 4 + (k64 & 1)];
        ft[0] = f * 64.f;
        ft[2] = f * 0.25f;
      }
    }
  }

  // ---- per-lane constants of the main loop
  const uint32_t sh1 = 6u - 2u * (uint32_t)(g >> 1), sh2 = 2u - 2u * (uint32_t)(g >> 1);
  auto chunk_at = [&](int c) {
    const int pos = c + n < kQ6RowChunks ? c + n : c + n - kQ6RowChunks;
    return (uint32_t)((n * kQ6RowChunks + pos) * 16);
  };
  // The wavefront's block of the round.  Wavefronts w and w + 4 share a SIMD: one of them takes an even block, the
  // other an odd one (which costs a dozen instructions more per unit), so that the four SIMDs carry the same load.
  const int blk = wave < 4 ? 2 * wave : 2 * wave - 7;
  const int slot = blk * kQ6SlotChunks;
  // activation operand: lane (i, g) holds row i = 8 (token of the pair) + 4 plane + sub-block, values 16 g .. of the
  // k-set: something only where the sub-block is g.  The other lanes read zeros in front of the tables (the
  // offsets of pair and k-set lead to zeros as well).  Unit u = 2 block + half starts at value 128 u.
  const uint32_t xa_base = sm_lds(xa);
  const bool mine = (n & 3) == g;
  const uint32_t u0 = (uint32_t)(2 * blk);                 // the wavefront's first unit of a group's first round
  const uint32_t a_addr = mine ? xa_base + (uint32_t)((n >> 3) * kXaTok + kXaHead + 32 * g + 16 * ((n >> 2) & 1)) + 256u * u0
                               : xa_base + (uint32_t)(32 * g + 32);
  const uint32_t a_step = mine ? 256u : 0u;                // per unit 256 bytes of table, per round 16 units
  // accumulator lane (n, g): token g / 2 of the pair, plane g % 2; its scales for the two k-sets are neighbours
  const uint32_t fac_addr0 = sm_lds(fac) + (uint32_t)((g >> 1) * kFacTok + 8 * (g & 1)) + 16u * u0;
  const uint32_t wbuf_base = sm_lds(wbuf);
  const uint32_t stage_base = sm_lds(&stage[0][0][0][0][0]);
  const uint32_t total_base = sm_lds(&total[0][0][0]);
  const uint32_t stage_addr = stage_base + (uint32_t)(wave * kStageWave + (g >> 1) * 64 + 4 * n);

  sm_barrier();                         // the plane tables are complete
#pragma unroll
  for (int i = kEarlyRounds; i < kBufs; i++)
    if (i < nrounds) request_next();

  // the eight wavefronts' sums of group `grp` (complete since a barrier) -> its totals, in wavefront order
  // the eight wavefronts' sums of group `grp` (complete since a barrier) -> its totals, in wavefront order
  auto reduce_group = [&](int grp) {
    if (lane < TOK * 16) {
      // one set of sums, or with unevenly folded rows one per real row of the streamed row
      const int sets = per_round ? (1 << fold_log2) : 1;
      for (int r = 0; r < sets; r++) {
        const uint32_t a = stage_base + (uint32_t)((grp & 1) * kStageHalf + r * (TOK * 64) + 4 * lane);
        float v[kQ6Waves];
        asm volatile(
            "ds_read_b32 %0, %8\n\t"
            "ds_read_b32 %1, %8 offset:%9\n\t"
            "ds_read_b32 %2, %8 offset:%10\n\t"
            "ds_read_b32 %3, %8 offset:%11\n\t"
            "ds_read_b32 %4, %8 offset:%12\n\t"
            "ds_read_b32 %5, %8 offset:%13\n\t"
            "ds_read_b32 %6, %8 offset:%14\n\t"
            "ds_read_b32 %7, %8 offset:%15\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
            : "v"(a), "n"(kStageWave), "n"(2 * kStageWave), "n"(3 * kStageWave), "n"(4 * kStageWave), "n"(5 * kStageWave),
              "n"(6 * kStageWave), "n"(7 * kStageWave)
            : "memory");
        if (per_round) {
          // (a wavefront without a block of real row r in this group left a zero)
          float sum = v[0];
#pragma unroll
          for (int wv = 1; wv < kQ6Waves; wv++) sum += v[wv];
          sm_write_f32(total_base + (uint32_t)(((grp << fold_log2) + r) * (TOK * 64) + 4 * lane), sum);
        } else if (fold_log2 == 0) {
          float sum = v[0];
#pragma unroll
          for (int wv = 1; wv < kQ6Waves; wv++) sum += v[wv];
          const uint32_t ta = total_base + (uint32_t)(grp * (TOK * 64) + 4 * lane);
          if (KP > 1 && kp > 0) {             // on top of the earlier parts of K
            float before;
            asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(before) : "v"(ta) : "memory");
            sum += before;
          }
          sm_write_f32(ta, sum);
        } else {
          // folded rows: the wavefronts whose blocks belong to real row fs of the streamed one (wavefront wv has
          // block wv < 4 ? 2 wv : 2 wv - 7), in wavefront order; a group's totals are 2^fold_log2 sets
          for (int fs = 0; fs < (1 << fold_log2); fs++) {
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < kQ6Waves; wv++) {
              const int b = wv < 4 ? 2 * wv : 2 * wv - 7;
              if ((b >> (3 - fold_log2)) == fs) sum += v[wv];
            }
            sm_write_f32(total_base + (uint32_t)(((grp << fold_log2) + fs) * (TOK * 64) + 4 * lane), sum);
          }
        }
      }
    }
  };

  // ODD: the wavefront's blocks sit two bytes into their slots
  auto run_rounds = [&](auto oddc) {
    constexpr bool ODD = decltype(oddc)::value;
    // unit hf (half of the block): ql chunk 4 hf + g, qh chunk 8 + 2 hf + g % 2 (plus the first dword of the
    // chunk after it when the block is shifted); the unit's eight scales are bytes 8 hf .. of chunk 12; d near the
    // end of chunk 13
    const uint32_t ql_off0 = chunk_at(slot + g), ql_off1 = chunk_at(slot + 4 + g);
    const uint32_t qh_off0 = chunk_at(slot + 8 + (g & 1)), qh_off1 = chunk_at(slot + 10 + (g & 1));
    const uint32_t qlx_off0 = chunk_at(slot + g + 1), qlx_off1 = chunk_at(slot + 4 + g + 1);
    const uint32_t qhx_off0 = chunk_at(slot + 8 + (g & 1) + 1), qhx_off1 = chunk_at(slot + 10 + (g & 1) + 1);
    const uint32_t sc_off = chunk_at(slot + 12);
    // shifted: the dword after the unit's eight bytes (for the second unit that is byte 12 of chunk 13, which holds
    // the block's bytes 194..209)
    const uint32_t scx_off0 = sc_off + 8u, scx_off1 = chunk_at(slot + 13) + 12u;
    const uint32_t d_off = chunk_at(slot + 13) + (uint32_t)(kQ6DAt + (ODD ? 2 : 0));

    // a unit's weights, and its activations: the operand rows of the tokens and the scales of their sums
    struct Regs { sm_u32x4 ql, qh; sm_u32x2 sc; uint32_t d, qlx, qhx, scx; };
    struct Acts { sm_u32x4 a[TOK]; sm_u32x2 f[kPairs]; };
    // unit ui of a group (16 to a round)
    auto issue_acts = [&](uint32_t ui, Acts& t) {
      const uint32_t xaddr = a_addr + ui * a_step;
      const uint32_t fa = fac_addr0 + 16u * ui;
      asm volatile(
          "ds_read_b128 %0, %3\n\t"
          "ds_read_b128 %1, %3 offset:128\n\t"
          "ds_read_b64 %2, %4"
          : "=&v"(t.a[0]), "=&v"(t.a[1]), "=&v"(t.f[0])
          : "v"(xaddr), "v"(fa)
          : "memory");
      if constexpr (TOK == 4) {
        asm volatile(
            "ds_read_b128 %0, %3 offset:%5\n\t"
            "ds_read_b128 %1, %3 offset:%6\n\t"
            "ds_read_b64 %2, %4 offset:%7"
            : "=&v"(t.a[2]), "=&v"(t.a[3]), "=&v"(t.f[kPairs - 1])
            : "v"(xaddr), "v"(fa), "n"(2 * kXaTok), "n"(2 * kXaTok + 128), "n"(2 * kFacTok)
            : "memory");
      }
    };
    // (behind a wait) the registers hold what was read
    auto settle_acts = [&](Acts& t) {
      asm volatile("" : "+v"(t.a[0]), "+v"(t.a[1]), "+v"(t.f[0]));
      if constexpr (TOK == 4) asm volatile("" : "+v"(t.a[2]), "+v"(t.a[3]), "+v"(t.f[kPairs - 1]));
    };
    // unit hf of the round in `buf`
    auto issue = [&](auto hc, uint32_t buf, Regs& r) {
      constexpr int hf = decltype(hc)::value;
      const uint32_t a_ql = buf + (hf ? ql_off1 : ql_off0), a_qh = buf + (hf ? qh_off1 : qh_off0);
      const uint32_t a_sc = buf + sc_off, a_d = buf + d_off;
      asm volatile(
          "ds_read_b128 %0, %4\n\t"
          "ds_read_b128 %1, %5\n\t"
          "ds_read_b64 %2, %6 offset:%8\n\t"
          "ds_read_u16 %3, %7"
          : "=&v"(r.ql), "=&v"(r.qh), "=&v"(r.sc), "=&v"(r.d)
          : "v"(a_ql), "v"(a_qh), "v"(a_sc), "v"(a_d), "n"(8 * hf)
          : "memory");
      if constexpr (ODD) {
        const uint32_t a_qlx = buf + (hf ? qlx_off1 : qlx_off0), a_qhx = buf + (hf ? qhx_off1 : qhx_off0);
        const uint32_t a_scx = buf + (hf ? scx_off1 : scx_off0);
        asm volatile(
            "ds_read_b32 %0, %3\n\t"
            "ds_read_b32 %1, %4\n\t"
            "ds_read_b32 %2, %5"
            : "=&v"(r.qlx), "=&v"(r.qhx), "=&v"(r.scx)
            : "v"(a_qlx), "v"(a_qhx), "v"(a_scx)
            : "memory");
      }
    };
    constexpr int kReads = 4 + (ODD ? 3 : 0) + (RPG > 0 ? 0 : TOK + kPairs);   // LDS reads of a unit
    static_assert(kReads <= 15, "the wait counts reads of the other unit");
    auto settle = [&](auto pending, Regs& r) {
      constexpr int P = decltype(pending)::value;
      asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r.ql), "+v"(r.qh), "+v"(r.sc), "+v"(r.d) : "n"(P) : "memory");
      if constexpr (ODD) asm volatile("" : "+v"(r.qlx), "+v"(r.qhx), "+v"(r.scx));
    };
    float acc[kPairs];
#pragma unroll
    for (int q = 0; q < kPairs; q++) acc[q] = 0.f;
    auto compute = [&](const Regs& r, const Acts& t) {
      uint32_t ql[4], qh[4], sc[2];
      if constexpr (ODD) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          ql[i] = __builtin_amdgcn_alignbit(i < 3 ? r.ql[i + 1] : r.qlx, r.ql[i], 16);
          qh[i] = __builtin_amdgcn_alignbit(i < 3 ? r.qh[i + 1] : r.qhx, r.qh[i], 16);
        }
        sc[0] = __builtin_amdgcn_alignbit(r.sc[1], r.sc[0], 16);
        sc[1] = __builtin_amdgcn_alignbit(r.scx, r.sc[1], 16);
      } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          ql[i] = r.ql[i];
          qh[i] = r.qh[i];
        }
        sc[0] = r.sc[0];
        sc[1] = r.sc[1];
      }
      v4i_t B[2];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        // 4 * (q - 32) as a signed byte: nibble into bits 2-5, bit pair into bits 6-7, low bits cleared and
        // the top bit flipped
        const uint32_t t1 = ((ql[i] << 2) & 0x3C3C3C3Cu) | ((qh[i] << sh1) & ~0x3C3C3C3Cu);
        const uint32_t t2 = ((ql[i] >> 2) & 0x3C3C3C3Cu) | ((qh[i] << sh2) & ~0x3C3C3C3Cu);
        B[0][i] = (int)((t1 & 0xFCFCFCFCu) ^ 0x80808080u);
        B[1][i] = (int)((t2 & 0xFCFCFCFCu) ^ 0x80808080u);
      }
      int s8[2][4];
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int s = (int)sc[h];
        s8[h][0] = (int)(int8_t)(s & 0xFF);
        s8[h][1] = (int)(int8_t)((s >> 8) & 0xFF);
        s8[h][2] = (int)(int8_t)((s >> 16) & 0xFF);
        s8[h][3] = s >> 24;
      }
      const float d = f16_bits_to_f32((uint16_t)(r.d & 0xFFFFu));
      const v4i_t zero = {0, 0, 0, 0};
#pragma unroll
      for (int q = 0; q < kPairs; q++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
          v4i_t A;
#pragma unroll
          for (int i = 0; i < 4; i++) A[i] = (int)t.a[2 * q + h][i];
          const v4i_t C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B[h], zero, 0, 0, 0);
          // 24-bit multiplies (full rate; a 32-bit one takes four times as long): |C| <= 16 * 128 * 128
          const int ts = __mul24(s8[h][0], C[0]) + __mul24(s8[h][1], C[1]) +
                         __mul24(s8[h][2], C[2]) + __mul24(s8[h][3], C[3]);
          acc[q] = fmaf_((float)ts * __uint_as_float(t.f[q][h]), d, acc[q]);
        }
        // pins the arithmetic here: left alone the compiler moves it behind later waits
        asm volatile("" : "+v"(acc[q]));
      }
    };

    using U0 = std::integral_constant<int, 0>;
    using U1 = std::integral_constant<int, 1>;
    // Short rows (RPG rounds to a group, known at compile time): the wavefront's place in a group's rounds never
    // changes, so neither do the activations it multiplies: they stay in registers for all its groups.
    Acts held[RPG > 0 ? RPG : 1][2];
    if constexpr (RPG > 0) {
#pragma unroll
      for (int kr = 0; kr < RPG; kr++) {
        issue_acts(16u * (uint32_t)kr, held[kr][0]);
        issue_acts(16u * (uint32_t)kr + 1u, held[kr][1]);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int kr = 0; kr < RPG; kr++) {
        settle_acts(held[kr][0]);
        settle_acts(held[kr][1]);
      }
    }
    int bufi = 0, rr = 0;
    // round kr of its group; ta, tb: the activations of its two units
    auto round = [&](uint32_t kr, Acts& ta, Acts& tb) {
      // the round's buffer: own requests landed, then everybody's
      const int later = min(nrounds - 1 - rr, kBufs - 1);          // rounds requested after this one
      if (later == 2) wait_rounds(I2{});
      else if (later == 1) wait_rounds(I1{});
      else wait_rounds(I0{});
      sm_barrier();
      const uint32_t buf = wbuf_base + (uint32_t)(bufi * kQ6BufBytes);
      Regs ra, rb;
      issue(U0{}, buf, ra);
      if constexpr (RPG == 0) issue_acts(16u * kr, ta);
      issue(U1{}, buf, rb);
      if constexpr (RPG == 0) issue_acts(16u * kr + 1u, tb);
      settle(std::integral_constant<int, kReads>{}, ra);
      if constexpr (RPG == 0) settle_acts(ta);
      compute(ra, ta);
      settle(I0{}, rb);
      if constexpr (RPG == 0) settle_acts(tb);
      // every wavefront has read what it needs of the buffer: a later round may land there
      sm_barrier();
      if (rr + kBufs < nrounds) request_next();
      bufi = bufi == kBufs - 1 ? 0 : bufi + 1;
      rr++;
      compute(rb, tb);
    };
    // Unevenly folded rows: the sums per real row of the streamed row.  The real row of the wavefront's block in
    // round kr is (8 kr + blk) / fold_nb, the same for all lanes: a quotient and a remainder that advance by eight
    // blocks per round.
    float accf[kPairs][SETS];
#pragma unroll
    for (int q = 0; q < kPairs; q++)
#pragma unroll
      for (int r = 0; r < SETS; r++) accf[q][r] = 0.f;
    const int fq0 = per_round ? blk / fold_nb : 0, fr0 = per_round ? blk - fq0 * fold_nb : 0;
    int fq = fq0, fr = fr0;
    auto to_real_row = [&]() {
#pragma unroll
      for (int q = 0; q < kPairs; q++) {
#pragma unroll
        for (int r = 0; r < SETS; r++)
          if (fq == r) accf[q][r] += acc[q];
        acc[q] = 0.f;
      }
      fr += 8;
      while (fr >= fold_nb) {
        fr -= fold_nb;
        fq++;
      }
    };
    // the wavefront's sums of group `idx`: the two planes of a (row, token) are 16 lanes apart; then the group
    // before it, which every wavefront handed over before the barriers since
    auto hand_over = [&](int idx) {
      if (per_round) {
#pragma unroll
        for (int q = 0; q < kPairs; q++)
#pragma unroll
          for (int r = 0; r < SETS; r++) {
            const float v = add_xor16(accf[q][r]);
            if ((g & 1) == 0) sm_write_f32(stage_addr + (uint32_t)((idx & 1) * kStageHalf + r * (TOK * 64) + q * 128), v);
            accf[q][r] = 0.f;
          }
        fq = fq0;
        fr = fr0;
      } else {
#pragma unroll
        for (int q = 0; q < kPairs; q++) {
          acc[q] = add_xor16(acc[q]);
          if ((g & 1) == 0) sm_write_f32(stage_addr + (uint32_t)((idx & 1) * kStageHalf + q * 128), acc[q]);
          acc[q] = 0.f;
        }
      }
      if (idx > 0 && wave == ((idx - 1) & 7)) reduce_group(idx - 1);
    };
    for (int gi = 0; gi < ng; gi++) {
      if constexpr (RPG > 0) {
#pragma unroll
        for (int kr = 0; kr < RPG; kr++) round((uint32_t)kr, held[kr][0], held[kr][1]);
      } else {
        for (int kr = 0; kr < rpg; kr++) {
          Acts ta, tb;
          round((uint32_t)kr, ta, tb);
          if (per_round) to_real_row();
        }
      }
      hand_over(gi);     // the group is complete
    }
  };
  if (blk & 1) run_rounds(std::true_type{});
  else run_rounds(std::false_type{});
  // every wavefront has left its last sums and is done with the buffers and the tables
  sm_barrier();
  if (wave == ((ng - 1) & 7)) reduce_group(ng - 1);
  }   // parts of K
  // every request has landed (plain loads are safe again)
  __syncthreads();
  for (int t = tid; t < (ng * TOK * 16) << fold_log2; t += kQ6Threads) {
    // set gs = (group, real row of the streamed row); folded launches keep ng << fold_log2 <= MAXG
    const int gs = t / (TOK * 16), tok = (t >> 4) % TOK, nn = t & 15;
    const int grp = gs >> fold_log2, fs = gs & ((1 << fold_log2) - 1);
    if (m0 + tok < m) {
      const int row = (((grp0 + grp) * 16 + nn) << fold_log2) + fs;
      YElem<YT>::store(y + (((int64_t)(m0 + tok) * n_out) << fold_log2), row,
                       total[gs][tok][nn] + load_bias(bias, bias_dtype, row));
    }
  }
}

// Which shape takes (m, n_out, n_in): 0 none, else 1 Q6M2Head, 2 Q6M2One, 3 Q6M4One, 4 Q6M2Wide, 5 Q6M4Wide.
struct Q6MultiPlan { int kind, tok, num_wg, fold_log2, fold_nb; };
Q6MultiPlan q6_multi_plan(int64_t m, int64_t n_out, int64_t n_in) {
  Q6MultiPlan p{0, 0, 0, 0, 0};
  const Q6Plan single = q6_plan(n_out, n_in);              // the stream's own limits
  // (folded rows: the streamed shape)
  p.fold_log2 = single.fold_log2;
  const int64_t nb = (n_in << p.fold_log2) / 256, groups = (n_out >> p.fold_log2) / 16;
  // (more than four rows: passes of four on gridDim.y; the entry points hand over 65535 rows at most)
  static const int max_rows = dev_knob("TTQ_Q6_MULTI_MAX_ROWS", 65535);
  if (!single.ok || m < 2 || m > max_rows) return p;
  p.fold_nb = single.fold_nb;
  if (p.fold_nb && (1 << single.fold_log2) > Q6M2Wide::SETS) return p;     // (rows of an odd number of blocks)
  static_assert(Q6M4Wide::NBMAX * Q6M4Wide::KP >= Q6Wide::NBMAX && Q6M2Wide::NBMAX >= Q6Wide::NBMAX, "every row length of the stream");
  const int cus = device_num_cus();
  int maxg, wgs = 1;
  if (nb <= 16) {
    static const int force_tok = dev_knob("TTQ_Q6_MULTI_TOK", 0);
    static const int use_head = dev_knob("TTQ_Q6_MULTI_HEAD", 1);
    p.tok = force_tok ? force_tok : (m == 2 ? 2 : 4);
    if (p.tok == 4) {
      p.kind = 3;
      maxg = Q6M4One<1>::MAXG;
    } else if (groups >= 2 * (int64_t)Q6M2Head<1>::WGS * cus && use_head) {
      p.kind = 1;
      wgs = Q6M2Head<1>::WGS;
      maxg = Q6M2Head<1>::MAXG;
    } else {
      p.kind = 2;
      maxg = Q6M2One<1>::MAXG;
    }
  } else if (m == 2 || p.fold_nb) {      // (unevenly folded rows: two tokens a pass, one part of K)
    p.kind = 4;
    p.tok = 2;
    maxg = Q6M2Wide::MAXG;
  } else {
    p.kind = 5;
    p.tok = 4;
    maxg = Q6M4Wide::MAXG;
  }
  maxg >>= p.fold_log2;                                      // a folded group has that many sets of totals
  p.num_wg = (int)std::min<int64_t>(groups, (int64_t)wgs * cus);
  // (whole waves of workgroups, as in the single-row plan)
  if ((groups + p.num_wg - 1) / p.num_wg > maxg) p.num_wg *= (int)((groups + (int64_t)p.num_wg * maxg - 1) / ((int64_t)p.num_wg * maxg));
  return p;
}

template <typename XT, typename YT>
hipError_t q6_multi_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m,
                              int64_t n_out, int64_t n_in, hipStream_t s) {
  const Q6MultiPlan p = q6_multi_plan(m, n_out, n_in);
  if (!p.kind) return hipErrorInvalidValue;
  const int64_t rows = n_out >> p.fold_log2, nb = (n_in << p.fold_log2) / 256;      // the streamed shape
  const int groups = (int)(rows / 16);
  const dim3 grid((unsigned)p.num_wg, (unsigned)((m + p.tok - 1) / p.tok)), block(kQ6Threads);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)m, (int)rows, (int)nb, groups / p.num_wg,
                       groups % p.num_wg, p.fold_log2, p.fold_nb);
  };
  const bool one = nb == 8;                                  // else, for kinds 1 to 3, 16
  switch (p.kind) {
    case 1: one ? go(gemv_q6k_multi_kernel<XT, YT, Q6M2Head<1>>) : go(gemv_q6k_multi_kernel<XT, YT, Q6M2Head<2>>); break;
    case 2: one ? go(gemv_q6k_multi_kernel<XT, YT, Q6M2One<1>>) : go(gemv_q6k_multi_kernel<XT, YT, Q6M2One<2>>); break;
    case 3: one ? go(gemv_q6k_multi_kernel<XT, YT, Q6M4One<1>>) : go(gemv_q6k_multi_kernel<XT, YT, Q6M4One<2>>); break;
    case 4: go(gemv_q6k_multi_kernel<XT, YT, Q6M2Wide>); break;
    default: go(gemv_q6k_multi_kernel<XT, YT, Q6M4Wide>); break;
  }
  return hipGetLastError();
}

template <typename XT>
hipError_t q6_multi_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                             int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q6_multi_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return q6_multi_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return q6_multi_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool gemv_q6k_stream4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in) {
  if (format != kQ6_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  return q6_multi_plan(m, n_out, n_in).kind != 0;
}

hipError_t launch_gemv_q6k_stream4(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                   int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return q6_multi_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return q6_multi_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
