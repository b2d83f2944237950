// Decode GEMV for Q6_K weights on gfx950 with rows of 2048 to 14336 values (in a "Q4_K_M" file: the LM head
// and half of the down projections): the weight stream goes HBM -> LDS as whole cache lines and feeds the int8
// matrix cores.
//
// Operator: F.linear with a single-token activation (workspace/libtorch/src/abi/neural_nets.nim:64-81) over a
// weight stored as GGUF Q6_K blocks { u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d } of 256 weights,
// w = d * scale[e / 16] * (q6[e] - 32).
//
// A 210-byte block is neither a multiple of a cache line nor of a dword, so the per-wavefront line rings of the
// Q4_K kernel (ttq_gemv_q4k_stream.h) do not carry over.  What is line-shaped is a group of 16 rows: 53 760
// contiguous bytes = 420 lines.  So here the eight wavefronts of a workgroup share the stream:
//   * a round is eight blocks (2048 values) of one group of 16 rows: 16 runs of 1680 contiguous bytes, copied
//     into one of two or three LDS buffers by 28 requests of 1 KiB (global_load_lds_dwordx4, no registers), four or three per
//     wavefront.  On the way in every block is moved to a 16-byte boundary: it lands in a slot of 14 chunks
//     of 16 bytes, 13 fetched from consecutive addresses and one that ends with the block's last bytes, and
//     row n is rotated by n chunks, which puts the 16 rows of an operand read into 16 different bank groups.
//     Fetch addresses are rounded down to a dword: requests at 2 mod 4 were measured 15 % slower than
//     dword-aligned ones, and operand reads at 2 mod 4 -- which the packed layout would need for every other
//     block -- at three times the cost of the whole stream.  So an odd block lands two bytes into its slot,
//     and the wavefronts that multiply odd blocks (the odd ones: block = 8 * round + wavefront) shift their
//     operands by 16 bits in registers;
//   * while one buffer is multiplied, the next rounds are in flight or landed (a compute unit takes about
//     64 KiB of outstanding requests); a wavefront waits for its own requests on its own counter, a barrier
//     makes the buffer whole, a second one frees it for a later round;
//   * along K a round is split: wavefront w multiplies block w of the eight for all 16 rows, two units of
//     16 rows x 128 weights, two v_mfma_i32_16x16x64_i8 each;
//   * rows of 4096 values and many of them (the LM head): two workgroups per compute unit with two buffers
//     each, so that one's arithmetic falls into the other's waits; otherwise one workgroup with three buffers;
//   * rows of 2048 or 4096 values: a group is one or two rounds and a wavefront's place in them never changes, so
//     the activation operands and scales of its two or four units are read into registers once, not per unit.
// Arithmetic.  The activations are block fixed point, 15 bits in two byte planes with one power-of-two scale
// per 64 values.  A weight reaches the matrix core as the signed byte 4 * (q6 - 32) = ((q6 << 2) ^ 0x80), built
// from the nibble and the bit pair with four instructions per dword.  The 16 columns of the MFMA that a GEMV
// does not need carry the bookkeeping instead: the activation operand holds, in row 8 h + 4 p + j, plane p of
// the 16 values of sub-block j of k-set h and zeros elsewhere, so that one accumulator lane ends up with the
// four sub-block sums of one row, one plane, one k-set -- exactly the four that its four consecutive scale bytes
// weigh.  Integer sums are exact; each (row, unit) then takes one float multiply by a power of two and one
// fused multiply-add with d.  A unit-vector activation reproduces the canonical column bit for bit (d, scale
// and q6 - 32 have 11 + 7 + 6 significant bits, so every order of the products is exact).
#pragma once

#include "ttq_stream_common.h"

namespace ttq {

constexpr int kQ6Waves = 8;
constexpr int kQ6Threads = kQ6Waves * 64;
constexpr int kQ6RoundBlocks = 8;                          // blocks of a row in one round: one per wavefront
constexpr int kQ6SlotChunks = 14;                          // a block in LDS: 224 bytes
constexpr int kQ6TailAt = 196;                             // chunk 13 starts here, counted from the slot's first byte
constexpr int kQ6DAt = 208 - kQ6TailAt;                    // d in chunk 13 (+ 2 for an odd block)
constexpr int kQ6RowChunks = kQ6RoundBlocks * kQ6SlotChunks;   // 112
constexpr int kQ6Requests = 16 * kQ6RowChunks / 64;        // 28
constexpr int kQ6BufBytes = kQ6Requests * 1024;            // 28672
constexpr int kQ6ReqMax = (kQ6Requests + kQ6Waves - 1) / kQ6Waves;   // 4
constexpr int kQ6FullWaves = kQ6Requests - (kQ6ReqMax - 1) * kQ6Waves;   // wavefronts 0..3 make 4 requests, the others 3
static_assert(kQ6RoundBlocks == kQ6Waves, "one block of the round per wavefront");

// The two shapes of the kernel.  NBMAX: blocks per row it has tables for; BUFS: LDS buffers; WGS: workgroups per
// compute unit; MAXG: row groups of a workgroup (their partial sums wait in LDS, in the space where the raw
// activations land first).
// RPG: rounds per group when the kernel is built for one row length (2048 RPG values, NBMAX blocks), else 0.
// rows of 4096, many rows
struct Q6Head { static constexpr int NBMAX = 16, BUFS = 2, WGS = 2, MAXG = 20, RPG = 2; };
// rows of 2048 or 4096, fewer rows
template <int RPG_> struct Q6Short { static constexpr int NBMAX = 8 * RPG_, BUFS = 3, WGS = 1, MAXG = 56, RPG = RPG_; };
// rows up to 14336
struct Q6Wide { static constexpr int NBMAX = 56, BUFS = 3, WGS = 1, MAXG = 56, RPG = 0; };

// XT: bf16 or fp16 activations.  The row groups are dealt out in runs: the first groups_rem workgroups take
// groups_per_wg + 1 each, the others groups_per_wg.  nb: blocks per row, a multiple of eight.
// STAGE 0 is the GEMV; STAGE 1 leaves out the arithmetic on the operands, STAGE 2 the operand reads as well
// (requests, waits and barriers stay): what each part costs is measured by leaving it out.
template <typename XT, typename YT, typename CFG, int STAGE = 0>
__global__ void __launch_bounds__(kQ6Threads) __attribute__((amdgpu_waves_per_eu(2 * CFG::WGS, 2 * CFG::WGS)))
gemv_q6k_stream_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                       const void* __restrict__ bias, int bias_dtype, int n_out, int nb_arg, int groups_per_wg,
                       int groups_rem, int fold_log2, int fold_nb) {
  constexpr int kBufs = CFG::BUFS, RPG = CFG::RPG;
  static_assert(RPG == 0 || CFG::NBMAX == 8 * RPG, "a fixed row length is the table's");
  const int nb = RPG > 0 ? CFG::NBMAX : nb_arg;
  static_assert(kBufs >= 2 && kBufs <= 4, "the waits below count up to three later rounds");
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kBufs * kQ6BufBytes];
  __shared__ __attribute__((aligned(16))) v4i_t xa[CFG::NBMAX * 32 + 1];   // (16 values, plane) entries + one of zeros
  __shared__ __attribute__((aligned(16))) float fac[CFG::NBMAX * 4 * 2];   // (64 values, plane): scale of the integer sum
  // (the raw activations land here first: the partial sums are written after they have been read back)
  __shared__ __attribute__((aligned(1024))) float part[CFG::MAXG][kQ6Waves][16];
  static_assert(sizeof(part) >= CFG::NBMAX * 512, "room for the staged activations");
  uint8_t* xstage = reinterpret_cast<uint8_t*>(&part[0][0][0]);

  const int n_in = nb * 256;
  const int rpg = nb >> 3;                                // rounds per group
  const uint32_t row_bytes = (uint32_t)nb * 210u;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  // Folded rows (fold_log2 > 0): the matrix really has 2^fold_log2 times as many rows, of 2048 >> fold_log2 values
  // each; consecutive rows are contiguous in memory, so 2^fold_log2 of them are streamed as one row of eight
  // blocks against the activations repeated that often, and the wavefronts' sums are added per real row at the end.
  // fold_nb > 0: the real rows have fold_nb blocks, not a divisor of eight (1536, 2560, 3584, 5120 values ...), and
  // 2^fold_log2 = 8 / gcd(fold_nb, 8) of them make whole rounds.  A round's blocks then belong to different real
  // rows from one round to the next, so the wavefronts leave their sums after every round, not after every group,
  // and the end adds the (round, wavefront) sums of each real row's blocks.
  const int x_len = n_in >> fold_log2;
  const int x_mask = fold_log2 ? x_len - 1 : -1;          // (fold_nb == 0: a folded length is a power of two)
  const uint16_t* xm = x + (int64_t)blockIdx.y * x_len;
  YT* ym = y + (((int64_t)blockIdx.y * n_out) << fold_log2);
  const int bx = blockIdx.x;
  const int grp0 = bx * groups_per_wg + min(bx, groups_rem);
  const int ng = groups_per_wg + (bx < groups_rem ? 1 : 0);            // 1 .. CFG::MAXG
  const int nrounds = rpg * ng;

  // ---- the activations, as LDS requests too (a register load among the weight requests would make the
  // compiler wait for all of them at its first use): thread t stages x[8 t + 4096 i .. + 7]
  constexpr int kXPasses = (CFG::NBMAX * 256 + 8 * kQ6Threads - 1) / (8 * kQ6Threads);
#pragma unroll
  for (int i = 0; i < kXPasses; i++) {
    const int k0 = 8 * tid + i * (8 * kQ6Threads);
    if (k0 < n_in)                                        // whole wavefronts: n_in is a multiple of 512
      __builtin_amdgcn_global_load_lds((sm_gptr_t)(xm + (fold_nb ? k0 % x_len : (k0 & x_mask))),
                                       (sm_lptr_t)(xstage + i * (16 * kQ6Threads) + wave * 1024), 16, 0, 0);
  }
  // a compute unit serves its requests in the order they were made: every wavefront's activation requests are
  // queued before any weight request of the workgroup
  asm volatile("s_barrier" ::: "memory");

  // ---- requests of a round: request q = wave + 8 i fills LDS chunks 64 q .. 64 q + 63 of the buffer.  Chunk
  // position 112 n + (c + n) % 112 holds chunk c of row n's eight slots.
  uint32_t src_off[kQ6ReqMax];
#pragma unroll
  for (int i = 0; i < kQ6ReqMax; i++) {
    const int p = min(64 * (wave + kQ6Waves * i) + lane, 16 * kQ6RowChunks - 1);
    const int row = p / kQ6RowChunks, pos = p - row * kQ6RowChunks;
    const int c = pos >= row ? pos - row : pos - row + kQ6RowChunks;
    const int b = c / kQ6SlotChunks, j = c - b * kQ6SlotChunks;
    // an odd block starts at 2 mod 4: its slot starts two bytes early.  The last chunk of an even block reads two
    // bytes into the next block of the row; the last chunk of an odd block ends with the block.
    src_off[i] = (uint32_t)row * row_bytes + (uint32_t)(b * 210 - 2 * (b & 1) + (j < kQ6SlotChunks - 1 ? 16 * j : kQ6TailAt));
  }
  const bool full = wave < kQ6FullWaves;
  // rounds are requested in order: group by group, eight blocks by eight blocks
  // (every workgroup has a group; a workgroup without one would ask for the matrix's last group: never past the end,
  // and without a branch around the request, after which the compiler waits for every request in flight)
  uint32_t req_src = (uint32_t)min(grp0, n_out / 16 - 1) * 16u * row_bytes;    // byte offset of the next round to request
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
    // the next eight blocks of the rows, or the first eight of the next group
    req_kr++;
    req_src += kQ6RoundBlocks * 210;
    if (req_kr == rpg) {
      req_kr = 0;
      req_src += 15u * row_bytes;
    }
  };
  // all but the youngest `rounds_after` rounds of requests of this wavefront have landed
  auto wait_rounds = [&](auto rounds_after) {
    constexpr int A = decltype(rounds_after)::value;
    if (full) sm_wait_vmcnt<A * kQ6ReqMax>();
    else sm_wait_vmcnt<A * (kQ6ReqMax - 1)>();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // One round is requested now, the others once the plane table is built: a compute unit takes about 64 KiB of
  // outstanding requests, and a wavefront that asks for more sits in the request until earlier ones have landed --
  // with the activations still unprocessed behind it.
  request_next();

  // ---- the raw activations back into registers, then into the two byte planes
  wait_rounds(I1{});
  // Long rows: the activations have landed, and their share of what the compute unit has in flight goes to a
  // second round (measured on short rows, whose activations are a quarter of a round: slower by 0.2 - 0.4 us).
  constexpr int kEarlyRounds = RPG == 0 && kBufs > 2 ? 2 : 1;
  if (kEarlyRounds > 1 && 1 < nrounds) request_next();
  if (tid < 4) reinterpret_cast<uint32_t*>(&xa[CFG::NBMAX * 32])[tid] = 0u;
#pragma unroll
  for (int i = 0; i < kXPasses; i++) {
    const int k0 = 8 * tid + i * (8 * kQ6Threads);
    if (k0 >= n_in) break;
    float xf[8];
    const sm_u32x4 r = sm_read16(sm_lds(xstage) + (uint32_t)(i * (16 * kQ6Threads) + tid * 16));
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
    uint2* xa8 = reinterpret_cast<uint2*>(&xa[0]);
    const int e = (k0 >> 4) * 4 + ((k0 >> 3) & 1);
    xa8[e] = make_uint2(pack_bytes1(vb[0] + 128u, vb[1] + 128u, vb[2] + 128u, vb[3] + 128u),
                        pack_bytes1(vb[4] + 128u, vb[5] + 128u, vb[6] + 128u, vb[7] + 128u));
    xa8[e + 2] = make_uint2(pack_low_bytes((int)vb[0], (int)vb[1], (int)vb[2], (int)vb[3]),
                            pack_low_bytes((int)vb[4], (int)vb[5], (int)vb[6], (int)vb[7]));
    // the weights arrive as 4 * (q - 32): a quarter of the scale; the high plane counts 256
    if ((tid & 7) == 0) {
      fac[(k0 >> 6) * 2] = f * 64.f;
      fac[(k0 >> 6) * 2 + 1] = f * 0.25f;
    }
  }

  // ---- per-lane constants of the main loop
  // weight operand: row n, values 16 g .. 16 g + 15 of the k-set: ql bytes 16 g, qh bytes 16 (g % 2), bit pair
  // g / 2 (low nibbles) or 2 + g / 2 (high nibbles)
  const uint32_t sh1 = 6u - 2u * (uint32_t)(g >> 1), sh2 = 2u - 2u * (uint32_t)(g >> 1);
  // chunk c of row n's slots, as a byte offset into the buffer
  auto chunk_at = [&](int c) {
    const int pos = c + n < kQ6RowChunks ? c + n : c + n - kQ6RowChunks;
    return (uint32_t)((n * kQ6RowChunks + pos) * 16);
  };
  const int slot = wave * kQ6SlotChunks;                   // the wavefront's block of the round
  // activation operand: lane (i, g) of the first MFMA holds something only if i < 8 and i % 4 == g, of the
  // second only if i >= 8 and i % 4 == g; plane (i / 4) % 2.  Unit u = 2 block + half starts at value 128 u.
  const uint32_t xa_base = sm_lds(&xa[0]);
  const uint32_t zero_entry = xa_base + (uint32_t)(CFG::NBMAX * 32 * 16);
  const bool mine = (n & 3) == g;
  const uint32_t plane16 = (uint32_t)(((n >> 2) & 1) * 16);
  const bool act1 = mine && n < 8, act2 = mine && n >= 8;
  const uint32_t u0 = (uint32_t)(2 * wave);                // the wavefront's first unit of a group's first round
  const uint32_t a1_addr = act1 ? xa_base + 256u * u0 + 32u * (uint32_t)g + plane16 : zero_entry;
  const uint32_t a2_addr = act2 ? xa_base + 256u * u0 + 128u + 32u * (uint32_t)g + plane16 : zero_entry;
  // per unit 256 bytes of table, per round 16 units
  const uint32_t a1_step = act1 ? 256u : 0u, a2_step = act2 ? 256u : 0u;
  const uint32_t fac_addr0 = sm_lds(&fac[0]) + 16u * u0 + 4u * (uint32_t)g;
  const uint32_t wbuf_base = sm_lds(wbuf);

  sm_barrier();                         // the plane table is complete
#pragma unroll
  for (int i = kEarlyRounds; i < kBufs; i++)
    if (i < nrounds) request_next();

  const uint32_t part_addr = sm_lds(&part[0][0][0]) + (uint32_t)((wave * 16 + n) * 4);
  // ODD: the wavefront's blocks sit two bytes into their slots
  auto run_rounds = [&](auto oddc) {
    constexpr bool ODD = decltype(oddc)::value;
    // unit hf (half of the block): ql chunk 4 hf + g, qh chunk 8 + 2 hf + g % 2 (plus the first dword of the
    // chunk after it when the block is shifted); scales in chunk 12 (accumulator lane (n, g): row n, k-set
    // g / 2, plane g % 2; its four scales are consecutive bytes); d near the end of chunk 13
    const uint32_t ql_off0 = chunk_at(slot + g), ql_off1 = chunk_at(slot + 4 + g);
    const uint32_t qh_off0 = chunk_at(slot + 8 + (g & 1)), qh_off1 = chunk_at(slot + 10 + (g & 1));
    const uint32_t qlx_off0 = chunk_at(slot + g + 1), qlx_off1 = chunk_at(slot + 4 + g + 1);
    const uint32_t qhx_off0 = chunk_at(slot + 8 + (g & 1) + 1), qhx_off1 = chunk_at(slot + 10 + (g & 1) + 1);
    const uint32_t sc_off = chunk_at(slot + 12) + (uint32_t)(4 * (g >> 1));
    // shifted: the dword after the scales' (for the last one of the block that is byte 12 of chunk 13, which holds
    // the block's bytes 194..209)
    const uint32_t scx_off0 = sc_off + 4u;
    const uint32_t scx_off1 = (g >> 1) ? chunk_at(slot + 13) + 12u : sc_off + 12u;
    const uint32_t d_off = chunk_at(slot + 13) + (uint32_t)(kQ6DAt + (ODD ? 2 : 0));

    // a unit's weights, and its activations: the two operands and the scale of the sums
    struct Regs { sm_u32x4 ql, qh; uint32_t sc, d, qlx, qhx, scx; };
    struct Acts { sm_u32x4 a1, a2; uint32_t f; };
    // unit ui of a group (16 to a round)
    auto issue_acts = [&](uint32_t ui, Acts& t) {
      if constexpr (STAGE >= 2) return;
      const uint32_t x1 = a1_addr + ui * a1_step, x2 = a2_addr + ui * a2_step;
      const uint32_t fa = fac_addr0 + 16u * ui;
      asm volatile(
          "ds_read_b128 %0, %3\n\t"
          "ds_read_b128 %1, %4\n\t"
          "ds_read_b32 %2, %5"
          : "=&v"(t.a1), "=&v"(t.a2), "=&v"(t.f)
          : "v"(x1), "v"(x2), "v"(fa)
          : "memory");
    };
    // (behind a wait) the registers hold what was read
    auto settle_acts = [&](Acts& t) {
      if constexpr (STAGE >= 2) return;
      asm volatile("" : "+v"(t.a1), "+v"(t.a2), "+v"(t.f));
    };
    // unit hf of the round in `buf`
    auto issue = [&](auto hc, uint32_t buf, Regs& r) {
      constexpr int hf = decltype(hc)::value;
      const uint32_t a_ql = buf + (hf ? ql_off1 : ql_off0), a_qh = buf + (hf ? qh_off1 : qh_off0);
      const uint32_t a_sc = buf + sc_off, a_d = buf + d_off;
      if constexpr (STAGE >= 2) return;
      asm volatile(
          "ds_read_b128 %0, %4\n\t"
          "ds_read_b128 %1, %5\n\t"
          "ds_read_b32 %2, %6 offset:%8\n\t"
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
    constexpr int kReads = 4 + (ODD ? 3 : 0) + (RPG > 0 ? 0 : 3);   // LDS reads of a unit
    auto settle = [&](auto pending, Regs& r) {
      constexpr int P = decltype(pending)::value;
      if constexpr (STAGE >= 2) return;
      asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r.ql), "+v"(r.qh), "+v"(r.sc), "+v"(r.d) : "n"(P) : "memory");
      if constexpr (ODD) asm volatile("" : "+v"(r.qlx), "+v"(r.qhx), "+v"(r.scx));
    };
    float acc = 0.f;
    auto compute = [&](const Regs& r, const Acts& t) {
      if constexpr (STAGE >= 1) return;
      uint32_t ql[4], qh[4], sc4;
      if constexpr (ODD) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          ql[i] = __builtin_amdgcn_alignbit(i < 3 ? r.ql[i + 1] : r.qlx, r.ql[i], 16);
          qh[i] = __builtin_amdgcn_alignbit(i < 3 ? r.qh[i + 1] : r.qhx, r.qh[i], 16);
        }
        sc4 = __builtin_amdgcn_alignbit(r.scx, r.sc, 16);
      } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          ql[i] = r.ql[i];
          qh[i] = r.qh[i];
        }
        sc4 = r.sc;
      }
      v4i_t B1, B2, A1, A2;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        // 4 * (q - 32) as a signed byte: nibble into bits 2-5, bit pair into bits 6-7, low bits cleared and
        // the top bit flipped
        const uint32_t t1 = ((ql[i] << 2) & 0x3C3C3C3Cu) | ((qh[i] << sh1) & ~0x3C3C3C3Cu);
        const uint32_t t2 = ((ql[i] >> 2) & 0x3C3C3C3Cu) | ((qh[i] << sh2) & ~0x3C3C3C3Cu);
        B1[i] = (int)((t1 & 0xFCFCFCFCu) ^ 0x80808080u);
        B2[i] = (int)((t2 & 0xFCFCFCFCu) ^ 0x80808080u);
        A1[i] = (int)t.a1[i];
        A2[i] = (int)t.a2[i];
      }
      const v4i_t zero = {0, 0, 0, 0};
      v4i_t C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, B1, zero, 0, 0, 0);
      C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A2, B2, C, 0, 0, 0);
      const int sc = (int)sc4;
      // 24-bit multiplies (full rate; a 32-bit one takes four times as long): |C| <= 16 * 128 * 128
      int ts = __mul24((int)(int8_t)(sc & 0xFF), C[0]);
      ts += __mul24((int)(int8_t)((sc >> 8) & 0xFF), C[1]);
      ts += __mul24((int)(int8_t)((sc >> 16) & 0xFF), C[2]);
      ts += __mul24(sc >> 24, C[3]);
      const float d = f16_bits_to_f32((uint16_t)(r.d & 0xFFFFu));
      acc = fmaf_((float)ts * __uint_as_float(t.f), d, acc);
      // pins the arithmetic here: left alone the compiler moves it behind later waits
      asm volatile("" : "+v"(acc));
    };

    using U0 = std::integral_constant<int, 0>;
    using U1 = std::integral_constant<int, 1>;
    // One row length (RPG rounds to a group, known at compile time): the wavefront's place in a group's rounds
    // never changes, so neither do the activations it multiplies: they stay in registers for all its groups.
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
      if (later == 3) wait_rounds(I3{});
      else if (later == 2) wait_rounds(I2{});
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
    // the four accumulator lanes of a row -> the wavefront's sums, set `slot`
    auto leave_sums = [&](int slot) {
      acc = add_xor16(acc);
      acc = add_xor32(acc);
      if (lane < 16) sm_write_f32(part_addr + (uint32_t)(slot * (kQ6Waves * 16 * 4)), acc);
      acc = 0.f;
    };
    const bool per_round = fold_nb != 0;
    for (int gi = 0; gi < ng; gi++) {
      if constexpr (RPG > 0) {
#pragma unroll
        for (int kr = 0; kr < RPG; kr++) {
          round((uint32_t)kr, held[kr][0], held[kr][1]);
          if (per_round) leave_sums(gi * RPG + kr);
        }
      } else {
        for (int kr = 0; kr < rpg; kr++) {
          Acts ta, tb;
          round((uint32_t)kr, ta, tb);
          if (per_round) leave_sums(gi * rpg + kr);
        }
      }
      // the group is complete
      if (!per_round) leave_sums(gi);
    }
  };
  if (wave & 1) run_rounds(std::true_type{});
  else run_rounds(std::false_type{});
  // every request has landed (plain loads are safe again); the eight K-slices of a row add up in a fixed order
  __syncthreads();
  if (fold_log2 == 0) {
    for (int t = tid; t < ng * 16; t += kQ6Threads) {
      const int grp = t >> 4, nn = t & 15;
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < kQ6Waves; wv++) v += part[grp][wv][nn];
      const int row = (grp0 + grp) * 16 + nn;
      YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
    }
  } else if (fold_nb != 0) {
    // real row fs of streamed row nn: blocks fs * fold_nb ... of the streamed row; block b was wavefront b % 8's
    // in round b / 8
    for (int t = tid; t < (ng * 16) << fold_log2; t += kQ6Threads) {
      const int grp = t >> (4 + fold_log2), rem = t & ((16 << fold_log2) - 1);
      const int nn = rem >> fold_log2, fs = rem & ((1 << fold_log2) - 1);
      float v = 0.f;
      for (int b = fs * fold_nb; b < (fs + 1) * fold_nb; b++) v += part[grp * rpg + (b >> 3)][b & 7][nn];
      const int row = (((grp0 + grp) * 16 + nn) << fold_log2) + fs;
      YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
    }
  } else {
    // real row fs of streamed row nn: the blocks of wavefronts fs * (8 >> fold_log2) ...
    const int per = kQ6Waves >> fold_log2;
    for (int t = tid; t < (ng * 16) << fold_log2; t += kQ6Threads) {
      const int grp = t >> (4 + fold_log2), rem = t & ((16 << fold_log2) - 1);
      const int nn = rem >> fold_log2, fs = rem & ((1 << fold_log2) - 1);
      float v = 0.f;
      for (int wv = fs * per; wv < (fs + 1) * per; wv++) v += part[grp][wv][nn];
      const int row = (((grp0 + grp) * 16 + nn) << fold_log2) + fs;
      YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
    }
  }
}

// Which shape of the kernel takes (n_out, n_in), with how many workgroups; ok == false: neither.
// rpg: 1 or 2 for rows of 2048 or 4096 values (the kernels built for one row length), else 0.
// fold_log2: rows of 1024 / 512 / 256 values are streamed two / four / eight at a time as rows of 2048.
// fold_nb: other row lengths that are not whole rounds (fold_nb blocks): 8 / gcd(fold_nb, 8) rows at a time.
struct Q6Plan { bool ok, head; int num_wg, rpg, fold_log2, fold_nb; };
inline Q6Plan q6_plan(int64_t n_out, int64_t n_in) {
  Q6Plan p{false, false, 0, 0, 0, 0};
  if (n_in == 1024 || n_in == 512 || n_in == 256) {
    p.fold_log2 = n_in == 1024 ? 1 : (n_in == 512 ? 2 : 3);
    if (n_out % (16 << p.fold_log2) != 0) return p;
    n_out >>= p.fold_log2;
    n_in = 2048;
  } else if (n_in % 256 == 0 && n_in % 2048 != 0 && n_in > 0) {
    const int64_t nbr = n_in / 256;
    p.fold_log2 = nbr % 4 == 0 ? 1 : (nbr % 2 == 0 ? 2 : 3);
    if (n_out % (16 << p.fold_log2) != 0 || (nbr << p.fold_log2) > Q6Wide::NBMAX) {
      p.fold_log2 = 0;
      return p;
    }
    p.fold_nb = (int)nbr;
    n_out >>= p.fold_log2;
    n_in <<= p.fold_log2;
  }
  const int64_t nb = n_in / 256;
  // whole rounds of eight blocks, whole groups of 16 rows, 32-bit byte offsets into the weight buffer
  if (n_in % (256 * kQ6RoundBlocks) != 0 || nb > Q6Wide::NBMAX || n_out % 16 != 0) return p;
  if (n_out * nb * 210 >= ((int64_t)1 << 32)) return p;
  const int64_t groups = n_out / 16;
  const int cus = device_num_cus();
  if (groups < cus) return p;                              // a group or more for every compute unit
  // between one and two groups per compute unit the uneven ones decide (6144x4096: 7.9 us against 7.7 of the
  // packed-dot kernel, which deals rows out more finely)
  if (groups < 2 * cus && groups % cus != 0) return p;
  p.rpg = nb <= 16 ? (int)(nb / 8) : 0;
  int maxg;
  if (nb == Q6Head::NBMAX && groups >= 2 * (int64_t)Q6Head::WGS * cus) {
    // two workgroups per compute unit when each still gets two groups: their rounds interleave
    p.head = true;
    p.num_wg = Q6Head::WGS * cus;
    maxg = Q6Head::MAXG;
  } else {
    p.num_wg = cus;
    maxg = Q6Wide::MAXG;
  }
  if (p.fold_nb) maxg /= (int)(nb / 8);                    // sums are kept per round there
  // more groups than one workgroup per slot keeps sums for: whole waves of workgroups (a last wave with a few
  // workgroups in it would take as long as a full one)
  if ((groups + p.num_wg - 1) / p.num_wg > maxg) p.num_wg *= (int)((groups + (int64_t)p.num_wg * maxg - 1) / ((int64_t)p.num_wg * maxg));
  p.ok = true;
  return p;
}

template <typename XT, typename YT, int STAGE = 0>
inline hipError_t q6_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                        int64_t n_in, hipStream_t s) {
  const Q6Plan p = q6_plan(n_out, n_in);
  if (!p.ok) return hipErrorInvalidValue;
  // (folded rows: the kernel sees the streamed shape)
  const int64_t rows = n_out >> p.fold_log2, nb = (n_in << p.fold_log2) / 256;
  const int groups = (int)(rows / 16);
  const dim3 grid((unsigned)p.num_wg, (unsigned)m), block(kQ6Threads);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)rows, (int)nb, groups / p.num_wg,
                       groups % p.num_wg, p.fold_log2, p.fold_nb);
  };
  if (p.head) go(gemv_q6k_stream_kernel<XT, YT, Q6Head, STAGE>);
  else if (p.rpg == 1) go(gemv_q6k_stream_kernel<XT, YT, Q6Short<1>, STAGE>);
  else if (p.rpg == 2) go(gemv_q6k_stream_kernel<XT, YT, Q6Short<2>, STAGE>);
  else go(gemv_q6k_stream_kernel<XT, YT, Q6Wide, STAGE>);
  return hipGetLastError();
}

}  // namespace ttq
