// Decode GEMV for Q8_0 weights on gfx950: the weight stream goes HBM -> LDS as whole cache lines, exactly
// as it lies in memory, and feeds the int8 matrix cores without a single instruction spent on the weights.
//
// Operator: F.linear with a single-token activation (workspace/libtorch/src/abi/neural_nets.nim:64-81) over a
// weight stored as GGUF Q8_0 blocks { f16 d; i8 qs[32] } of 32 weights, w = d * qs[e].
//
// A block is 34 bytes: its weights start at 2 mod 4 in every other block, and no operand of 16 weights is
// aligned to anything.  Instead of moving the bytes, the K dimension of the MFMA is taken to be the raw byte
// string of the row: 64 consecutive bytes per v_mfma_i32_16x16x64_i8, 16 aligned bytes per lane, whatever
// they hold.  2048 weights are 64 blocks = 2176 bytes = 17 cache lines = 34 such MFMAs.  What makes this
// right is the activation operand: it is built once per launch in the same byte geometry -- at the position of
// weight e of block b the fixed-point value of x[32 b + e], at the position of a scale byte zero -- and it has one
// row per (block, byte plane): the 64 bytes of an MFMA touch at most three blocks, so six of its 16 rows are used,
// and two MFMAs (rows 0-7, rows 8-15) share an accumulator.  An accumulator lane then holds, for one weight
// row, the exact integer sums of up to two blocks and two planes, and finishes them with the blocks' d (read
// from the same landed bytes) and the blocks' power-of-two activation scale: d * (2^s * (256 hi + lo)), one
// rounding, which for a unit-vector activation is the canonical d * q bit for bit.  fp32 activations get three
// byte planes (23 bits: 1e-6 class instead of the 5e-5 of two planes on activations of uneven magnitude): nine operand
// rows per MFMA, no sharing of accumulators, the planes weighed in floating point.
//
// The stream is organized as in ttq_gemv_q6k_stream.hip: a round is 2048 weights of a group of 16 rows (16 runs of
// 17 whole lines), 34 requests of 1 KiB (global_load_lds_dwordx4) into one of three LDS buffers; a wavefront
// waits for its own requests on its own counter, a barrier makes the buffer whole, a second one frees it.
// Chunk c of row n lands at position 136 n + (c ^ (n / 2)): with the rows 8 chunks apart modulo 16, the 16 rows
// of an operand read hit 16 different bank groups.  Wavefront w multiplies MFMAs w, w + 8, ... of the round's 34.
#include "ttq_stream_common.h"

namespace ttq {

namespace {

constexpr int kQ8Waves = 8;
constexpr int kQ8Threads = kQ8Waves * 64;
constexpr int kQ8RoundBlocks = 64;                         // blocks of a row in one round: 2048 weights
constexpr int kQ8RoundBytes = kQ8RoundBlocks * 34;         // 2176 = 17 lines
constexpr int kQ8RowChunks = kQ8RoundBytes / 16;           // 136
constexpr int kQ8RoundMfma = kQ8RoundBytes / 64;           // 34
constexpr int kQ8Requests = 16 * kQ8RowChunks / 64;        // 34
constexpr int kQ8BufBytes = kQ8Requests * 1024;            // 34816
constexpr int kQ8Bufs = 3;
constexpr int kQ8ReqMax = (kQ8Requests + kQ8Waves - 1) / kQ8Waves;        // 5
constexpr int kQ8FullWaves = kQ8Requests - (kQ8ReqMax - 1) * kQ8Waves;    // wavefronts 0, 1: 5 requests and 5 MFMAs
constexpr int kQ8MaxRounds = 4;                            // rounds per row: n_in <= 8192
constexpr int kQ8MaxGroups = 32;                           // row groups of a workgroup; also 16 KiB of staging
constexpr int kQ8TableEntries = 2 * 4 * 136 * 2;            // the operand table: two planes x four rounds (or three x two) x 136 chunks x 2 entries

// eight activations of thread-owned positions k0 .. k0 + 7 from the staging area
template <typename XT> struct Q8Stage;
template <> struct Q8Stage<float> {
  static constexpr int kBytes = 32, kRequests = 2;
  static __device__ __forceinline__ void read(uint32_t a, uint32_t second, float (&f)[8]) {
    const sm_u32x4 r0 = sm_read16(a), r1 = sm_read16(a + second);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      f[i] = __uint_as_float(r0[i]);
      f[4 + i] = __uint_as_float(r1[i]);
    }
  }
};
template <typename XT> struct Q8Stage {
  static constexpr int kBytes = 16, kRequests = 1;
  static __device__ __forceinline__ void read(uint32_t a, uint32_t, float (&f)[8]) {
    const sm_u32x4 r = sm_read16(a);
    widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), f);
  }
};

// XT: float, bf16 or fp16 activations.  The row groups are dealt out in runs: the first groups_rem workgroups
// take groups_per_wg + 1 each, the others groups_per_wg.  rpg: rounds per row (n_in / 2048).
template <typename XT, typename YT>
__global__ void __launch_bounds__(kQ8Threads)
gemv_q8_stream_kernel(const uint8_t* __restrict__ w, const XT* __restrict__ x, YT* __restrict__ y,
                      const void* __restrict__ bias, int bias_dtype, int n_out, int rpg, int groups_per_wg,
                      int groups_rem) {
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kQ8Bufs * kQ8BufBytes];
  // the activation operand: per MFMA of the row 16 entries of 16 bytes; then 64 entries of zeros, one per lane
  // (lanes that all read one and the same entry are served one after the other: 1 us per launch)
  __shared__ __attribute__((aligned(16))) v4i_t xa[kQ8TableEntries + 64];
  __shared__ float ftab[kQ8MaxRounds * kQ8RoundBlocks];    // per block: the scale of its fixed-point activations
  // (the raw activations land here first: the partial sums are written after they have been read back)
  __shared__ __attribute__((aligned(1024))) float part[kQ8MaxGroups][kQ8Waves][16];
  static_assert(sizeof(part) >= 16384, "room for the staged activations");
  uint8_t* xstage = reinterpret_cast<uint8_t*>(&part[0][0][0]);

  // Byte planes of the activations.  The operand table is plane-major: per plane and 16-byte chunk of a row two
  // entries of 16 bytes (the chunk's first and second block), so that neighbouring threads of the scatter and
  // neighbouring lanes of an operand read are 32 bytes apart.
  constexpr int kPlanes = std::is_same<XT, float>::value ? 3 : 2;
  constexpr int kRoundTable = kQ8RowChunks * 2 * 16;      // bytes of one plane of one round: 4352
  const int n_in = rpg * 2048;
  const uint32_t plane_bytes = (uint32_t)(rpg * kRoundTable);
  const uint32_t row_bytes = (uint32_t)rpg * (uint32_t)kQ8RoundBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const XT* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const int bx = blockIdx.x;
  const int grp0 = bx * groups_per_wg + min(bx, groups_rem);
  const int ng = groups_per_wg + (bx < groups_rem ? 1 : 0);            // 1 .. kQ8MaxGroups
  const int nrounds = rpg * ng;

  // ---- the activations, as LDS requests too (a register load among the weight requests would make the
  // compiler wait for all of them at its first use): thread t stages x[8 t + 4096 i .. + 7]
  using ST = Q8Stage<XT>;
  constexpr int kXPasses = 16384 / (ST::kBytes * kQ8Threads);          // 2 (16-bit) or 1 (float) passes of 4096 values
  constexpr int kPassBytes = ST::kBytes * kQ8Threads;
#pragma unroll
  for (int i = 0; i < kXPasses; i++) {
    const int k0 = 8 * tid + i * (8 * kQ8Threads);
    if (k0 < n_in) {                                      // whole wavefronts: n_in is a multiple of 512
      const uint8_t* src = reinterpret_cast<const uint8_t*>(xm + k0);
#pragma unroll
      for (int r = 0; r < ST::kRequests; r++)
        __builtin_amdgcn_global_load_lds((sm_gptr_t)(src + 16 * r),
                                         (sm_lptr_t)(xstage + i * kPassBytes + r * (16 * kQ8Threads) + wave * 1024), 16, 0, 0);
    }
  }
  // a compute unit serves its requests in the order they were made: every wavefront's activation requests are
  // queued before any weight request of the workgroup
  asm volatile("s_barrier" ::: "memory");

  // ---- requests of a round: request q = wave + 8 i fills LDS chunks 64 q .. 64 q + 63 of the buffer
  uint32_t src_off[kQ8ReqMax];
#pragma unroll
  for (int i = 0; i < kQ8ReqMax; i++) {
    const int p = min(64 * (wave + kQ8Waves * i) + lane, 16 * kQ8RowChunks - 1);
    const int row = p / kQ8RowChunks, pos = p - row * kQ8RowChunks;
    src_off[i] = (uint32_t)row * row_bytes + (uint32_t)((pos ^ (row >> 1)) * 16);
  }
  const bool full = wave < kQ8FullWaves;
  // rounds are requested in order: group by group, 2048 weights by 2048 weights
  // (every workgroup has a group; a workgroup without one would ask for the matrix's last group: never past the end,
  // and without a branch around the request, after which the compiler waits for every request in flight)
  uint32_t req_src = (uint32_t)min(grp0, n_out / 16 - 1) * 16u * row_bytes;    // byte offset of the next round to request
  int req_kr = 0, req_buf = 0;
  auto request_next = [&]() {
    const uint8_t* src = w + (size_t)req_src;
    uint8_t* dst = wbuf + req_buf * kQ8BufBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kQ8ReqMax - 1; i++)
      __builtin_amdgcn_global_load_lds((sm_gptr_t)(src + src_off[i]), (sm_lptr_t)(dst + i * (kQ8Waves * 1024)), 16, 0, 2);
    if (full)
      __builtin_amdgcn_global_load_lds((sm_gptr_t)(src + src_off[kQ8ReqMax - 1]),
                                       (sm_lptr_t)(dst + (kQ8ReqMax - 1) * (kQ8Waves * 1024)), 16, 0, 2);
    req_buf = req_buf == kQ8Bufs - 1 ? 0 : req_buf + 1;
    req_kr++;
    req_src += kQ8RoundBytes;
    if (req_kr == rpg) {
      req_kr = 0;
      req_src += 15u * row_bytes;
    }
  };
  // all but the youngest `rounds_after` rounds of requests of this wavefront have landed
  auto wait_rounds = [&](int rounds_after) {
    if (full) {
      if (rounds_after >= 3) sm_wait_vmcnt<3 * kQ8ReqMax>();
      else if (rounds_after == 2) sm_wait_vmcnt<2 * kQ8ReqMax>();
      else if (rounds_after == 1) sm_wait_vmcnt<kQ8ReqMax>();
      else sm_wait_vmcnt<0>();
    } else {
      if (rounds_after >= 3) sm_wait_vmcnt<3 * (kQ8ReqMax - 1)>();
      else if (rounds_after == 2) sm_wait_vmcnt<2 * (kQ8ReqMax - 1)>();
      else if (rounds_after == 1) sm_wait_vmcnt<kQ8ReqMax - 1>();
      else sm_wait_vmcnt<0>();
    }
  };
  // One round is requested now, the others once the operand table is built (asking right after the activations
  // have landed, before the table is written, was measured 0.6 us slower): a compute unit takes about 64 KiB
  // of outstanding requests, and a wavefront that asks for more sits in the request until earlier ones have
  // landed -- with the activations still unprocessed behind it.
  const int npre = min(nrounds, kQ8Bufs);
  request_next();

  // ---- the operand table starts as zeros (scale bytes, other blocks' bytes, rows nobody uses)
  {
    uint4* z = reinterpret_cast<uint4*>(&xa[0]);
    const int entries = kPlanes * rpg * (kRoundTable / 16) + 64;
    for (int i = tid; i < entries; i += kQ8Threads) z[i] = make_uint4(0u, 0u, 0u, 0u);
  }
  // ---- per-lane constants of the main loop.  MFMA t2 of a round (0..33) covers bytes 64 t2 .. 64 t2 + 63 of the
  // round's 2176; the wavefront takes t2 = wave + 8 i.  Operand lane (r, g): weight row n = r, k-group g (weights)
  // or selector row r, k-group g (activations).  Selector row r of the i-th MFMA of a wavefront is used if
  // r / 8 == i % 2; it stands for block j0 + (r % 8) / 2 (j0: the first block with bytes in the MFMA) and plane r % 2.
  const uint32_t key = (uint32_t)(n >> 1);
  const uint32_t row_base = (uint32_t)(n * kQ8RoundBytes);
  const uint32_t xa_base = sm_lds(&xa[0]);
  // accumulators: with two planes two MFMAs share one (operand rows 0-7 and 8-15), with three every MFMA has its own
  constexpr int kAccs = kPlanes == 3 ? kQ8ReqMax : (kQ8ReqMax + 1) / 2;
  uint32_t b_off[kQ8ReqMax], a_off[kQ8ReqMax];             // per MFMA of the wavefront: weight and activation operand
  bool a_used[kQ8ReqMax];
#pragma unroll
  for (int i = 0; i < kQ8ReqMax; i++) {
    const int t2 = min(wave + kQ8Waves * i, kQ8RoundMfma - 1);
    b_off[i] = row_base + ((((uint32_t)(4 * t2 + g)) ^ key) << 4);
    const int j0 = (64 * t2) / 34;                         // the first block with bytes in this MFMA
    // selector row n: block j0 + lb, plane
    const int lb = kPlanes == 3 ? n / 3 : (n & 7) >> 1, plane = kPlanes == 3 ? n - 3 * (n / 3) : n & 1;
    const bool row_used = kPlanes == 3 ? n < 9 : (n >> 3) == (i & 1);
    const int c = 4 * t2 + g, first = (16 * c) / 34;       // the first block with bytes in this lane's chunk
    const int s = j0 + lb - first;
    a_used[i] = row_used && (s == 0 || s == 1) && j0 + lb < kQ8RoundBlocks;
    a_off[i] = (uint32_t)((c * 2 + (s & 1)) * 16) + (uint32_t)plane * plane_bytes;
  }
  // Accumulator lane (n, g) holds operand rows 4 g .. 4 g + 3 of its accumulator.
  //   two planes:   MFMA 2 a + g / 2 of the wavefront, blocks j0 + 2 (g % 2) + {0, 1}, planes {high, low} each
  //   three planes: MFMA a, rows r = 4 g + v -> block j0 + r / 3, plane r % 3 (r < 9): two blocks, A = the block of
  //                 v = 0 and B = the next one
  // (Blocks and MFMAs that do not exist have zero sums; their addresses are clamped to ones that do.)
  uint32_t d_off[kAccs][2], f_off[kAccs][2];
#pragma unroll
  for (int a = 0; a < kAccs; a++) {
    const int i = kPlanes == 3 ? a : min(2 * a + (g >> 1), kQ8ReqMax - 1);
    const int t2 = min(wave + kQ8Waves * i, kQ8RoundMfma - 1);
    const int j0 = (64 * t2) / 34;
    const int lb0 = kPlanes == 3 ? (4 * g) / 3 : 2 * (g & 1);
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int jb = min(j0 + lb0 + e, kQ8RoundBlocks - 1);
      const int P = 34 * jb;                               // d: the block's first two bytes
      d_off[a][e] = row_base + ((((uint32_t)(P >> 4)) ^ key) << 4) + (uint32_t)(P & 15);
      f_off[a][e] = (uint32_t)(4 * jb);
    }
  }
  // three planes: the weight of accumulator value v for block A / block B: 2^16, 2^8, 1 by plane, 0 where the
  // value belongs to the other block or to no operand row
  float pw_a[4], pw_b[4];
#pragma unroll
  for (int v = 0; v < 4; v++) {
    const int r = 4 * g + v, lbv = r / 3, pl = r - 3 * lbv;
    const float pwv = r < 9 ? (pl == 0 ? 65536.f : (pl == 1 ? 256.f : 1.f)) : 0.f;
    const bool is_b = lbv != (4 * g) / 3;
    pw_a[v] = is_b ? 0.f : pwv;
    pw_b[v] = is_b ? pwv : 0.f;
  }
  const uint32_t zero_entry = xa_base + (uint32_t)kPlanes * plane_bytes + (uint32_t)(lane * 16);
  const uint32_t ftab_base = sm_lds(&ftab[0]);
  const uint32_t wbuf_base = sm_lds(wbuf);
  const uint32_t part_addr = sm_lds(&part[0][0][0]) + (uint32_t)((wave * 16 + n) * 4);
  const int nmf = full ? kQ8ReqMax : kQ8ReqMax - 1;        // MFMAs of this wavefront per round

  // ---- the raw activations back into registers (they were requested before any weight, and the lane constants
  // above were computed while they were on their way), then pair by pair into the operand table: weight e of
  // block b sits at byte 34 b + 2 + e of the row = byte P % 16 of chunk P / 16; MFMA = chunk / 4, k-group =
  // chunk % 4, and the block is the first (0) or second (1) one that has bytes in this chunk
  sm_barrier();                         // the table is all zeros
  wait_rounds(1);
  {
#pragma unroll
    for (int i = 0; i < kXPasses; i++) {
      const int k0 = 8 * tid + i * (8 * kQ8Threads);
      if (k0 >= n_in) break;
      float xf[8];
      ST::read(sm_lds(xstage) + (uint32_t)(i * kPassBytes + tid * 16), 16u * kQ8Threads, xf);
      uint32_t amax = amax_bits(xf);
      // the four threads of a block are an aligned quad
      amax = umax(amax, dpp_quad_u32<0xB1>(amax));
      amax = umax(amax, dpp_quad_u32<0x4E>(amax));
      const uint32_t eb = amax >> 23;                        // biased exponent of max |x|; 255 for Inf and NaN
      // |v| < 2^(S+1) with S = 13 (two planes) or 21 (three); the scale 2^(E-S) stays a normal number
      constexpr uint32_t kS = kPlanes == 3 ? 21u : 13u;
      const uint32_t ec = eb < kS + 5u ? kS + 5u : eb;
      const float mul = __uint_as_float((254u + kS - ec) << 23);   // 2^(S-E)
      // non-finite activations poison their block instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - kS) << 23);
      const int b = k0 >> 5;
      if ((tid & 3) == 0) ftab[b] = f;
      // the thread's eight bytes start at byte P0 of the row and lie in chunk c0 or the one after it
      const int P0 = 34 * b + 2 + (k0 & 31), c0 = P0 >> 4, e0 = P0 & 15;
      const int base0 = ((c0 * 2 + (b - (16 * c0) / 34)) * 16) + e0;
      const int base1 = (((c0 + 1) * 2 + (b - (16 * (c0 + 1)) / 34)) * 16) + e0 - 16;
      // (e0 is even: the eight bytes are four aligned pairs, none of which straddles a chunk)
      uint16_t* xa16 = reinterpret_cast<uint16_t*>(&xa[0]);
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const int at = ((e0 + j < 16 ? base0 : base1) + j) >> 1;
        int pl[2][3];
#pragma unroll
        for (int h = 0; h < 2; h++) {
          // v = 256 (256 high + mid) + low with signed bytes; two planes: v = 256 high + low
          const int v = (int)rintf(xf[j + h] * mul);
          const int lo = (int)(int8_t)(v & 0xFF), v1 = (v - lo) >> 8;
          const int mid = (int)(int8_t)(v1 & 0xFF);
          pl[h][0] = kPlanes == 3 ? (v1 - mid) >> 8 : v1;
          pl[h][1] = kPlanes == 3 ? mid : lo;
          pl[h][2] = lo;
        }
#pragma unroll
        for (int q = 0; q < kPlanes; q++)
          xa16[at + q * (int)(plane_bytes >> 1)] = (uint16_t)((pl[0][q] & 0xFF) | ((pl[1][q] & 0xFF) << 8));
      }
    }
  }

  sm_barrier();                         // the operand table is complete
  for (int i = 1; i < npre; i++) request_next();
  // (from here on the staging area is `part`)

  float acc = 0.f;
  int bufi = 0, kr = 0, gi = 0;
  for (int rr = 0; rr < nrounds; rr++) {
    const uint32_t buf = wbuf_base + (uint32_t)(bufi * kQ8BufBytes);
    const uint32_t xa_round = xa_base + (uint32_t)(kr * kRoundTable);
    const uint32_t f_round = ftab_base + (uint32_t)(kr * (kQ8RoundBlocks * 4));
    // every operand of the round in one go, at most five MFMAs.  What does not depend on the landed bytes -- the
    // activation operands and scales -- is asked for first, before the wait for the buffer
    sm_u32x4 bw[kQ8ReqMax], aw[kQ8ReqMax];
    uint32_t dd[kAccs][2], ff[kAccs][2];
#pragma unroll
    for (int i = 0; i < kQ8ReqMax; i++) {
      const uint32_t aa = a_used[i] ? xa_round + a_off[i] : zero_entry;
      asm volatile("ds_read_b128 %0, %1" : "=&v"(aw[i]) : "v"(aa) : "memory");
    }
#pragma unroll
    for (int p = 0; p < kAccs; p++) {
      const uint32_t fa0 = f_round + f_off[p][0], fa1 = f_round + f_off[p][1];
      asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %3" : "=&v"(ff[p][0]), "=&v"(ff[p][1]) : "v"(fa0), "v"(fa1) : "memory");
    }
    // the round's buffer: own requests landed, then everybody's
    wait_rounds(min(nrounds - 1 - rr, kQ8Bufs - 1));
    sm_barrier();
#pragma unroll
    for (int i = 0; i < kQ8ReqMax; i++) {
      const uint32_t ab = buf + b_off[i];
      asm volatile("ds_read_b128 %0, %1" : "=&v"(bw[i]) : "v"(ab) : "memory");
    }
#pragma unroll
    for (int p = 0; p < kAccs; p++) {
      const uint32_t da0 = buf + d_off[p][0], da1 = buf + d_off[p][1];
      asm volatile("ds_read_u16 %0, %2\n\tds_read_u16 %1, %3" : "=&v"(dd[p][0]), "=&v"(dd[p][1]) : "v"(da0), "v"(da1) : "memory");
    }
    // all of them have arrived (the asm statements tie every register to the wait)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < kQ8ReqMax; i++) asm volatile("" : "+v"(bw[i]), "+v"(aw[i]));
#pragma unroll
    for (int p = 0; p < kAccs; p++) asm volatile("" : "+v"(dd[p][0]), "+v"(dd[p][1]), "+v"(ff[p][0]), "+v"(ff[p][1]));
    // every wavefront has read what it needs of the buffer: a later round may land there
    sm_barrier();
    if (rr + kQ8Bufs < nrounds) request_next();
    bufi = bufi == kQ8Bufs - 1 ? 0 : bufi + 1;
    if constexpr (kPlanes == 3) {
#pragma unroll
      for (int a = 0; a < kAccs; a++) {
        if (a >= nmf) break;
        const v4i_t zero = {0, 0, 0, 0};
        v4i_t A0, B0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          A0[q] = (int)aw[a][q];
          B0[q] = (int)bw[a][q];
        }
        const v4i_t C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, B0, zero, 0, 0, 0);
        // exact integers, weighed by plane in floating point (a sum of one term is exact)
        float ta = 0.f, tb = 0.f;
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const float cf = (float)C[v];
          ta = fmaf_(cf, pw_a[v], ta);
          tb = fmaf_(cf, pw_b[v], tb);
        }
        acc = fmaf_(ta * __uint_as_float(ff[a][0]), f16_bits_to_f32((uint16_t)(dd[a][0] & 0xFFFFu)), acc);
        acc = fmaf_(tb * __uint_as_float(ff[a][1]), f16_bits_to_f32((uint16_t)(dd[a][1] & 0xFFFFu)), acc);
      }
    } else {
#pragma unroll
      for (int p = 0; p < kAccs; p++) {
        if (2 * p >= nmf) break;
        const v4i_t zero = {0, 0, 0, 0};
        v4i_t A0, B0, A1, B1;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          A0[q] = (int)aw[2 * p][q];
          B0[q] = (int)bw[2 * p][q];
          A1[q] = (int)aw[2 * p + 1 < kQ8ReqMax ? 2 * p + 1 : 2 * p][q];
          B1[q] = (int)bw[2 * p + 1 < kQ8ReqMax ? 2 * p + 1 : 2 * p][q];
        }
        v4i_t C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, B0, zero, 0, 0, 0);
        if (2 * p + 1 < nmf) C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, B1, C, 0, 0, 0);
        // exact integers; d * (2^s * sum), one rounding per block
        const float t0 = (float)(C[0] * 256 + C[1]) * __uint_as_float(ff[p][0]);
        const float t1 = (float)(C[2] * 256 + C[3]) * __uint_as_float(ff[p][1]);
        acc = fmaf_(t0, f16_bits_to_f32((uint16_t)(dd[p][0] & 0xFFFFu)), acc);
        acc = fmaf_(t1, f16_bits_to_f32((uint16_t)(dd[p][1] & 0xFFFFu)), acc);
      }
    }
    if (++kr == rpg) {
      // the group is complete: the four accumulator lanes of a row
      acc = add_xor16(acc);
      acc = add_xor32(acc);
      if (lane < 16) sm_write_f32(part_addr + (uint32_t)(gi * (kQ8Waves * 16 * 4)), acc);
      acc = 0.f;
      kr = 0;
      gi++;
    }
  }
  // every request has landed (plain loads are safe again); the eight wavefronts' sums of a row add up in a fixed order
  __syncthreads();
  for (int t = tid; t < ng * 16; t += kQ8Threads) {
    const int grp = t >> 4, nn = t & 15;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < kQ8Waves; wv++) v += part[grp][wv][nn];
    const int row = (grp0 + grp) * 16 + nn;
    YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
  }
}

// How many workgroups take (n_out, n_in); 0: the kernel does not take the shape.
int q8_plan(int x_dtype, int64_t n_out, int64_t n_in) {
  // whole rounds of 2048 weights, whole groups of 16 rows, tables and staging within LDS, 32-bit byte offsets
  if (n_in % 2048 != 0 || n_in > 2048 * kQ8MaxRounds || n_out % 16 != 0) return 0;
  if (x_dtype == kF32 && n_in > 4096) return 0;           // three planes: twice the operand table; 16 KiB of staging
  if (n_out * (n_in / 32) * 34 >= ((int64_t)1 << 32)) return 0;
  const int64_t groups = n_out / 16;
  const int cus = device_num_cus();
  if (groups < cus) return 0;                              // a group or more for every workgroup
  // fp32 activations, between one and two groups per compute unit: the uneven ones decide (6144x4096: 8.8 us against
  // 8.4 of the aligned-window kernel)
  if (x_dtype == kF32 && groups < 2 * cus && groups % cus != 0) return 0;
  int num_wg = cus;
  if ((groups + num_wg - 1) / num_wg > kQ8MaxGroups) num_wg = (int)((groups + kQ8MaxGroups - 1) / kQ8MaxGroups);
  return num_wg;
}

template <typename XT, typename YT>
hipError_t q8s_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                         int64_t n_in, int num_wg, hipStream_t s) {
  const int groups = (int)(n_out / 16);
  const dim3 grid((unsigned)num_wg, (unsigned)m), block(kQ8Threads);
  hipLaunchKernelGGL((gemv_q8_stream_kernel<XT, YT>), grid, block, 0, s, static_cast<const uint8_t*>(w),
                     static_cast<const XT*>(x), static_cast<YT*>(y), bias, bias_dtype, (int)n_out, (int)(n_in / 2048),
                     groups / num_wg, groups % num_wg);
  return hipGetLastError();
}

template <typename XT>
hipError_t q8s_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                        int64_t n_out, int64_t n_in, int num_wg, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q8s_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, num_wg, s);
    case kF16: return q8s_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, num_wg, s);
    case kBF16: return q8s_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, num_wg, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool gemv_q8_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  if (format != kQ8_0 || !(x_dtype == kF32 || x_dtype == kBF16 || x_dtype == kF16)) return false;
  return q8_plan(x_dtype, n_out, n_in) > 0;
}

hipError_t launch_gemv_q8_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  const int num_wg = q8_plan(x_dtype, n_out, n_in);
  if (num_wg <= 0) return hipErrorInvalidValue;
  if (x_dtype == kF32) return q8s_launch_x<float>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, num_wg, s);
  if (x_dtype == kBF16) return q8s_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, num_wg, s);
  if (x_dtype == kF16) return q8s_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, num_wg, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
