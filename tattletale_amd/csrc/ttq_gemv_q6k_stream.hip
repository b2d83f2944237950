// Decode GEMV for Q6_K weights on gfx950 with rows of 4096 values (the LM head of a "Q4_K_M" file):
// the weight stream goes HBM -> LDS as whole cache lines and feeds the int8 matrix cores.
//
// Operator: F.linear with a single-token activation (workspace/libtorch/src/abi/neural_nets.nim:64-81) over a
// weight stored as GGUF Q6_K blocks { u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d } of 256 weights,
// w = d * scale[e / 16] * (q6[e] - 32).
//
// A 210-byte block is neither a multiple of a cache line nor of a dword, so the per-wavefront line rings of the
// Q4_K kernel (ttq_gemv_q4k_stream.h) do not carry over.  What is line-shaped is a group of 16 rows: 53 760
// contiguous bytes = 420 lines.  So here the eight wavefronts of a workgroup share the stream:
//   * a round is half of K of one group of 16 rows: 16 runs of 1680 contiguous bytes, copied into one of three
//     LDS buffers by 28 requests of 1 KiB (global_load_lds_dwordx4, no registers), four or three per
//     wavefront.  On the way in every block is moved to a 16-byte boundary: it lands in a slot of 14 chunks
//     of 16 bytes, 13 fetched from consecutive addresses and one that ends with the block's last bytes, and
//     row n is rotated by n chunks, which puts the 16 rows of an operand read into 16 different bank groups.
//     Fetch addresses are rounded down to a dword: requests at 2 mod 4 were measured 15 % slower than
//     dword-aligned ones, and operand reads at 2 mod 4 -- which the packed layout would need for every other
//     block -- at three times the cost of the whole stream.  So an odd block lands two bytes into its slot,
//     and the wavefronts that multiply odd blocks (the odd ones: block = 8 * half + wavefront) shift their
//     operands by 16 bits in registers;
//   * while one buffer is multiplied, the next two rounds are in flight or landed (a compute unit takes about
//     64 KiB of outstanding requests); a wavefront waits for its own requests on its own counter, a barrier
//     makes the buffer whole, a second one frees it for the round three later;
//   * along K a round is split: wavefront w multiplies block w of the half for all 16 rows, two units of
//     16 rows x 128 weights, two v_mfma_i32_16x16x64_i8 each.
// Arithmetic.  The activations are block fixed point, 15 bits in two byte planes with one power-of-two scale
// per 64 values.  A weight reaches the matrix core as the signed byte 4 * (q6 - 32) = ((q6 << 2) ^ 0x80), built
// from the nibble and the bit pair with four instructions per dword.  The 16 columns of the MFMA that a GEMV
// does not need carry the bookkeeping instead: the activation operand holds, in row 8 h + 4 p + j, plane p of
// the 16 values of sub-block j of k-set h and zeros elsewhere, so that one accumulator lane ends up with the
// four sub-block sums of one row, one plane, one k-set -- exactly the four that its four consecutive scale bytes
// weigh.  Integer sums are exact; each (row, unit) then takes one float multiply by a power of two and one
// fused multiply-add with d.  A unit-vector activation reproduces the canonical column bit for bit (d, scale
// and q6 - 32 have 11 + 7 + 6 significant bits, so every order of the products is exact).
#include "ttq_gemv_mfma_common.h"

namespace ttq {

namespace {

constexpr int kQ6Waves = 8;
constexpr int kQ6Threads = kQ6Waves * 64;
constexpr int kQ6Nb = 16;                                  // blocks per row: n_in = 4096
constexpr int kQ6RowBytes = kQ6Nb * 210;                   // 3360
constexpr int kQ6GroupBytes = 16 * kQ6RowBytes;            // 53760 in memory
constexpr int kQ6HalfBlocks = kQ6Nb / 2;                   // blocks of a row in one round: one per wavefront
constexpr int kQ6SlotChunks = 14;                          // a block in LDS: 224 bytes
constexpr int kQ6TailAt = 196;                             // chunk 13 starts here, counted from the slot's first byte
constexpr int kQ6DAt = 208 - kQ6TailAt;                    // d in chunk 13 (+ 2 for an odd block)
constexpr int kQ6RowChunks = kQ6HalfBlocks * kQ6SlotChunks;   // 112
constexpr int kQ6Requests = 16 * kQ6RowChunks / 64;        // 28
constexpr int kQ6BufBytes = kQ6Requests * 1024;            // 28672
#ifndef Q6_ORDER
#define Q6_ORDER 0
#endif
#ifndef Q6_BUFS
#define Q6_BUFS 2
#endif
#ifndef Q6_WGS_PER_CU
#define Q6_WGS_PER_CU 2
#endif
constexpr int kQ6Bufs = Q6_BUFS;
constexpr int kQ6ReqMax = (kQ6Requests + kQ6Waves - 1) / kQ6Waves;   // 4
constexpr int kQ6FullWaves = kQ6Requests - (kQ6ReqMax - 1) * kQ6Waves;   // wavefronts 0..3 make 4 requests, the others 3
constexpr int kQ6WgsPerCu = Q6_WGS_PER_CU;
constexpr int kQ6MaxGroups = 40 / kQ6WgsPerCu;                           // row groups of a workgroup (their partial sums wait in LDS)
constexpr int kQ6MinGroups = 2;
static_assert(kQ6HalfBlocks == kQ6Waves, "one block of the half per wavefront");
static_assert(kQ6Bufs >= 2 && kQ6Bufs <= 4, "the waits below count up to three later rounds");

typedef const __attribute__((address_space(1))) void* q6_gptr_t;
typedef __attribute__((address_space(3))) void* q6_lptr_t;
typedef uint32_t q6_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t q6_u32x2 __attribute__((ext_vector_type(2)));

template <int N>
__device__ __forceinline__ void q6_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}
// a barrier that leaves the outstanding requests alone
__device__ __forceinline__ void q6_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ uint32_t q6_lds(const void* p) { return (uint32_t)(size_t)(q6_lptr_t)(p); }
// LDS accesses the compiler must not see: it cannot tell them from the asynchronous writes of the requests in
// flight and would wait for every one of those first
__device__ __forceinline__ q6_u32x4 q6_read16(uint32_t a) {
  q6_u32x4 v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(a) : "memory");
  return v;
}
__device__ __forceinline__ float q6_read_f32(uint32_t a) {
  float v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(a) : "memory");
  return v;
}
__device__ __forceinline__ void q6_write_f32(uint32_t a, float v) {
  asm volatile("ds_write_b32 %0, %1" ::"v"(a), "v"(v) : "memory");
}

// XT: bf16 or fp16 activations.  The row groups are dealt out in runs: the first groups_rem workgroups take
// groups_per_wg + 1 each, the others groups_per_wg.
// STAGE 0 is the GEMV; STAGE 1 leaves out the arithmetic on the operands, STAGE 2 the operand reads as well
// (requests, waits and barriers stay): what each part costs is measured by leaving it out.
template <typename XT, typename YT, int STAGE = 0>
__global__ void __launch_bounds__(kQ6Threads) __attribute__((amdgpu_waves_per_eu(2 * kQ6WgsPerCu, 2 * kQ6WgsPerCu)))
gemv_q6k_stream_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                       const void* __restrict__ bias, int bias_dtype, int n_out, int groups_per_wg, int groups_rem) {
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kQ6Bufs * kQ6BufBytes];
  __shared__ __attribute__((aligned(16))) v4i_t xa[kQ6Nb * 32 + 1];    // (16 values, plane) entries + one of zeros
  __shared__ __attribute__((aligned(16))) float fac[kQ6Nb * 4 * 2];    // (64 values, plane): scale of the integer sum
  // (the raw activations land here first: the partial sums are written after they have been read back)
  __shared__ __attribute__((aligned(1024))) float part[kQ6MaxGroups][kQ6Waves][16];
  static_assert(sizeof(part) >= kQ6Threads * 16, "room for the staged activations");
  uint8_t* xstage = reinterpret_cast<uint8_t*>(&part[0][0][0]);

  constexpr int n_in = kQ6Nb * 256;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const uint16_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const int bx = blockIdx.x;
  const int grp0 = bx * groups_per_wg + min(bx, groups_rem);
  const int ng = groups_per_wg + (bx < groups_rem ? 1 : 0);            // kQ6MinGroups .. kQ6MaxGroups
  const int nrounds = 2 * ng;

  // ---- the activations, as an LDS request too (a register load among the weight requests would make the
  // compiler wait for all of them at its first use): thread t stages x[8 t .. 8 t + 7]
  const int k0 = 8 * tid;
  __builtin_amdgcn_global_load_lds((q6_gptr_t)(xm + k0), (q6_lptr_t)(xstage + wave * 1024), 16, 0, 0);
  // a compute unit serves its requests in the order they were made: every wavefront's activation request is
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
    src_off[i] = (uint32_t)(row * kQ6RowBytes + b * 210 - 2 * (b & 1) + (j < kQ6SlotChunks - 1 ? 16 * j : kQ6TailAt));
  }
  const bool full = wave < kQ6FullWaves;
  // round rr = 2 * (group - grp0) + (half of K)
  auto request_round = [&](int rr, int buf) {
    const uint8_t* src = w + (size_t)((uint32_t)(grp0 + (rr >> 1)) * (uint32_t)kQ6GroupBytes +
                                      (uint32_t)((rr & 1) * (kQ6HalfBlocks * 210)));
    uint8_t* dst = wbuf + buf * kQ6BufBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < kQ6ReqMax - 1; i++)
      __builtin_amdgcn_global_load_lds((q6_gptr_t)(src + src_off[i]), (q6_lptr_t)(dst + i * (kQ6Waves * 1024)), 16, 0, 2);
    if (full)
      __builtin_amdgcn_global_load_lds((q6_gptr_t)(src + src_off[kQ6ReqMax - 1]),
                                       (q6_lptr_t)(dst + (kQ6ReqMax - 1) * (kQ6Waves * 1024)), 16, 0, 2);
  };
  // all but the youngest `rounds_after` rounds of requests of this wavefront have landed
  auto wait_rounds = [&](auto rounds_after) {
    constexpr int A = decltype(rounds_after)::value;
    if (full) q6_wait_vmcnt<A * kQ6ReqMax>();
    else q6_wait_vmcnt<A * (kQ6ReqMax - 1)>();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
#pragma unroll
  for (int i = 0; i < kQ6Bufs; i++) request_round(i, i);      // nrounds >= 4

  // ---- the raw activations back into registers, then into the two byte planes
  float xf[8];
  {
    wait_rounds(std::integral_constant<int, kQ6Bufs>{});
    const q6_u32x4 r = q6_read16(q6_lds(xstage) + (uint32_t)(tid * 16));
    widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), xf);
  }
  if (tid < 4) reinterpret_cast<uint32_t*>(&xa[kQ6Nb * 32])[tid] = 0u;
  {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(xf[i]));
    // the eight threads of 64 values are an aligned octet
    amax = fmaxf(amax, dpp_quad<0xB1>(amax));
    amax = fmaxf(amax, dpp_quad<0x4E>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 4, kWave));
    const uint32_t eb = __float_as_uint(amax) >> 23;       // biased exponent (amax >= 0)
    const uint32_t ec = eb < 18u ? 18u : eb;               // 2^(E-13) / 4 stays a normal number
    const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
    // non-finite activations poison their 64 values instead of being clipped
    const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
    int hi[8], lo[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int v = (int)rintf(xf[i] * mul);
      hi[i] = (v + 128) >> 8;
      lo[i] = v;                     // only the low byte is used, as a signed byte
    }
    // entry (k / 16, plane), 16 bytes; this thread's eight values are one half of it
    uint2* xa8 = reinterpret_cast<uint2*>(&xa[0]);
    const int e = (k0 >> 4) * 4 + ((k0 >> 3) & 1);
    xa8[e] = make_uint2(pack_low_bytes(hi[0], hi[1], hi[2], hi[3]), pack_low_bytes(hi[4], hi[5], hi[6], hi[7]));
    xa8[e + 2] = make_uint2(pack_low_bytes(lo[0], lo[1], lo[2], lo[3]), pack_low_bytes(lo[4], lo[5], lo[6], lo[7]));
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
  const int slot = wave * kQ6SlotChunks;                   // the wavefront's block of the half
  // activation operand: lane (i, g) of the first MFMA holds something only if i < 8 and i % 4 == g, of the
  // second only if i >= 8 and i % 4 == g; plane (i / 4) % 2.  Unit u = 2 block + half starts at value 128 u.
  const uint32_t xa_base = q6_lds(&xa[0]);
  const uint32_t zero_entry = xa_base + (uint32_t)(kQ6Nb * 32 * 16);
  const bool mine = (n & 3) == g;
  const uint32_t plane16 = (uint32_t)(((n >> 2) & 1) * 16);
  const bool act1 = mine && n < 8, act2 = mine && n >= 8;
  const uint32_t u0 = (uint32_t)(2 * wave);                // the wavefront's first unit of a first half of K
  const uint32_t a1_addr = act1 ? xa_base + 256u * u0 + 32u * (uint32_t)g + plane16 : zero_entry;
  const uint32_t a2_addr = act2 ? xa_base + 256u * u0 + 128u + 32u * (uint32_t)g + plane16 : zero_entry;
  // per unit 256 bytes of table, per half of K 16 units
  const uint32_t a1_step = act1 ? 256u : 0u, a2_step = act2 ? 256u : 0u;
  const uint32_t fac_addr0 = q6_lds(&fac[0]) + 16u * u0 + 4u * (uint32_t)g;
  const uint32_t wbuf_base = q6_lds(wbuf);

  q6_barrier();                         // the plane table is complete

  const uint32_t part_addr = q6_lds(&part[0][0][0]) + (uint32_t)((wave * 16 + n) * 4);
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

    struct Regs { q6_u32x4 ql, qh, a1, a2; uint32_t sc, d, f, qlx, qhx, scx; };
    // unit hf of the round, k-half kh
    auto issue = [&](auto hc, uint32_t buf, uint32_t kh, Regs& r) {
      constexpr int hf = decltype(hc)::value;
      const uint32_t a_ql = buf + (hf ? ql_off1 : ql_off0), a_qh = buf + (hf ? qh_off1 : qh_off0);
      const uint32_t a_sc = buf + sc_off, a_d = buf + d_off;
      const uint32_t ui = 16u * kh + (uint32_t)hf;
      const uint32_t x1 = a1_addr + ui * a1_step, x2 = a2_addr + ui * a2_step;
      const uint32_t fa = fac_addr0 + 16u * ui;
      if constexpr (STAGE >= 2) return;
      asm volatile(
          "ds_read_b128 %0, %7\n\t"
          "ds_read_b128 %1, %8\n\t"
          "ds_read_b128 %2, %9\n\t"
          "ds_read_b128 %3, %10\n\t"
          "ds_read_b32 %4, %11 offset:%13\n\t"
          "ds_read_u16 %5, %12\n\t"
          "ds_read_b32 %6, %14"
          : "=&v"(r.ql), "=&v"(r.qh), "=&v"(r.a1), "=&v"(r.a2), "=&v"(r.sc), "=&v"(r.d), "=&v"(r.f)
          : "v"(a_ql), "v"(a_qh), "v"(x1), "v"(x2), "v"(a_sc), "v"(a_d), "n"(8 * hf), "v"(fa)
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
    constexpr int kReads = ODD ? 10 : 7;                   // LDS reads of a unit
    auto settle = [&](auto pending, Regs& r) {
      constexpr int P = decltype(pending)::value;
      if constexpr (STAGE >= 2) return;
      if constexpr (ODD)
        asm volatile("s_waitcnt lgkmcnt(%10)"
                     : "+v"(r.ql), "+v"(r.qh), "+v"(r.a1), "+v"(r.a2), "+v"(r.sc), "+v"(r.d), "+v"(r.f), "+v"(r.qlx),
                       "+v"(r.qhx), "+v"(r.scx)
                     : "n"(P)
                     : "memory");
      else
        asm volatile("s_waitcnt lgkmcnt(%7)"
                     : "+v"(r.ql), "+v"(r.qh), "+v"(r.a1), "+v"(r.a2), "+v"(r.sc), "+v"(r.d), "+v"(r.f)
                     : "n"(P)
                     : "memory");
    };
    float acc = 0.f;
    auto compute = [&](const Regs& r) {
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
        A1[i] = (int)r.a1[i];
        A2[i] = (int)r.a2[i];
      }
      const v4i_t zero = {0, 0, 0, 0};
      v4i_t C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, B1, zero, 0, 0, 0);
      C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A2, B2, C, 0, 0, 0);
      const int sc = (int)sc4;
      int t = (int)(int8_t)(sc & 0xFF) * C[0];
      t += (int)(int8_t)((sc >> 8) & 0xFF) * C[1];
      t += (int)(int8_t)((sc >> 16) & 0xFF) * C[2];
      t += (sc >> 24) * C[3];
      const float d = f16_bits_to_f32((uint16_t)(r.d & 0xFFFFu));
      acc = fmaf_((float)t * __uint_as_float(r.f), d, acc);
      // pins the arithmetic here: left alone the compiler moves it behind later waits
      asm volatile("" : "+v"(acc));
    };

    using U0 = std::integral_constant<int, 0>;
    using U1 = std::integral_constant<int, 1>;
    int bufi = 0;
    for (int rr = 0; rr < nrounds; rr++) {
      // the round's buffer: own requests landed, then everybody's
      const int later = min(nrounds - 1 - rr, kQ6Bufs - 1);        // rounds requested after this one
      if (later == 3) wait_rounds(I3{});
      else if (later == 2) wait_rounds(I2{});
      else if (later == 1) wait_rounds(I1{});
      else wait_rounds(I0{});
      q6_barrier();
      const uint32_t buf = wbuf_base + (uint32_t)(bufi * kQ6BufBytes);
      const uint32_t kh = (uint32_t)(rr & 1);
      Regs ra, rb;
      issue(U0{}, buf, kh, ra);
      issue(U1{}, buf, kh, rb);
      settle(std::integral_constant<int, kReads>{}, ra);
      compute(ra);
      settle(I0{}, rb);
      // every wavefront has read what it needs of the buffer: the round kQ6Bufs later may land there
      q6_barrier();
      if (rr + kQ6Bufs < nrounds) request_round(rr + kQ6Bufs, bufi);
      bufi = bufi == kQ6Bufs - 1 ? 0 : bufi + 1;
      compute(rb);
      if (kh) {
        // the four accumulator lanes of a row
        acc += __shfl_xor(acc, 16, kWave);
        acc += __shfl_xor(acc, 32, kWave);
        if (lane < 16) q6_write_f32(part_addr + (uint32_t)((rr >> 1) * (kQ6Waves * 16 * 4)), acc);
        acc = 0.f;
      }
    }
  };
  if (wave & 1) run_rounds(std::true_type{});
  else run_rounds(std::false_type{});
  // every request has landed (plain loads are safe again); the eight K-slices of a row add up in a fixed order
  __syncthreads();
  for (int t = tid; t < ng * 16; t += kQ6Threads) {
    const int grp = t >> 4, nn = t & 15;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < kQ6Waves; wv++) v += part[grp][wv][nn];
    const int row = (grp0 + grp) * 16 + nn;
    YElem<YT>::store(ym, row, v + load_bias(bias, bias_dtype, row));
  }
}

template <typename XT, typename YT>
hipError_t q6_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                        hipStream_t s) {
  const int groups = (int)(n_out / 16);
  // two workgroups per compute unit when every one of them still gets two groups: their rounds interleave
  int num_wg = min(kQ6WgsPerCu * device_num_cus(), groups / kQ6MinGroups);
  if ((groups + num_wg - 1) / num_wg > kQ6MaxGroups) num_wg = (groups + kQ6MaxGroups - 1) / kQ6MaxGroups;
  const dim3 grid((unsigned)num_wg, (unsigned)m), block(kQ6Threads);
  hipLaunchKernelGGL((gemv_q6k_stream_kernel<XT, YT>), grid, block, 0, s, static_cast<const uint8_t*>(w),
                     static_cast<const uint16_t*>(x), static_cast<YT*>(y), bias, bias_dtype, (int)n_out, groups / num_wg,
                     groups % num_wg);
  return hipGetLastError();
}

template <typename XT>
hipError_t q6_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                       int64_t n_out, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return q6_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, s);
    case kF16: return q6_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, s);
    case kBF16: return q6_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

// Whole groups of 16 rows, at least two per compute unit (the two LDS buffers are requested before anything
// else), 32-bit byte offsets into the weight buffer.
bool gemv_q6k_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  if (format != kQ6_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  if (n_in != kQ6Nb * 256 || n_out % 16 != 0) return false;
  static const int off = dev_knob("TTQ_Q6K_STREAM_OFF", 0);
  if (off) return false;
  return n_out / 16 >= (int64_t)kQ6MinGroups * device_num_cus() && n_out * kQ6RowBytes < ((int64_t)1 << 32);
}

hipError_t launch_gemv_q6k_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  (void)n_in;
  if (x_dtype == kBF16) return q6_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, s);
  if (x_dtype == kF16) return q6_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
