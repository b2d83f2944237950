// Decode GEMV for Q4_K weights with long rows (6144 .. 14336 inputs: the down projection of a gated
// MLP, workspace/transformers/src/layers/mlp.nim:47-52, through F.linear,
// workspace/libtorch/src/abi/neural_nets.nim:64-81).
//
// The LDS-streamed kernel of ttq_gemv_q4k_stream.h keeps the quantized activations of the whole row
// in one table per workgroup; at 14336 inputs that table (28 KiB) no longer fits beside eight 18 KiB
// stream buffers.  Here K is dealt to the wavefronts instead: a row is cut into slices of 2048 inputs
// (8 super-blocks, the block of the streamed kernel), wavefront w owns slice w % nks of every row group
// it works on, and everything it needs about the activations -- the two byte planes of its 2048
// values (4 KiB), the scales / sums of its 64 sub-blocks (512 bytes) -- is private to it.  So:
//   * seven wavefronts, each with its own stream buffer, plane table and scale table: 7 x 23 KiB;
//   * the prologue has no workgroup barrier: a wavefront fetches its slice of x (four LDS requests,
//     landing where the plane table will be), asks for the first weight lines, and quantizes while
//     they travel.  A lane owns a whole sub-block of 32 values, the scale needs no cross-lane step;
//   * block fixed point, operand layout, MFMA and scale arithmetic are the streamed kernel's; the
//     per-pair constants are packed into one 16-byte entry (the two power-of-two scales as the upper
//     halves of their fp32 bits) so that a super-block takes eight LDS reads;
//   * the nks partial sums of a row meet in LDS after one barrier at the end, added in slice order.
#include "ttq_gemv_q4k_stream.h"

namespace ttq {

namespace {

constexpr int kSlWaves = 7;
constexpr int kSlThreads = kSlWaves * 64;
constexpr int kSlPlaneBytes = 4096 + 16;      // two byte planes of 2048 activations + one zero entry
constexpr int kSlConstBytes = 512;            // 8 super-blocks x 4 pairs of sub-blocks x 16 bytes
constexpr int kSlMaxBlocks = 38;              // (row groups of a workgroup) x (slices): their sums wait in LDS
constexpr int kSlUpFirst = 4;                 // weight requests made before the activations are quantized

__device__ __forceinline__ void sl_write16(uint32_t a, st_u32x4 v) {
  asm volatile("ds_write_b128 %0, %1" : : "v"(a), "v"(v) : "memory");
}

// UP: weight requests of a block in flight before its first super-block is multiplied (even, 6 .. 18).
// FEW: a wavefront has one or two blocks, the bytes arrive in a burst (see ttq_gemv_q4k_stream.h).
template <typename XT, typename YT, int UP, bool FEW>
__global__ void __launch_bounds__(kSlThreads)
gemv_q4k_slice_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ x, YT* __restrict__ y,
                      const void* __restrict__ bias, int bias_dtype, int n_out, int nks, int rows_per_wg) {
  static_assert(UP % 2 == 0 && UP >= kSlUpFirst + 2 && UP <= kStBlockRequests, "requests go out in pairs");
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kSlWaves * kStBlockBytes];
  __shared__ __attribute__((aligned(16))) uint8_t planes[kSlWaves * kSlPlaneBytes];
  __shared__ __attribute__((aligned(16))) uint8_t consts[kSlWaves * kSlConstBytes];
  __shared__ float part[kSlMaxBlocks][16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int n_in = nks * 2048;
  const uint16_t* xm = x + (int64_t)blockIdx.y * n_in;
  YT* ym = y + (int64_t)blockIdx.y * n_out;
  const uint32_t rb = (uint32_t)nks * (uint32_t)kStSegBytes;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int last = wg_row_end - 1;
  const int ngroups = (wg_row_end - wg_row0 + 15) >> 4;                  // row groups of 16 outputs
  // wavefront -> (slice, first row group, row group stride)
  const int wps = kSlWaves / nks;
  const int ks = wave % nks, rg0 = wave / nks;

  if (wave < wps * nks && rg0 < ngroups) {
    uint8_t* mybuf = wbuf + wave * kStBlockBytes;
    uint8_t* myplanes = planes + wave * kSlPlaneBytes;
    const uint32_t xa_base = (uint32_t)(size_t)(st_lptr_t)(myplanes);
    const uint32_t cst_base = (uint32_t)(size_t)(st_lptr_t)(consts + wave * kSlConstBytes);

    // ---- the slice of x, raw, as the wavefront's four oldest requests: request j brings
    // x[2048 ks + 512 j + 8 lane ..] to byte 1024 j + 16 lane, i.e. the slice in order
    {
      const uint16_t* xs = xm + ks * 2048 + lane * 8;
#pragma unroll
      for (int j = 0; j < 4; j++)
        __builtin_amdgcn_global_load_lds((st_gptr_t)(xs + j * 512), (st_lptr_t)(myplanes + j * 1024), 16, 0, 0);
    }

    // ---- requests of a block: as in the streamed kernel (line `line` of row 8 o + lane / 8, chunk
    // (lane % 8) ^ key(row)), the block being slice ks of row group rg
    uint32_t lane_off[2];
    auto set_block = [&](int rg) {
      const int r8 = lane >> 3;
#pragma unroll
      for (int o = 0; o < 2; o++) {
        const int row16 = 8 * o + r8;
        const int row = min(wg_row0 + rg * 16 + row16, last);         // past the end: the last row again, never used
        lane_off[o] = (uint32_t)row * rb + (uint32_t)(ks * kStSegBytes) + (uint32_t)(((lane & 7) ^ ((row16 >> 1) & 7)) * 16);
      }
    };
    auto request = [&](int i) {
      const int line = i >> 1, o = i & 1;
      __builtin_amdgcn_global_load_lds((st_gptr_t)(w + (size_t)(lane_off[o] + (uint32_t)(line * 128))),
                                       (st_lptr_t)(mybuf + o * kStHalfBytes + line * 1024), 16, 0, 2);
    };
    set_block(rg0);
#pragma unroll
    for (int i = 0; i < kSlUpFirst; i++) request(i);

    // ---- quantize: lane l owns sub-block l of the slice (32 values, bytes 64 l .. 64 l + 63 of the raw
    // slice) and overwrites exactly those bytes with its four plane entries
    st_wait_vmcnt<kSlUpFirst>();
    request(kSlUpFirst);
    request(kSlUpFirst + 1);
    {
      float xf[32];
      st_u32x4 raw[4];
      asm volatile(
          "ds_read_b128 %0, %4\n\t"
          "ds_read_b128 %1, %4 offset:16\n\t"
          "ds_read_b128 %2, %4 offset:32\n\t"
          "ds_read_b128 %3, %4 offset:48\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(raw[0]), "=&v"(raw[1]), "=&v"(raw[2]), "=&v"(raw[3])
          : "v"(xa_base + (uint32_t)(lane * 64))
          : "memory");
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const st_u32x4 r = raw[c];
        float t[8];
        widen8<XT>(make_uint4(r[0], r[1], r[2], r[3]), t);
#pragma unroll
        for (int i = 0; i < 8; i++) xf[8 * c + i] = t[i];
      }
      const uint32_t eb = amax_bits(xf) >> 23;              // biased exponent of max |x|; 255 for Inf and NaN
      const uint32_t ec = eb < 18u ? 18u : eb;              // 2^(E-13) / 16 stays a normal number
      const float mul = __uint_as_float((267u - ec) << 23);  // 2^(13-E)
      // non-finite activations poison the sub-block instead of being clipped
      const float f = eb == 255u ? __uint_as_float(0x7FC00000u) : __uint_as_float((ec - 13u) << 23);
      // v = rint(x * 2^(13-E)), |v| <= 2^14, read off the low bits of x * 2^(13-E) + 1.5 * 2^23 (one fused
      // multiply-add rounds to the integer grid, nearest-even like rintf; the product itself is exact)
      uint32_t vbits[32], vacc = 0u;
#pragma unroll
      for (int i = 0; i < 32; i++) {
        vbits[i] = __float_as_uint(fmaf_(xf[i], mul, __uint_as_float(kRoundMagicBits)));
        vacc += vbits[i];
      }
      const int vsum = (int)(vacc - 32u * kRoundMagicBits);      // modulo 2^32: the sum itself is below 2^19
      // sum(x) of the sub-block as the fixed-point values give it: the row sum is then exactly the dot
      // product of the dequantized weights with the quantized activations
      const float sum = (float)vsum * f;
      st_u32x4 ent[4];       // hi plane of values 0-15, 16-31, lo plane of values 0-15, 16-31
#pragma unroll
      for (int q = 0; q < 8; q++) {
        const uint32_t* v = &vbits[4 * q];
        // hi = (v + 128) >> 8 and lo = v, one byte each
        ent[q >> 2][q & 3] = pack_bytes1(v[0] + 128u, v[1] + 128u, v[2] + 128u, v[3] + 128u);
        ent[2 + (q >> 2)][q & 3] = pack_low_bytes((int)v[0], (int)v[1], (int)v[2], (int)v[3]);
      }
#pragma unroll
      for (int c = 0; c < 4; c++) sl_write16(xa_base + (uint32_t)(lane * 64 + c * 16), ent[c]);
      if (lane == 0) sl_write16(xa_base + 4096u, st_u32x4{0u, 0u, 0u, 0u});
      // per pair of sub-blocks (2p, 2p+1), written by the odd one's lane:
      //   {bits 31-16 of 2^(E-13) of 2p | of 2^(E-13) / 16 of 2p+1, sum(x) of 2p, sum(x) of 2p+1, 128 * sum(v) of 2p+1}
      // (the odd sub-block's nibbles reach the MFMA as 16 * (q - 8))
      const float fv = (lane & 1) ? f * 0.0625f : f;
      const uint32_t f_even = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(fv), 0xB1, 0xF, 0xF, false);
      const float sum_even = dpp_quad<0xB1>(sum);
      if (lane & 1)
        sl_write16(cst_base + (uint32_t)((lane >> 1) * 16),
                   st_u32x4{(f_even >> 16) | (__float_as_uint(fv) & 0xFFFF0000u), __float_as_uint(sum_even),
                            __float_as_uint(sum), (uint32_t)(128 * vsum)});
    }
#pragma unroll
    for (int i = kSlUpFirst + 2; i < UP; i++) request(i);

    // ---- per-lane constants of the main loop (the streamed kernel's)
    const bool upper = g >= 2;
    const uint32_t m_lo = upper ? 0x0F0F0F0Fu : 0x3F3F3F3Fu, m_top = upper ? 0x30303030u : 0u;
    const uint32_t pair_shift = 16u * (uint32_t)(g & 1);
    constexpr uint32_t N4 = 0x0F0F0F0Fu;
    uint32_t a_addr[4], a_step[4];
    {
      const int mrow = lane & 15, ga = lane >> 4, j = mrow >> 1;
      const bool valid = (ga >> 1) == ((j & 3) >> 1);
      const int qstar = 2 * (j >> 2) + (j & 1);
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const bool mine = valid && q == qstar;
        a_addr[q] = xa_base + 16u * (mine ? (uint32_t)(mrow * 2 + (ga & 1)) : 256u);
        a_step[q] = mine ? 512u : 0u;
      }
    }
    const uint32_t cst_addr = cst_base + (uint32_t)(g * 16);
    const uint32_t key = (uint32_t)(n >> 1) & 7u;
    const uint32_t rowbase = (uint32_t)(size_t)(st_lptr_t)(mybuf) + (uint32_t)((n >> 3) * kStHalfBytes + (n & 7) * 128);

    struct Regs { st_u32x4 hdr, c0, c1, a0, a1, a2, a3, cst; };
    auto topup = [&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if constexpr (UP + 2 * s < kStBlockRequests) {
        request(UP + 2 * s);
        request(UP + 2 * s + 1);
      }
    };
    auto issue = [&](auto sc, Regs& r) {
      constexpr int s = decltype(sc)::value;
      // super-block s needs requests 0 .. 2 s + 3 (its two top-up requests have been made by now)
      constexpr int kIssued = UP + 2 * (s + 1) < kStBlockRequests ? UP + 2 * (s + 1) : kStBlockRequests;
      st_wait_vmcnt<kIssued - (2 * s + 4)>();
      const uint32_t e0 = ((1u + (uint32_t)g + (uint32_t)s) ^ key), e1 = ((5u + (uint32_t)g + (uint32_t)s) ^ key);
      const uint32_t a_h = rowbase + ((key ^ (uint32_t)s) << 4);
      const uint32_t a_0 = rowbase + ((e0 & 8u) << 7) + ((e0 & 7u) << 4);
      const uint32_t a_1 = rowbase + ((e1 & 8u) << 7) + ((e1 & 7u) << 4);
      const uint32_t x0 = a_addr[0] + (uint32_t)s * a_step[0], x1 = a_addr[1] + (uint32_t)s * a_step[1];
      const uint32_t x2 = a_addr[2] + (uint32_t)s * a_step[2], x3 = a_addr[3] + (uint32_t)s * a_step[3];
      const uint32_t ca = cst_addr;
      asm volatile(
          "ds_read_b128 %0, %8 offset:%15\n\t"
          "ds_read_b128 %1, %9 offset:%15\n\t"
          "ds_read_b128 %2, %10 offset:%15\n\t"
          "ds_read_b128 %3, %11\n\t"
          "ds_read_b128 %4, %12\n\t"
          "ds_read_b128 %5, %13\n\t"
          "ds_read_b128 %6, %14\n\t"
          "ds_read_b128 %7, %16 offset:%17"
          : "=&v"(r.hdr), "=&v"(r.c0), "=&v"(r.c1), "=&v"(r.a0), "=&v"(r.a1), "=&v"(r.a2), "=&v"(r.a3), "=&v"(r.cst)
          : "v"(a_h), "v"(a_0), "v"(a_1), "v"(x0), "v"(x1), "v"(x2), "v"(x3), "n"(s * 1024), "v"(ca), "n"(s * 64)
          : "memory");
    };
    auto settle = [&](auto pending, Regs& r) {
      constexpr int P = decltype(pending)::value;
      asm volatile("s_waitcnt lgkmcnt(%8)"
                   : "+v"(r.hdr), "+v"(r.c0), "+v"(r.c1), "+v"(r.a0), "+v"(r.a1), "+v"(r.a2), "+v"(r.a3), "+v"(r.cst)
                   : "n"(P)
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
      const float q1 = (float)(C[0] * 256 + C[1]) * __uint_as_float(r.cst[0] << 16);
      const float q2 = (float)(C[2] * 256 + C[3] + (int)r.cst[3]) * __uint_as_float(r.cst[0] & 0xFFFF0000u);
      // (d * sc) * q - (dmin * m) * sum(x), in the canonical dequantizer's rounding order
      acc = fmaf_(d * sc1, q1, acc);
      acc = fmaf_(-(dmin * mn1), __uint_as_float(r.cst[1]), acc);
      acc = fmaf_(d * sc2, q2, acc);
      acc = fmaf_(-(dmin * mn2), __uint_as_float(r.cst[2]), acc);
      asm volatile("" : "+v"(acc));     // keeps the arithmetic between the waits it was written between
    };

    // ---- the wavefront's blocks: row groups rg0, rg0 + wps, ...  A block starts with UP requests outstanding.
    auto run_block = [&](const int rg) {
      acc = 0.f;
      Regs ra, rb2;
      using I0 = std::integral_constant<int, 0>;
      if constexpr (!FEW) {
        topup(std::integral_constant<int, 0>{}); issue(std::integral_constant<int, 0>{}, ra);
        topup(std::integral_constant<int, 1>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 1>{}, rb2);
        topup(std::integral_constant<int, 2>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 2>{}, ra);
        topup(std::integral_constant<int, 3>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 3>{}, rb2);
        topup(std::integral_constant<int, 4>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 4>{}, ra);
        topup(std::integral_constant<int, 5>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 5>{}, rb2);
        topup(std::integral_constant<int, 6>{}); settle(I0{}, rb2); compute(rb2); issue(std::integral_constant<int, 6>{}, ra);
        topup(std::integral_constant<int, 7>{}); settle(I0{}, ra); compute(ra); issue(std::integral_constant<int, 7>{}, rb2);
      } else {
        using I8 = std::integral_constant<int, 8>;
        topup(std::integral_constant<int, 0>{}); issue(std::integral_constant<int, 0>{}, ra);
        topup(std::integral_constant<int, 1>{}); issue(std::integral_constant<int, 1>{}, rb2); settle(I8{}, ra); compute(ra);
        topup(std::integral_constant<int, 2>{}); issue(std::integral_constant<int, 2>{}, ra); settle(I8{}, rb2); compute(rb2);
        topup(std::integral_constant<int, 3>{}); issue(std::integral_constant<int, 3>{}, rb2); settle(I8{}, ra); compute(ra);
        topup(std::integral_constant<int, 4>{}); issue(std::integral_constant<int, 4>{}, ra); settle(I8{}, rb2); compute(rb2);
        topup(std::integral_constant<int, 5>{}); issue(std::integral_constant<int, 5>{}, rb2); settle(I8{}, ra); compute(ra);
        topup(std::integral_constant<int, 6>{}); issue(std::integral_constant<int, 6>{}, ra); settle(I8{}, rb2); compute(rb2);
        topup(std::integral_constant<int, 7>{}); issue(std::integral_constant<int, 7>{}, rb2); settle(I8{}, ra); compute(ra);
      }
      settle(I0{}, rb2);
      // every request of the block has landed and been read: the next block may use the buffer
      const int next = rg + wps;
      if (next < ngroups) {
        set_block(next);
#pragma unroll
        for (int i = 0; i < UP; i++) request(i);
      }
      compute(rb2);
      acc = add_xor16(acc);
      acc = add_xor32(acc);
      if (lane < 16) part[rg * nks + ks][lane] = acc;
    };
    int rg = rg0;
    run_block(rg);
    for (rg += wps; rg < ngroups; rg += wps) run_block(rg);
  }

  // every request has landed; the slices of a row add up in slice order
  __syncthreads();
  for (int t = tid; t < ngroups * 16; t += kSlThreads) {
    const int grp = t >> 4, nn = t & 15;
    float v = part[grp * nks][nn];
    for (int k = 1; k < nks; k++) v += part[grp * nks + k][nn];
    const int row = wg_row0 + t;
    if (row < wg_row_end) YElem<YT>::store_through(ym, row, v + load_bias(bias, bias_dtype, row));
  }
}

struct SlPlan { bool ok; int num_wg, rows_per_wg, nks, blocks_per_wave; };

SlPlan sl_plan(int64_t n_out, int64_t n_in) {
  SlPlan p{};
  if (n_in % 2048 != 0 || n_in < 3 * 2048 || n_in > kSlWaves * 2048) return p;
  if (n_out < 16 * (int64_t)device_num_cus() || n_out * (n_in / 256) * 144 >= ((int64_t)1 << 32)) return p;
  p.nks = (int)(n_in / 2048);
  p.rows_per_wg = st_rows_per_wg(n_out, &p.num_wg);
  const int groups = (p.rows_per_wg + 15) / 16, wps = kSlWaves / p.nks;
  if (groups * p.nks > kSlMaxBlocks) return p;
  p.blocks_per_wave = (groups + wps - 1) / wps;
  p.ok = true;
  return p;
}

template <typename XT, typename YT>
hipError_t sl_launch_xy(const void* w, const void* x, void* y, const void* bias, int bias_dtype, int64_t m,
                        int64_t n_out, int64_t n_in, hipStream_t s) {
  const SlPlan p = sl_plan(n_out, n_in);
  if (!p.ok) return hipErrorInvalidValue;
  const dim3 grid((unsigned)p.num_wg, (unsigned)m), block(kSlThreads);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(x),
                       static_cast<YT*>(y), bias, bias_dtype, (int)n_out, p.nks, p.rows_per_wg);
  };
  static const int up_knob = dev_knob("TTQ_SLICE_UP", 0);
  if (up_knob == 6) go(gemv_q4k_slice_kernel<XT, YT, 6, false>);
  else if (up_knob == 8) go(gemv_q4k_slice_kernel<XT, YT, 8, false>);
  else if (up_knob == 12) go(gemv_q4k_slice_kernel<XT, YT, 12, true>);
  else if (up_knob == 18) go(gemv_q4k_slice_kernel<XT, YT, 18, true>);
  else go(gemv_q4k_slice_kernel<XT, YT, 6, false>);
  return hipGetLastError();
}

template <typename XT>
hipError_t sl_launch_x(const void* w, const void* x, void* y, int y_dtype, const void* bias, int bias_dtype,
                       int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (y_dtype) {
    case kF32: return sl_launch_xy<XT, float>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kF16: return sl_launch_xy<XT, f16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    case kBF16: return sl_launch_xy<XT, bf16_tag>(w, x, y, bias, bias_dtype, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

bool gemv_q4k_slice_supported(int format, int x_dtype, int64_t n_out, int64_t n_in) {
  if (format != kQ4_K || !(x_dtype == kBF16 || x_dtype == kF16)) return false;
  return sl_plan(n_out, n_in).ok;
}

hipError_t launch_gemv_q4k_slice(const void* w, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  if (x_dtype == kBF16) return sl_launch_x<bf16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  if (x_dtype == kF16) return sl_launch_x<f16_tag>(w, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
  return hipErrorInvalidValue;
}

}  // namespace ttq
