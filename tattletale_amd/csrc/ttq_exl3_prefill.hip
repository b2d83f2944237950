// Trellis-coded (EXL3-style) linear layer for many activation rows: Y = svh o H( T * H(suh o X^T) ),
// the prefill side of Linear.forward (workspace/transformers/src/layers/linear.nim:45-57; the
// projections see seq_len rows at prefill, attn.nim:154-156).
//
// Two launches.  The first rotates the activations once -- x o suh, the 128-group butterfly, 1/sqrt(128),
// rounded to fp16 -- into a workspace, in the fragment order of the matrix cores: every output group needs every
// rotated row, and rotating inside each workgroup would cost more vector work than decoding its weights.  The
// second is the producer/consumer GEMM of ttq_gemm_exl3_pc.h (tiles of 64, 128 or 256 rows x 128 columns, split along K
// while the compute units are not all taken), whose epilogue rotates the 128 sums of each row and applies svh and the
// bias.
//
// Accuracy: the rotated activations are rounded to fp16 once (2^-11 relative per element, about 3e-4
// on a row product); weights are exact fp16, sums fp32.  The decode kernel's two-term split is for
// callers that ask for its accuracy class whatever the row count.
#include "ttq_exl3_common.h"

#include <algorithm>

namespace ttq {

// ---- pass one: Xp = fp16( H(x o suh) / sqrt(128) ) in the fragment order of the matrix cores,
//   Xp[step of 64 k][block of 16 rows][half of 32 k][lane 64] x 16 bytes: row 16 rb + lane % 16, k = 64 ks + 32 h + 8 (lane / 16) .. + 7,
// so that an A fragment of v_mfma_f32_16x16x32_f16 is one kilobyte of consecutive bytes.  A workgroup takes a block of
// 16 rows and one 128-group of k: a half wavefront per row rotates its 128 values in registers (four per lane), the
// 4 KB of results are put in fragment order in LDS and leave as two runs of 2 KB (steps 2 G and 2 G + 1 of the row
// block).  Rows past the end are written as zeros.
template <typename XT>
__global__ void __launch_bounds__(512)
exl3_rotate_pack_kernel(const XT* __restrict__ x, const uint16_t* __restrict__ suh, uint16_t* __restrict__ xp,
                        int64_t rows, int64_t n_in, int row_blocks) {
  __shared__ __attribute__((aligned(16))) uint8_t blk[4096];
  const int tid = threadIdx.x, lane = tid & 63, l32 = tid & 31;
  const int r = tid >> 5;                                    // row of the block
  const int64_t rb = blockIdx.y, grp = blockIdx.x;
  const int64_t row = rb * 16 + r;
  const int64_t k = grp * 128 + 4 * l32;
  uint2 o = make_uint2(0u, 0u);
  if (row < rows) {
    uint2 sraw;
    __builtin_memcpy(&sraw, __builtin_assume_aligned(suh + k, 8), 8);
    float v[4];
    load_x4(x + row * n_in + k, v);
    v[0] *= f16_bits_to_f32((uint16_t)sraw.x);
    v[1] *= f16_bits_to_f32((uint16_t)(sraw.x >> 16));
    v[2] *= f16_bits_to_f32((uint16_t)sraw.y);
    v[3] *= f16_bits_to_f32((uint16_t)(sraw.y >> 16));
    fwht128_quad(v, lane);
    o.x = (uint32_t)f32_to_f16_bits(v[0] * 0.08838834764831845f) | ((uint32_t)f32_to_f16_bits(v[1] * 0.08838834764831845f) << 16);
    o.y = (uint32_t)f32_to_f16_bits(v[2] * 0.08838834764831845f) | ((uint32_t)f32_to_f16_bits(v[3] * 0.08838834764831845f) << 16);
  }
  // k inside the group: 4 * l32 = 64 * step + 32 * half + 8 * g + e
  const int kk = 4 * l32;
  const int st = kk >> 6, h = (kk >> 5) & 1, g = (kk >> 3) & 3, e = kk & 7;
  *reinterpret_cast<uint2*>(blk + (st * 2 + h) * 1024 + (g * 16 + r) * 16 + e * 2) = o;
  __syncthreads();
  // thread t moves bytes 8 t .. 8 t + 7 of the block: the first 2 KB are step 2 grp, the others step 2 grp + 1
  const uint2 v8 = *reinterpret_cast<const uint2*>(blk + tid * 8);
  const int st2 = tid >> 8;
  uint8_t* dst = reinterpret_cast<uint8_t*>(xp) + (((2 * grp + st2) * row_blocks + rb) * 2) * 1024 + (tid & 255) * 8;
  *reinterpret_cast<uint2*>(dst) = v8;
}

// ------------------------------------------------------------------------------ launch
bool gemm_exl3_preferred(int64_t m, int64_t n_out, int64_t n_in) {
  // Measured against passes of the decode kernel (8 rows each; 4096 x 4096, 14336 x 4096, 4096 x 14336, 1024 x 4096 at
  // 8 .. 64 rows): the tiled form wins from the third pass (17 rows) on matrices of 2048 output channels or more, from
  // the second (9 rows: 30.5 against 37 us) on the largest ones, from 48 rows on short ones.
  if (n_in % 128 != 0 || m < 9) return false;
  if (n_out * n_in >= ((int64_t)48 << 20)) return true;
  return m >= 48 || (m >= 17 && n_out >= 2048);
}

constexpr int64_t kXpMaxRows = 4096;       // rows rotated into the workspace at a time

// The producer/consumer form: tiles of 128 rows x 128 columns (64 rows when there are no more; 256 for launches that
// are large enough), and -- while all copies of the tile grid fit one round of workgroups -- 2, 4 or 8 copies along K,
// each with an even number of at least eight 64-k steps: the decode of a tile is paid once per 128 rows, and every
// compute unit gets a share of it.
struct XgChoice { int mb, splits; int64_t tiles; };
static XgChoice xg_choose(int64_t rows, int64_t n_out, int64_t n_in) {
  XgChoice c;
  const int64_t steps = n_in / 64, cus = device_num_cus();
  // 256-row tiles (every tile decoded once per 256 rows, by four producers instead of eight) where they alone give
  // every compute unit a workgroup
  c.mb = (n_out / 128) * ((rows + 255) / 256) >= cus ? 4 : (rows > 64 ? 2 : 1);
  c.tiles = (n_out / 128) * ((rows + 64 * c.mb - 1) / (64 * c.mb));
  c.splits = 1;
  for (int sp = 2; sp <= 8; sp *= 2)
    if (c.tiles * sp <= cus && steps % sp == 0 && (steps / sp) % 2 == 0 && steps / sp >= 8 && c.tiles * 4 <= kPcMaxCounters)
      c.splits = sp;
  return c;
}
static size_t xg_partials_bytes(const XgChoice& c) {
  return c.splits > 1 ? (size_t)c.tiles * 4 * (size_t)c.splits * (size_t)(c.mb * 8 * 1024) : 0;
}
size_t gemm_exl3_partials_bytes(int64_t m, int64_t n_out, int64_t n_in) {
  if (m <= 0 || n_out <= 0 || n_in % 128 != 0) return 0;
  size_t most = 0;
  const int64_t rows[3] = {m < kXpMaxRows ? m : kXpMaxRows, m % kXpMaxRows, 0};
  for (int64_t r : rows)
    if (r > 0) most = std::max(most, xg_partials_bytes(xg_choose(r, n_out, n_in)));
  return most;
}

hipError_t launch_gemm_exl3(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, const void* x,
                            int x_dtype, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                            int64_t n_out, int64_t n_in, int bits, int cb, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (route_probe(kRouteExl3Gemm)) return hipSuccess;
  const int64_t block_rows = m < kXpMaxRows ? m : kXpMaxRows;
  void* ws = nullptr;
  hipError_t e = stream_workspace(kWsExl3Rotated, s, (size_t)((block_rows + 15) / 16 * 16) * n_in * sizeof(uint16_t), &ws);
  uint16_t* xr = static_cast<uint16_t*>(ws);
  if (e != hipSuccess) return e;
  const int64_t xsize = x_dtype == kF32 ? 4 : 2;
  // partial sums and arrival counters of launches split along K: asked for once, for the largest need of any chunk
  void* part = nullptr;
  void* cnt = nullptr;
  {
    const size_t pbytes = gemm_exl3_partials_bytes(m, n_out, n_in);
    if (pbytes > 0) {
      e = stream_workspace(kWsGemmPartials, s, pbytes, &part);
      if (e == hipSuccess) e = stream_workspace(kWsGemmCounters, s, (size_t)kPcMaxCounters * 4, &cnt, true);
      if (e != hipSuccess) return e;
    }
  }
  for (int64_t r0 = 0; r0 < m; r0 += kXpMaxRows) {
    const int64_t rows = m - r0 < kXpMaxRows ? m - r0 : kXpMaxRows;
    const char* xb = static_cast<const char*>(x) + r0 * n_in * xsize;
    // rotated activations in fragment order, then the tiled GEMM (n_in is a whole number of Hadamard groups, i.e. an
    // even number of 64-k steps)
    const int row_blocks = (int)((rows + 15) / 16);
    const dim3 rgrid((unsigned)(n_in / 128), (unsigned)row_blocks), rblock(512);
    switch (x_dtype) {
      case kF32:
        hipLaunchKernelGGL(exl3_rotate_pack_kernel<float>, rgrid, rblock, 0, s, reinterpret_cast<const float*>(xb), suh,
                           xr, rows, n_in, row_blocks);
        break;
      case kF16:
        hipLaunchKernelGGL(exl3_rotate_pack_kernel<f16_tag>, rgrid, rblock, 0, s, reinterpret_cast<const f16_tag*>(xb),
                           suh, xr, rows, n_in, row_blocks);
        break;
      case kBF16:
        hipLaunchKernelGGL(exl3_rotate_pack_kernel<bf16_tag>, rgrid, rblock, 0, s, reinterpret_cast<const bf16_tag*>(xb),
                           suh, xr, rows, n_in, row_blocks);
        break;
      default: return hipErrorInvalidValue;
    }
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    void* yb = static_cast<char*>(y) + r0 * n_out * (y_dtype == kF32 ? 4 : 2);
    const XgChoice c = xg_choose(rows, n_out, n_in);
    PcSplit sp{1, 0, nullptr, nullptr};
    if (c.splits > 1) {
      if (!part || !cnt) return hipErrorInvalidValue;
      sp.splits = c.splits;
      sp.partials = static_cast<float*>(part);
      sp.counters = static_cast<uint32_t*>(cnt);
    }
    e = launch_gemm_exl3_pc(bits, cb, c.mb, trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, sp, s);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace ttq
