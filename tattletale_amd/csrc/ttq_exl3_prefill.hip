// Trellis-coded (EXL3-style) linear layer for many activation rows: Y = svh o H( T * H(suh o X^T) ),
// the prefill side of Linear.forward (workspace/transformers/src/layers/linear.nim:45-57; the
// projections see seq_len rows at prefill, attn.nim:154-156).
//
// Two launches.  The first rotates the activations once -- x o suh, the 128-group butterfly, 1/sqrt(128),
// rounded to fp16 -- into a workspace: every output group needs every rotated row, and the rotation of a
// pass of 64 rows would cost a workgroup more vector work than decoding the pass's weights.  The second
// is the decode GEMV's workgroup (128 output channels, 16 wavefronts, weights staged through LDS as a
// big-endian bit string, four weights per lane decoded into an A fragment) with 64 rows per workgroup:
// each pair of decoded fragments feeds four v_mfma_f32_16x16x32_f16, one per block of 16 rows, so the decode --
// which bounds the single-row kernel -- is paid once per 64 rows; a wavefront takes two tile columns, so
// that every activation fragment it reads from LDS serves two of them.  A workgroup covers the whole
// reduction, rotates its 64 x 128 sums and writes y; no workspace is shared between workgroups.
//
// Accuracy: the rotated activations are rounded to fp16 once (2^-11 relative per element, about 3e-4
// on a row product); weights are exact fp16, sums fp32.  The decode kernel's two-term split is for
// callers that ask for its accuracy class whatever the row count.
#include "ttq_exl3_common.h"

namespace ttq {

constexpr int kXpRows = 64;                                   // activation rows per workgroup
constexpr int kXpRowBlocks = kXpRows / 16;
// A wavefront takes two adjacent tile columns and two of every group's eight k-tiles: a B fragment (16 rows x 16 k
// of activations) read from LDS then serves two matrix instructions instead of one.
constexpr int kXpCols = 2;                                    // tile columns per wavefront
constexpr int kXpKParts = kXmThreads / kWave / (8 / kXpCols); // wavefronts along k: 4
constexpr int kXpTiles = 8 / kXpKParts;                       // k-tiles of a group per wavefront: 2
constexpr int kXpXPieces = kXpRows * (kXmChunkK / 8) / kXmThreads;   // 16-byte pieces of X per thread and pass

// ---- pass one: Xr[row][k] = fp16( H(x o suh) / sqrt(128) ), one 32-lane half wavefront per (row, 128-group)
template <typename XT>
__global__ void __launch_bounds__(256)
exl3_rotate_rows_kernel(const XT* __restrict__ x, const uint16_t* __restrict__ suh, uint16_t* __restrict__ xr,
                        int64_t items, int groups_per_row, int64_t n_in) {
  const int lane = threadIdx.x & 63, l32 = threadIdx.x & 31;
  const int64_t item = (int64_t)blockIdx.x * (256 / 32) + (threadIdx.x >> 5);
  if (item >= items) return;
  const int64_t row = item / groups_per_row;
  const int64_t k = (item - row * groups_per_row) * 128 + 4 * l32;
  uint2 sraw;
  __builtin_memcpy(&sraw, __builtin_assume_aligned(suh + k, 8), 8);
  float v[4];
  load_x4(x + row * n_in + k, v);
  v[0] *= f16_bits_to_f32((uint16_t)sraw.x);
  v[1] *= f16_bits_to_f32((uint16_t)(sraw.x >> 16));
  v[2] *= f16_bits_to_f32((uint16_t)sraw.y);
  v[3] *= f16_bits_to_f32((uint16_t)(sraw.y >> 16));
  fwht128_quad(v, lane);
  uint2 o;
  o.x = (uint32_t)f32_to_f16_bits(v[0] * 0.08838834764831845f) | ((uint32_t)f32_to_f16_bits(v[1] * 0.08838834764831845f) << 16);
  o.y = (uint32_t)f32_to_f16_bits(v[2] * 0.08838834764831845f) | ((uint32_t)f32_to_f16_bits(v[3] * 0.08838834764831845f) << 16);
  __builtin_memcpy(__builtin_assume_aligned(xr + row * n_in + k, 8), &o, 8);
}

// ---- pass two
template <int BITS, int CB>
__global__ void __launch_bounds__(kXmThreads)
gemm_exl3_mfma_kernel(const uint16_t* __restrict__ trellis, const uint16_t* __restrict__ svh,
                      const uint16_t* __restrict__ xr, void* __restrict__ y, int y_dtype, const void* __restrict__ bias,
                      int bias_dtype, int m, int n_out, int n_in) {
  using G = XmGeom<BITS>;
  // one pass of tiles, then 64 rows of rotated activations; the epilogue's sums reuse the activations' space
  __shared__ uint32_t slab[G::kSlabDw];
  __shared__ __attribute__((aligned(16))) _Float16 xs[kXpRows * kXmColStride];
  static_assert(sizeof(_Float16) * kXpRows * kXmColStride >= sizeof(float) * 2 * kXpRows * 128, "two copies of the sums fit");

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = blockIdx.x;
  const int t0 = blockIdx.y * kXpRows;
  const int rows = min(kXpRows, m - t0);
  const int nt_n = n_out >> 4, kt_n = n_in >> 4;
  const int col = lane & 15, q = lane >> 4;
  const int tcol0 = (wave & 3) * kXpCols, kpart = wave >> 2;

  XmLane<BITS> ln;
  ln.init(lane);

  const char* wbase = reinterpret_cast<const char*>(trellis) + (int64_t)grp * 8 * (32 * BITS);
  const int64_t row_bytes = (int64_t)nt_n * (32 * BITS);
  uint4 pre[G::kSets];
  uint4 xpre[kXpXPieces];
  auto request = [&](int kt_first, int cnt) {
    // activations first: piece p = (row, 8 columns); rows past the end re-read the last row
#pragma unroll
    for (int i = 0; i < kXpXPieces; i++) {
      const int p = tid + i * kXmThreads;
      const int r = p >> 6, c = p & 63;
      xpre[i] = *reinterpret_cast<const uint4*>(xr + (int64_t)(t0 + min(r, rows - 1)) * n_in + (int64_t)kt_first * 16 +
                                                min(c, 2 * cnt - 1) * 8);
    }
#pragma unroll
    for (int i = 0; i < G::kSets; i++) {
      const int p = tid + i * kXmThreads;
      const int ktl = p / G::kRunPieces, r = p - ktl * G::kRunPieces;
      pre[i] = *reinterpret_cast<const uint4*>(wbase + (int64_t)(kt_first + min(ktl, cnt - 1)) * row_bytes + r * 16);
    }
  };
  auto stage = [&](int cnt) {
#pragma unroll
    for (int i = 0; i < kXpXPieces; i++) {
      const int p = tid + i * kXmThreads;
      const int r = p >> 6, c = p & 63;
      *reinterpret_cast<uint4*>(xs + r * kXmColStride + c * 8) = xpre[i];
    }
#pragma unroll
    for (int i = 0; i < G::kSets; i++) {
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
    }
  };

  request(0, min(kXmChunkTiles, kt_n));

  f32x4_t acc[kXpCols][kXpRowBlocks];
#pragma unroll
  for (int c = 0; c < kXpCols; c++)
#pragma unroll
    for (int rb = 0; rb < kXpRowBlocks; rb++) acc[c][rb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  constexpr int kWin = XmLane<BITS>::kWin;
  const uint32_t* wcol = slab + 1 + (kpart * kXpTiles * 8 + tcol0) * G::kTileStride;
  const _Float16* xcol = xs + col * kXmColStride + kpart * kXpTiles * 16 + 4 * q;

  for (int kt0 = 0; kt0 < kt_n; kt0 += kXmChunkTiles) {
    const int cnt = min(kXmChunkTiles, kt_n - kt0);       // a multiple of 8
    const int ngl = cnt >> 3;
    if (kt0 != 0) __syncthreads();                          // the previous pass has been read
    stage(cnt);
    if (kt0 + kXmChunkTiles < kt_n) request(kt0 + kXmChunkTiles, min(kXmChunkTiles, kt_n - kt0 - kXmChunkTiles));
    __syncthreads();
    // this wavefront's tile column and its share of every group's 8 k-tiles; a group's window dwords are
    // read while the group before it is decoded, the B fragments right before their matrix instructions
    uint32_t cw[2][kXpTiles][kXpCols][kWin][2];
    auto fetch_group = [&](int gl, int buf) {
#pragma unroll
      for (int i = 0; i < kXpTiles; i++)
#pragma unroll
        for (int c = 0; c < kXpCols; c++) ln.fetch(wcol + ((gl * 8 + i) * 8 + c) * G::kTileStride, cw[buf][i][c]);
    };
    // The wavefront's two k-tiles of a group go through one v_mfma_f32_16x16x32_f16: a lane's eight k positions
    // are its four of the first tile followed by its four of the second -- any assignment of the 32 k's to
    // (lane group, element) does, as long as the activation fragment uses the same one -- so the decode and the
    // LDS reads are those of the 16-k form and there are half as many matrix instructions, each as long as
    // one of those (measured: 19 ns per instruction and wavefront for either, all SIMDs busy).
    auto compute_group = [&](int gl, int buf) {
      static_assert(kXpTiles == 2, "two k-tiles per matrix instruction");
      f16x8_t a[kXpCols];
#pragma unroll
      for (int c = 0; c < kXpCols; c++) {
        const f16x4_t a0 = ln.template decode<CB>(cw[buf][0][c]), a1 = ln.template decode<CB>(cw[buf][1][c]);
        a[c] = f16x8_t{a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      }
      const _Float16* xb = xcol + gl * 8 * 16;
#pragma unroll
      for (int rb = 0; rb < kXpRowBlocks; rb++) {
        const f16x4_t b0 = *reinterpret_cast<const f16x4_t*>(xb + rb * 16 * kXmColStride);
        const f16x4_t b1 = *reinterpret_cast<const f16x4_t*>(xb + 16 + rb * 16 * kXmColStride);
        const f16x8_t b = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
#pragma unroll
        for (int c = 0; c < kXpCols; c++) acc[c][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[c], b, acc[c][rb], 0, 0, 0);
      }
    };
    fetch_group(0, 0);
    for (int gl = 0; gl < ngl; gl += 2) {
      if (gl + 1 < ngl) fetch_group(gl + 1, 1);
      compute_group(gl, 0);
      if (gl + 1 < ngl) {
        if (gl + 2 < ngl) fetch_group(gl + 2, 0);
        compute_group(gl + 1, 1);
      }
    }
  }

  // ---- the sums of the workgroup's four k parts meet in LDS (over the activations, which are done with): parts 0
  // and 1 write a copy each, then parts 2 and 3 add theirs onto them -- every element by the lane that owns it
  __syncthreads();
  float* yp = reinterpret_cast<float*>(xs);
#pragma unroll
  for (int round = 0; round < 2; round++) {
    if ((kpart >> 1) == round) {
      float* dst = yp + (kpart & 1) * (kXpRows * 128);
#pragma unroll
      for (int c = 0; c < kXpCols; c++)
#pragma unroll
        for (int rb = 0; rb < kXpRowBlocks; rb++) {
          const int r = rb * 16 + col;
          if (r < rows) {
            float4* p4 = reinterpret_cast<float4*>(dst + r * 128 + (tcol0 + c) * 16 + 4 * q);
            float4 v = make_float4(acc[c][rb][0], acc[c][rb][1], acc[c][rb][2], acc[c][rb][3]);
            if (round == 1) {
              const float4 o = *p4;
              v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
            }
            *p4 = v;
          }
        }
    }
    __syncthreads();
  }
  // ---- output side: rotate the 128 sums of each row, svh, bias; 32 lanes per row
  {
    const int hw = tid >> 5, l32 = tid & 31;
    const int n = grp * 128 + 4 * l32;
    uint2 sraw;
    __builtin_memcpy(&sraw, __builtin_assume_aligned(svh + n, 8), 8);
    const float svf[4] = {f16_bits_to_f32((uint16_t)sraw.x), f16_bits_to_f32((uint16_t)(sraw.x >> 16)),
                          f16_bits_to_f32((uint16_t)sraw.y), f16_bits_to_f32((uint16_t)(sraw.y >> 16))};
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
      for (int i = 0; i < 4; i++) bv[i] = load_bias(bias, bias_dtype, n + i);
    }
    for (int r = hw; r < rows; r += kXmThreads / 32) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kp = 0; kp < 2; kp++) {
        const float4 t = *reinterpret_cast<const float4*>(yp + kp * (kXpRows * 128) + r * 128 + 4 * l32);
        v[0] += t.x; v[1] += t.y; v[2] += t.z; v[3] += t.w;
      }
      fwht128_quad(v, lane);
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; i++) o[i] = v[i] * 0.08838834764831845f * svf[i] + bv[i];
      xm_store4(y, y_dtype, (int64_t)(t0 + r) * n_out + n, o);
    }
  }
}

// ------------------------------------------------------------------------------ launch
bool gemm_exl3_preferred(int64_t m, int64_t n_out, int64_t n_in) {
  // worth it once the 64-row workgroups cover at least half of the compute units; below that the decode
  // kernel's 8-row groups spread over more of them
  const int64_t wgs = (n_out / 128) * ((m + kXpRows - 1) / kXpRows);
  return m >= 16 && n_in % 128 == 0 && wgs * 2 >= device_num_cus();
}

template <int BITS>
static hipError_t xp_launch(const uint16_t* trellis, const uint16_t* svh, const uint16_t* xr, void* y, int y_dtype,
                            const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int cb,
                            hipStream_t s) {
  const dim3 grid((unsigned)(n_out / 128), (unsigned)((m + kXpRows - 1) / kXpRows)), block(kXmThreads);
  if (cb == 0)
    hipLaunchKernelGGL((gemm_exl3_mfma_kernel<BITS, 0>), grid, block, 0, s, trellis, svh, xr, y, y_dtype, bias,
                       bias_dtype, (int)m, (int)n_out, (int)n_in);
  else
    hipLaunchKernelGGL((gemm_exl3_mfma_kernel<BITS, 1>), grid, block, 0, s, trellis, svh, xr, y, y_dtype, bias,
                       bias_dtype, (int)m, (int)n_out, (int)n_in);
  return hipGetLastError();
}

constexpr int64_t kXpMaxRows = 4096;       // rows rotated into the workspace at a time

hipError_t launch_gemm_exl3(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, const void* x,
                            int x_dtype, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                            int64_t n_out, int64_t n_in, int bits, int cb, hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (route_probe(kRouteExl3Gemm)) return hipSuccess;
  const int64_t block_rows = m < kXpMaxRows ? m : kXpMaxRows;
  void* ws = nullptr;
  hipError_t e = stream_workspace(kWsExl3Rotated, s, (size_t)block_rows * n_in * sizeof(uint16_t), &ws);
  uint16_t* xr = static_cast<uint16_t*>(ws);
  if (e != hipSuccess) return e;
  const int64_t xsize = x_dtype == kF32 ? 4 : 2;
  for (int64_t r0 = 0; r0 < m; r0 += kXpMaxRows) {
    const int64_t rows = m - r0 < kXpMaxRows ? m - r0 : kXpMaxRows;
    const char* xb = static_cast<const char*>(x) + r0 * n_in * xsize;
    const int groups_per_row = (int)(n_in / 128);
    const int64_t items = rows * groups_per_row;
    const dim3 rgrid((unsigned)((items + 7) / 8)), rblock(256);
    switch (x_dtype) {
      case kF32:
        hipLaunchKernelGGL(exl3_rotate_rows_kernel<float>, rgrid, rblock, 0, s, reinterpret_cast<const float*>(xb), suh,
                           xr, items, groups_per_row, n_in);
        break;
      case kF16:
        hipLaunchKernelGGL(exl3_rotate_rows_kernel<f16_tag>, rgrid, rblock, 0, s, reinterpret_cast<const f16_tag*>(xb),
                           suh, xr, items, groups_per_row, n_in);
        break;
      case kBF16:
        hipLaunchKernelGGL(exl3_rotate_rows_kernel<bf16_tag>, rgrid, rblock, 0, s, reinterpret_cast<const bf16_tag*>(xb),
                           suh, xr, items, groups_per_row, n_in);
        break;
      default: return hipErrorInvalidValue;
    }
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    void* yb = static_cast<char*>(y) + r0 * n_out * (y_dtype == kF32 ? 4 : 2);
    switch (bits) {
      case 1: e = xp_launch<1>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 2: e = xp_launch<2>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 3: e = xp_launch<3>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 4: e = xp_launch<4>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 5: e = xp_launch<5>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 6: e = xp_launch<6>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 7: e = xp_launch<7>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      case 8: e = xp_launch<8>(trellis, svh, xr, yb, y_dtype, bias, bias_dtype, rows, n_out, n_in, cb, s); break;
      default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace ttq
