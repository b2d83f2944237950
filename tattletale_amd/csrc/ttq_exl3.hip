// EXL3-style trellis-coded weights on gfx950: tile decoder, decode GEMV with the input-side
// Hadamard rotation fused into its prologue, and the 128-group Hadamard epilogue.
//
//   y = svh o H( T * H(suh o x) )
//
// T (n_out, n_in) are the decoded trellis values, H the orthonormal Sylvester-Hadamard
// transform applied to each group of 128, suh/svh fp16 vectors.  This is the quantized
// counterpart of F.linear(x, weight) (workspace/libtorch/src/abi/neural_nets.nim:64-81);
// the reference holds only the format's metadata
// (workspace/transformers/tests/fixtures/configs/config-GLM-4.7-EXL3-3.84bpw.json:43-54).
//
// Format.  A 16x16 tile is one cyclic string of 256*bits bits kept in 16*bits u16 words,
// most significant bit of each word first.  Weight i = 16*n_local + k_local is decoded
// from the 16-bit window that starts at bit i*bits.  Tiles are laid out
// trellis[k_tile][n_tile][16*bits].  Because 16*bits is a multiple of 16, the 16 weights
// of one output channel inside a tile start on a word boundary and span bits+1 words; one
// lane decodes exactly those 16 weights, so all window shifts are compile-time constants.
#include "ttq_exl3_common.h"

namespace ttq {

// The bits+1 words that hold the 16 windows of output channel j of a tile, as big-endian
// 32-bit chunks (first stream bit = bit 31 of chunk 0).
template <int BITS>
struct LaneBits {
  static constexpr int kWords = BITS + 1;
  static constexpr int kChunks = (kWords + 1) / 2;
  uint32_t c[kChunks];
  // One load of the 2 * kWords bytes plus the tile's first word.  Channels 0..14 read their words
  // where they lie; channel 15, whose last word is the tile's first (the string is cyclic), starts
  // one word early so that it never reads past the tile, and shifts by a word while the 16-bit
  // halves are swapped into stream order (a byte permute either way).
  __device__ __forceinline__ void load(const uint16_t* tile, int j) {
    const bool last = j == 15;
    const uint16_t* p = tile + j * BITS - (last ? 1 : 0);
    uint16_t w[kWords];
    __builtin_memcpy(w, __builtin_assume_aligned(p, 2), 2 * kWords);
    const uint32_t wrap = tile[0];
    // little-endian dwords of the words, continued by the wrap word: d[i] = w[2i] | w[2i+1] << 16
    uint32_t d[kChunks + 1];
#pragma unroll
    for (int i = 0; i <= kChunks; i++) {
      const uint32_t lo = 2 * i < kWords ? (uint32_t)w[2 * i] : (2 * i == kWords ? wrap : 0u);
      const uint32_t hi = 2 * i + 1 < kWords ? (uint32_t)w[2 * i + 1] : (2 * i + 1 == kWords ? wrap : 0u);
      d[i] = lo | (hi << 16);
    }
    // channels 0..14: (w[2t] << 16) | w[2t+1]; channel 15: (w[2t+1] << 16) | w[2t+2]
    const uint32_t sel = last ? 0x03020504u : 0x01000302u;
#pragma unroll
    for (int t = 0; t < kChunks; t++) c[t] = __builtin_amdgcn_perm(d[t + 1], d[t], sel);
  }
  // the window of weight KK in bits 0..15; bits 16..31 hold whatever precedes it in the stream
  template <int KK>
  __device__ __forceinline__ uint32_t state() const {
    constexpr int q = KK * BITS;
    constexpr int ci = q >> 5, o = q & 31;
    if constexpr (o == 16) {
      return c[ci];
    } else if constexpr (o < 16) {
      return c[ci] >> (16 - o);
    } else {
      return __builtin_amdgcn_alignbit(c[ci], c[ci + 1 < kChunks ? ci + 1 : ci], 48 - o);
    }
  }
};

template <int BITS, int CB, int KK>
struct DecodeLoop {
  static __device__ __forceinline__ void run(const LaneBits<BITS>& lb, const Codebook<CB>& cb, _Float16* out) {
    out[KK] = cb.code(lb.template state<KK>());
    if constexpr (KK + 1 < 16) DecodeLoop<BITS, CB, KK + 1>::run(lb, cb, out);
  }
};

// ------------------------------------------------------------------ tile decoder
// One thread per (tile, output channel): writes 16 consecutive fp16 values of a row.
template <int BITS, int CB>
__global__ void __launch_bounds__(256) dequant_exl3_kernel(const uint16_t* __restrict__ trellis,
                                                           uint16_t* __restrict__ out, int nt_n,
                                                           int64_t nthreads, int n_in) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= nthreads) return;
  const int j = (int)(g & 15);
  const int64_t tile = g >> 4;
  const int64_t kt = tile / nt_n, nt = tile % nt_n;
  LaneBits<BITS> lb;
  lb.load(trellis + tile * (16 * BITS), j);
  Codebook<CB> cb;
  cb.init();
  _Float16 v[16];
  DecodeLoop<BITS, CB, 0>::run(lb, cb, v);
  uint16_t* o = out + (nt * 16 + j) * (int64_t)n_in + kt * 16;
#pragma unroll
  for (int kk = 0; kk < 16; kk++) {
    uint16_t b;
    __builtin_memcpy(&b, &v[kk], 2);
    o[kk] = b;
  }
}

// ------------------------------------------------------------------ GEMV
constexpr int kExl3Threads = 1024;
constexpr int kExl3Waves = kExl3Threads / kWave;

// One workgroup per n_tile (16 output channels).  Lane = (k-tile slot g = lane/16, channel
// j = lane%16); the 16 waves times 4 slots walk the k tiles 64 at a time.  Partial sums are
// combined across slots with lane shuffles and across waves through LDS.
// The packed bits of a lane's first kPre tiles are requested before anything else, so that they
// travel while the activations are loaded and rotated; later tiles are requested one batch ahead.
// TOK activation rows ("tokens") per workgroup: decoding a weight costs about ten vector-ALU
// issue slots, multiplying it one per token, so the decode is shared by up to eight tokens
// (blockIdx.y walks the groups of TOK tokens; the last group may hold fewer).
template <int BITS, int CB, typename XT, int TOK>
__global__ void __launch_bounds__(kExl3Threads)
gemv_exl3_kernel(const uint16_t* __restrict__ trellis, const uint16_t* __restrict__ suh,
                 const XT* __restrict__ x, float* __restrict__ y, int m, int n_out, int n_in) {
  extern __shared__ float xs[];          // TOK x n_in rotated activations, then kExl3Waves*16*TOK partials
  constexpr int kPre = 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t0 = blockIdx.y * TOK;
  const int ntok = min(TOK, m - t0);       // tokens of this group that exist
  const int nt = blockIdx.x, nt_n = n_out >> 4, kt_n = n_in >> 4;
  const int g = lane >> 4, j = lane & 15;
  const int kt0 = wave * 4 + g;
  constexpr int kStride = kExl3Waves * 4;

  LaneBits<BITS> cur[kPre];
  auto load_batch = [&](LaneBits<BITS> (&dst)[kPre], int kt_first) {
#pragma unroll
    for (int i = 0; i < kPre; i++) {
      const int kt = min(kt_first + i * kStride, kt_n - 1);     // past the end: a harmless re-read
      dst[i].load(trellis + ((int64_t)kt * nt_n + nt) * (16 * BITS), j);
    }
  };
  load_batch(cur, kt0);

  // input side: x o suh, then the Hadamard rotation of every group of 128 (32 lanes x 4 values)
  for (int k4 = tid * 4; k4 < n_in; k4 += kExl3Threads * 4) {
    uint2 sraw;
    __builtin_memcpy(&sraw, __builtin_assume_aligned(suh + k4, 8), 8);
    const float sg[4] = {f16_bits_to_f32((uint16_t)sraw.x), f16_bits_to_f32((uint16_t)(sraw.x >> 16)),
                         f16_bits_to_f32((uint16_t)sraw.y), f16_bits_to_f32((uint16_t)(sraw.y >> 16))};
#pragma unroll
    for (int t = 0; t < TOK; t++) {
      if (t < ntok) {          // uniform; no `break`, so that the loop unrolls and acc[] stays in registers
        const XT* xm = x + (int64_t)(t0 + t) * n_in;
        float v[4];
        load_x4(xm + k4, v);
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] *= sg[i];
        fwht128_quad(v, lane);
        *reinterpret_cast<float4*>(xs + (size_t)t * n_in + k4) = make_float4(v[0], v[1], v[2], v[3]);
      }
    }
  }
  __syncthreads();
  const float kNorm = 0.08838834764831845f;  // 1/sqrt(128), applied to the dot product

  Codebook<CB> cb;
  cb.init();
  // two partial sums per token (even and odd quads of the tile row): independent chains for the
  // multiply-adds
  float acc[TOK][2];
#pragma unroll
  for (int t = 0; t < TOK; t++) acc[t][0] = acc[t][1] = 0.f;
  for (int ktb = kt0; ktb < kt_n; ktb += kPre * kStride) {
    LaneBits<BITS> nxt[kPre];
    const bool more = ktb + kPre * kStride < kt_n;
    if (more) load_batch(nxt, ktb + kPre * kStride);
#pragma unroll
    for (int i = 0; i < kPre; i++) {
      const int kt = ktb + i * kStride;
      if (kt < kt_n) {
        _Float16 v[16];
        DecodeLoop<BITS, CB, 0>::run(cur[i], cb, v);
#pragma unroll
        for (int t = 0; t < TOK; t++) {
          if (t < ntok) {
            const float4* xv = reinterpret_cast<const float4*>(xs + (size_t)t * n_in + 16 * kt);
#pragma unroll
            for (int q = 0; q < 4; q++) {
              const float4 xq = xv[q];
              float a = acc[t][q & 1];
              a = fmaf_((float)v[4 * q + 0], xq.x, a);
              a = fmaf_((float)v[4 * q + 1], xq.y, a);
              a = fmaf_((float)v[4 * q + 2], xq.z, a);
              a = fmaf_((float)v[4 * q + 3], xq.w, a);
              acc[t][q & 1] = a;
            }
          }
        }
      }
    }
    if (more) {
#pragma unroll
      for (int i = 0; i < kPre; i++) cur[i] = nxt[i];
    }
  }
  float* red = xs + (size_t)TOK * n_in;
#pragma unroll
  for (int t = 0; t < TOK; t++) {
    float a = acc[t][0] + acc[t][1];
    a = add_xor16(a);
    a = add_xor32(a);
    if (lane < 16) red[(t * kExl3Waves + wave) * 16 + lane] = a;
  }
  __syncthreads();
  if (tid < 16 * TOK) {
    const int t = tid >> 4, c = tid & 15;
    float s = 0.f;
#pragma unroll
    for (int wv = 0; wv < kExl3Waves; wv++) s += red[(t * kExl3Waves + wv) * 16 + c];
    if (t0 + t < m) y[(int64_t)(t0 + t) * n_out + nt * 16 + c] = s * kNorm;
  }
}

// ------------------------------------------------------------------ Hadamard epilogue
// One wavefront per 128-group: v <- post o H(pre o v) (+ bias), in place.  Lane l holds elements
// l and l + 64: stages 1..32 against the lanes 1..32 away, stage 64 inside the lane (the stage
// order of the textbook loop).  `period` is the length after which pre/post/bias repeat (n_out
// for batched outputs).
constexpr int kHadThreads = 256;
__global__ void __launch_bounds__(kHadThreads)
hadamard128_kernel(float* __restrict__ v, const uint16_t* __restrict__ pre,
                   const uint16_t* __restrict__ post, const void* __restrict__ bias, int bias_dtype,
                   int64_t period, int64_t groups) {
  const int lane = threadIdx.x & 63;
  const int64_t grp = (int64_t)blockIdx.x * (kHadThreads / kWave) + (threadIdx.x >> 6);
  if (grp >= groups) return;
  float a[2];
  int64_t ch[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int64_t idx = grp * 128 + lane + 64 * h;
    ch[h] = idx % period;
    a[h] = v[idx];
    if (pre) a[h] *= f16_bits_to_f32(pre[ch[h]]);
  }
  fwht_lane_stage<1>(a, lane);
  fwht_lane_stage<2>(a, lane);
  fwht_lane_stage<4>(a, lane);
  fwht_lane_stage<8>(a, lane);
  fwht_lane_stage<16>(a, lane);
  fwht_lane_stage<32>(a, lane);
  const float lo = a[0] + a[1], hi = a[0] - a[1];
  a[0] = lo;
  a[1] = hi;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    float r = a[h] * 0.08838834764831845f;
    if (post) r *= f16_bits_to_f32(post[ch[h]]);
    if (bias) {
      if (bias_dtype == kF32) r += static_cast<const float*>(bias)[ch[h]];
      else {
        const uint16_t b = static_cast<const uint16_t*>(bias)[ch[h]];
        r += (bias_dtype == kF16) ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
      }
    }
    v[grp * 128 + lane + 64 * h] = r;
  }
}

// ------------------------------------------------------------------ launchers
template <int BITS>
static hipError_t dequant_bits(const uint16_t* trellis, uint16_t* out, int64_t n_out, int64_t n_in,
                               int cb, hipStream_t s) {
  const int nt_n = (int)(n_out / 16);
  const int64_t nthreads = (n_out / 16) * (n_in / 16) * 16;
  if (nthreads == 0) return hipSuccess;
  const dim3 grid((unsigned)((nthreads + 255) / 256)), block(256);
  if (cb == 0)
    hipLaunchKernelGGL((dequant_exl3_kernel<BITS, 0>), grid, block, 0, s, trellis, out, nt_n, nthreads, (int)n_in);
  else
    hipLaunchKernelGGL((dequant_exl3_kernel<BITS, 1>), grid, block, 0, s, trellis, out, nt_n, nthreads, (int)n_in);
  return hipGetLastError();
}

hipError_t launch_dequant_exl3(const uint16_t* trellis, uint16_t* out_f16, int64_t n_out, int64_t n_in,
                               int bits, int cb, hipStream_t s) {
  switch (bits) {
    case 1: return dequant_bits<1>(trellis, out_f16, n_out, n_in, cb, s);
    case 2: return dequant_bits<2>(trellis, out_f16, n_out, n_in, cb, s);
    case 3: return dequant_bits<3>(trellis, out_f16, n_out, n_in, cb, s);
    case 4: return dequant_bits<4>(trellis, out_f16, n_out, n_in, cb, s);
    case 5: return dequant_bits<5>(trellis, out_f16, n_out, n_in, cb, s);
    case 6: return dequant_bits<6>(trellis, out_f16, n_out, n_in, cb, s);
    case 7: return dequant_bits<7>(trellis, out_f16, n_out, n_in, cb, s);
    case 8: return dequant_bits<8>(trellis, out_f16, n_out, n_in, cb, s);
    default: return hipErrorInvalidValue;
  }
}

constexpr int kExl3Tok = 8;              // tokens per workgroup when there are several and they fit LDS
template <int BITS, int CB, typename XT, int TOK>
static hipError_t gemv_bits_cb_t(const uint16_t* trellis, const uint16_t* suh, const void* x, float* y, int64_t m,
                                 int64_t n_out, int64_t n_in, hipStream_t s) {
  const dim3 grid((unsigned)(n_out / 16), (unsigned)((m + TOK - 1) / TOK)), block(kExl3Threads);
  const size_t lds = ((size_t)TOK * n_in + (size_t)kExl3Waves * 16 * TOK) * sizeof(float);
  auto kernel = gemv_exl3_kernel<BITS, CB, XT, TOK>;
  if (lds > 64 * 1024) {
    static LargeLds configured;
    {
      const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kernel), configured);
      if (e != hipSuccess) return e;
    }
  }
  hipLaunchKernelGGL(kernel, grid, block, lds, s, trellis, suh, static_cast<const XT*>(x), y, (int)m, (int)n_out,
                     (int)n_in);
  return hipGetLastError();
}

template <int BITS, int CB, typename XT>
static hipError_t gemv_bits_cb_x(const uint16_t* trellis, const uint16_t* suh, const void* x, float* y, int64_t m,
                                 int64_t n_out, int64_t n_in, hipStream_t s) {
  const size_t lds8 = ((size_t)kExl3Tok * n_in + (size_t)kExl3Waves * 16 * kExl3Tok) * sizeof(float);
  if (m >= 2 && lds8 <= 150 * 1024)
    return gemv_bits_cb_t<BITS, CB, XT, kExl3Tok>(trellis, suh, x, y, m, n_out, n_in, s);
  return gemv_bits_cb_t<BITS, CB, XT, 1>(trellis, suh, x, y, m, n_out, n_in, s);
}

template <int BITS, int CB>
static hipError_t gemv_bits_cb(const uint16_t* trellis, const uint16_t* suh, const void* x, int x_dtype,
                               float* y, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s) {
  switch (x_dtype) {
    case kF32: return gemv_bits_cb_x<BITS, CB, float>(trellis, suh, x, y, m, n_out, n_in, s);
    case kF16: return gemv_bits_cb_x<BITS, CB, f16_tag>(trellis, suh, x, y, m, n_out, n_in, s);
    case kBF16: return gemv_bits_cb_x<BITS, CB, bf16_tag>(trellis, suh, x, y, m, n_out, n_in, s);
    default: return hipErrorInvalidValue;
  }
}

template <int BITS>
static hipError_t gemv_bits(const uint16_t* trellis, const uint16_t* suh, const void* x, int x_dtype,
                            float* y, int64_t m, int64_t n_out, int64_t n_in, int cb, hipStream_t s) {
  return cb == 0 ? gemv_bits_cb<BITS, 0>(trellis, suh, x, x_dtype, y, m, n_out, n_in, s)
                 : gemv_bits_cb<BITS, 1>(trellis, suh, x, x_dtype, y, m, n_out, n_in, s);
}

hipError_t launch_gemv_exl3(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                            const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int bits, int cb,
                            hipStream_t s) {
  if (m == 0 || n_out == 0) return hipSuccess;
  hipError_t e;
  static const int two_launches = dev_knob("TTQ_EXL3_TWO_LAUNCHES", 0);
  if (!two_launches || n_in > kMaxGemvInF32) {      // (the two-launch form stages a whole row of activations in LDS)
    const Exl3Plan plan = exl3_mfma_plan(m, n_out, n_in);
    if (route_probe(plan.slices > 1 ? kRouteExl3GemvSliced : kRouteExl3Gemv)) return hipSuccess;
    unsigned long long* accum = nullptr;
    if (plan.slices > 1) {
      e = exl3_workspace(s, &accum);
      if (e != hipSuccess) return e;
    }
    return launch_gemv_exl3_mfma(plan, trellis, suh, svh, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, bits,
                                 cb, accum, s);
  }
  if (route_probe(kRouteExl3GemvTwoLaunches)) return hipSuccess;
  if (y_dtype != kF32) return hipErrorInvalidValue;     // the two-kernel form rotates an fp32 buffer in place
  float* yf = static_cast<float*>(y);
  switch (bits) {
    case 1: e = gemv_bits<1>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 2: e = gemv_bits<2>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 3: e = gemv_bits<3>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 4: e = gemv_bits<4>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 5: e = gemv_bits<5>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 6: e = gemv_bits<6>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 7: e = gemv_bits<7>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    case 8: e = gemv_bits<8>(trellis, suh, x, x_dtype, yf, m, n_out, n_in, cb, s); break;
    default: return hipErrorInvalidValue;
  }
  if (e != hipSuccess) return e;
  const int64_t groups = m * n_out / 128;
  constexpr int kPerBlock = kHadThreads / kWave;
  hipLaunchKernelGGL(hadamard128_kernel, dim3((unsigned)((groups + kPerBlock - 1) / kPerBlock)), dim3(kHadThreads), 0,
                     s, yf, (const uint16_t*)nullptr, svh, bias, bias_dtype, n_out, groups);
  return hipGetLastError();
}

hipError_t launch_hadamard128(float* v, const uint16_t* pre, const uint16_t* post, int64_t n,
                              hipStream_t s) {
  if (n == 0) return hipSuccess;
  constexpr int kPerBlock = kHadThreads / kWave;
  const int64_t groups = n / 128;
  hipLaunchKernelGGL(hadamard128_kernel, dim3((unsigned)((groups + kPerBlock - 1) / kPerBlock)), dim3(kHadThreads), 0,
                     s, v, pre, post, (const void*)nullptr, 0, n, groups);
  return hipGetLastError();
}

}  // namespace ttq
