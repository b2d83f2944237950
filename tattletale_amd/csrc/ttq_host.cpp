// Host-side (CPU) weight preparation for libttq_hip.so: a counter-based normal generator,
// quantizers that produce valid packed buffers for each format, and 16-bit float
// conversions.  None of this is on the hot path: it runs once when a layer is built, in
// the place where the reference assembles the dense weight it hands to Linear.init
// (workspace/transformers/src/layers/linear.nim:29-43, mlp.nim:39-41).
//
// Only the *decoders* of the formats are contracts; the quantizers here are simple
// deterministic fits (no iterative search), good enough to give realistic packed data.
#include "../../include/ttq.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

// ------------------------------------------------------------------ parallel helper
template <class Fn>
void parallel_for(int64_t n, int64_t grain, Fn fn) {
  unsigned hw = std::thread::hardware_concurrency();
  if (hw == 0) hw = 1;
  if (hw > 32) hw = 32;
  int64_t nt = std::min<int64_t>(hw, (n + grain - 1) / grain);
  if (nt <= 1) { fn(0, n); return; }
  std::vector<std::thread> th;
  const int64_t chunk = (n + nt - 1) / nt;
  for (int64_t t = 0; t < nt; t++) {
    const int64_t lo = t * chunk, hi = std::min(n, lo + chunk);
    if (lo >= hi) break;
    th.emplace_back([=] { fn(lo, hi); });
  }
  for (auto& t : th) t.join();
}

// ------------------------------------------------------------------ 16-bit floats
inline uint32_t f2u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float u2f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline float half_to_float(uint16_t h) {
  // shift the 15 magnitude bits into place, then fix the exponent bias by a multiply
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t mag = (uint32_t)(h & 0x7FFFu) << 13;
  float f;
  if ((h & 0x7C00u) == 0x7C00u) f = u2f(mag | 0x7F800000u);        // inf / nan
  else f = u2f(mag) * u2f(0x77800000u);                            // * 2^112 (handles subnormals)
  return u2f(f2u(f) | sign);
}

inline uint16_t float_to_half(float f) {
  // round-to-nearest-even through a float addition that aligns the rounding position
  const uint32_t x = f2u(f);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t ax = x & 0x7FFFFFFFu;
  if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x1FFu));
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
  if (ax < 0x38800000u) {  // below the smallest normal half: result is subnormal or zero
    const float a = u2f(ax) + 0.5f;  // 0.5f has ulp 2^-24 in [0.5,1): the add rounds to half subnormal grid
    return (uint16_t)(sign | (f2u(a) - 0x3F000000u));
  }
  uint32_t r = ax - 0x38000000u;            // rebias exponent
  const uint32_t odd = (r >> 13) & 1u;
  r += 0xFFFu + odd;
  return (uint16_t)(sign | (r >> 13));
}

inline uint16_t float_to_bf16(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7FFFu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

// ------------------------------------------------------------------ RNG
inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
inline uint64_t rng_key(uint64_t seed, uint64_t stream) { return mix64(seed ^ mix64(stream + 0x632BE59BD9B4E019ull)); }
inline uint64_t rng_at(uint64_t key, uint64_t i) { return mix64(key + (i + 1) * 0x9E3779B97F4A7C15ull); }

// ------------------------------------------------------------------ codebook (EXL3)
inline float codebook_value(uint32_t state, int cb) {
  uint32_t u = (cb == TTQ_CB_3INST) ? (state * 89226354u + 64248484u) : (state * 0xCBAC1FEDu);
  u = (u & 0x8FFF8FFFu) ^ 0x3B603B60u;
  const float s = half_to_float((uint16_t)(u & 0xFFFFu)) + half_to_float((uint16_t)(u >> 16));
  return half_to_float(float_to_half(s));
}

void fwht128(float* p, int64_t stride) {
  for (int len = 1; len < 128; len <<= 1)
    for (int i = 0; i < 128; i += 2 * len)
      for (int j = i; j < i + len; j++) {
        const float a = p[j * stride], b = p[(j + len) * stride];
        p[j * stride] = a + b;
        p[(j + len) * stride] = a - b;
      }
  const float s = 0.08838834764831845f;
  for (int i = 0; i < 128; i++) p[i * stride] *= s;
}

int check_block_args(const void* a, const void* b, int64_t n_out, int64_t n_in, int64_t mult) {
  if (!a || !b) return TTQ_ERR_NULL;
  if (n_out < 0 || n_in <= 0 || n_in % mult != 0) return TTQ_ERR_SHAPE;
  return TTQ_OK;
}

}  // namespace

extern "C" {

int ttq_host_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
  if (!in || !out) return TTQ_ERR_NULL;
  for (int64_t i = 0; i < n; i++) out[i] = float_to_bf16(in[i]);
  return TTQ_OK;
}
int ttq_host_f32_to_f16(const float* in, uint16_t* out, int64_t n) {
  if (!in || !out) return TTQ_ERR_NULL;
  for (int64_t i = 0; i < n; i++) out[i] = float_to_half(in[i]);
  return TTQ_OK;
}
int ttq_host_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
  if (!in || !out) return TTQ_ERR_NULL;
  for (int64_t i = 0; i < n; i++) out[i] = u2f((uint32_t)in[i] << 16);
  return TTQ_OK;
}
int ttq_host_f16_to_f32(const uint16_t* in, float* out, int64_t n) {
  if (!in || !out) return TTQ_ERR_NULL;
  for (int64_t i = 0; i < n; i++) out[i] = half_to_float(in[i]);
  return TTQ_OK;
}

int ttq_host_fill_normal(uint64_t seed, uint64_t stream, float sigma, float* out, int64_t n) {
  if (!out) return TTQ_ERR_NULL;
  if (n < 0) return TTQ_ERR_SHAPE;
  const uint64_t key = rng_key(seed, stream);
  parallel_for(n, 1 << 16, [=](int64_t lo, int64_t hi) {
    for (int64_t i = lo; i < hi; i++) {
      const uint64_t r = rng_at(key, (uint64_t)i);
      const double u1 = ((double)(uint32_t)(r >> 32) + 0.5) * (1.0 / 4294967296.0);
      const double u2 = ((double)(uint32_t)r + 0.5) * (1.0 / 4294967296.0);
      const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
      out[i] = (float)((double)sigma * z);
    }
  });
  return TTQ_OK;
}

// Q8_0: d = max|w| / 127 per block of 32, q = round(w / d).
int ttq_host_quantize_q8_0(const float* w, void* out, int64_t n_out, int64_t n_in) {
  const int rc = check_block_args(w, out, n_out, n_in, 32);
  if (rc) return rc;
  const int64_t nb = n_out * (n_in / 32);
  uint8_t* o = static_cast<uint8_t*>(out);
  parallel_for(nb, 4096, [=](int64_t lo, int64_t hi) {
    for (int64_t b = lo; b < hi; b++) {
      const float* x = w + 32 * b;
      float amax = 0.f;
      for (int i = 0; i < 32; i++) amax = std::max(amax, std::fabs(x[i]));
      const float d = amax / 127.f;
      const float id = d != 0.f ? 1.f / d : 0.f;
      uint8_t* p = o + 34 * b;
      const uint16_t dh = float_to_half(d);
      std::memcpy(p, &dh, 2);
      for (int i = 0; i < 32; i++) {
        int q = (int)std::lround(x[i] * id);
        q = std::max(-127, std::min(127, q));
        p[2 + i] = (uint8_t)(int8_t)q;
      }
    }
  });
  return TTQ_OK;
}

// Q4_K: per sub-block affine fit w ~ scale*q - min with q in 0..15, min >= 0; 6-bit
// sub-block scale/min against fp16 super-block d / dmin; nibbles re-fit against the stored
// (rounded) scales.
int ttq_host_quantize_q4_k(const float* w, void* out, int64_t n_out, int64_t n_in) {
  const int rc = check_block_args(w, out, n_out, n_in, 256);
  if (rc) return rc;
  const int64_t nb = n_out * (n_in / 256);
  uint8_t* o = static_cast<uint8_t*>(out);
  parallel_for(nb, 512, [=](int64_t lo, int64_t hi) {
    for (int64_t b = lo; b < hi; b++) {
      const float* x = w + 256 * b;
      float scale[8], mn[8];
      float max_scale = 0.f, max_min = 0.f;
      for (int j = 0; j < 8; j++) {
        float vmin = x[32 * j], vmax = x[32 * j];
        for (int i = 1; i < 32; i++) { vmin = std::min(vmin, x[32 * j + i]); vmax = std::max(vmax, x[32 * j + i]); }
        mn[j] = std::max(0.f, -vmin);
        scale[j] = std::max(0.f, (vmax + mn[j]) / 15.f);
        max_scale = std::max(max_scale, scale[j]);
        max_min = std::max(max_min, mn[j]);
      }
      const uint16_t dh = float_to_half(max_scale / 63.f), mh = float_to_half(max_min / 63.f);
      const float d = half_to_float(dh), dmin = half_to_float(mh);
      uint8_t sc[8], mm[8];
      for (int j = 0; j < 8; j++) {
        int s = d > 0.f ? (int)std::lround(scale[j] / d) : 0;
        int m = dmin > 0.f ? (int)std::lround(mn[j] / dmin) : 0;
        sc[j] = (uint8_t)std::max(0, std::min(63, s));
        mm[j] = (uint8_t)std::max(0, std::min(63, m));
      }
      uint8_t* p = o + 144 * b;
      std::memcpy(p, &dh, 2);
      std::memcpy(p + 2, &mh, 2);
      uint8_t* s12 = p + 4;
      for (int j = 0; j < 4; j++) {
        s12[j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
        s12[j + 4] = (uint8_t)((mm[j] & 63) | ((mm[j + 4] >> 4) << 6));
        s12[j + 8] = (uint8_t)((sc[j + 4] & 0xF) | ((mm[j + 4] & 0xF) << 4));
      }
      uint8_t* qs = p + 16;
      for (int c = 0; c < 4; c++) {
        for (int l = 0; l < 32; l++) {
          uint8_t nib[2];
          for (int h = 0; h < 2; h++) {
            const int j = 2 * c + h;
            const float dj = d * (float)sc[j], mj = dmin * (float)mm[j];
            int q = dj > 0.f ? (int)std::lround((x[64 * c + 32 * h + l] + mj) / dj) : 0;
            nib[h] = (uint8_t)std::max(0, std::min(15, q));
          }
          qs[32 * c + l] = (uint8_t)(nib[0] | (nib[1] << 4));
        }
      }
    }
  });
  return TTQ_OK;
}

// Q6_K: per 16-weight sub-block the extreme element maps to -32; int8 sub-block scales
// against an fp16 super-block d; 6-bit quants re-fit against the stored scales.
int ttq_host_quantize_q6_k(const float* w, void* out, int64_t n_out, int64_t n_in) {
  const int rc = check_block_args(w, out, n_out, n_in, 256);
  if (rc) return rc;
  const int64_t nb = n_out * (n_in / 256);
  uint8_t* o = static_cast<uint8_t*>(out);
  parallel_for(nb, 512, [=](int64_t lo, int64_t hi) {
    for (int64_t b = lo; b < hi; b++) {
      const float* x = w + 256 * b;
      float scale[16];
      float amax_scale = 0.f;
      for (int j = 0; j < 16; j++) {
        float ext = 0.f;
        for (int i = 0; i < 16; i++) if (std::fabs(x[16 * j + i]) > std::fabs(ext)) ext = x[16 * j + i];
        scale[j] = -ext / 32.f;
        amax_scale = std::max(amax_scale, std::fabs(scale[j]));
      }
      const uint16_t dh = float_to_half(amax_scale / 127.f);
      const float d = half_to_float(dh);
      int8_t sc[16];
      uint8_t q[256];
      for (int j = 0; j < 16; j++) {
        int s = d > 0.f ? (int)std::lround(scale[j] / d) : 0;
        sc[j] = (int8_t)std::max(-128, std::min(127, s));
        const float ds = d * (float)sc[j];
        for (int i = 0; i < 16; i++) {
          int v = ds != 0.f ? (int)std::lround(x[16 * j + i] / ds) : 0;
          q[16 * j + i] = (uint8_t)(std::max(-32, std::min(31, v)) + 32);
        }
      }
      uint8_t* p = o + 210 * b;
      uint8_t* ql = p;
      uint8_t* qh = p + 128;
      for (int h = 0; h < 2; h++) {
        for (int l = 0; l < 32; l++) {
          const uint8_t q1 = q[128 * h + l], q2 = q[128 * h + l + 32];
          const uint8_t q3 = q[128 * h + l + 64], q4 = q[128 * h + l + 96];
          ql[64 * h + l] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
          ql[64 * h + l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
          qh[32 * h + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
      }
      std::memcpy(p + 192, sc, 16);
      std::memcpy(p + 208, &dh, 2);
    }
  });
  return TTQ_OK;
}

// EXL3-style: normalise rows, flip signs, rotate both sides with 128-wide Hadamard
// transforms, then encode each 16x16 tile as a cyclic bit string whose 16-bit windows index
// the codebook.  The search is greedy with a tail-biting wrap: the last few weights of a
// tile see windows that wrap onto the already chosen first bits.
int ttq_host_quantize_exl3(const float* w, uint16_t* trellis, uint16_t* suh_f16, uint16_t* svh_f16,
                           int64_t n_out, int64_t n_in, int bits, int codebook, uint64_t seed) {
  if (!w || !trellis || !suh_f16 || !svh_f16) return TTQ_ERR_NULL;
  if (bits < 1 || bits > 8 || (codebook != TTQ_CB_3INST && codebook != TTQ_CB_MCG)) return TTQ_ERR_FORMAT;
  if (n_out <= 0 || n_in <= 0 || n_out % 128 || n_in % 128) return TTQ_ERR_SHAPE;

  std::vector<float> cbv(65536);
  double m1 = 0, m2 = 0;
  for (uint32_t s = 0; s < 65536; s++) { cbv[s] = codebook_value(s, codebook); m1 += cbv[s]; m2 += (double)cbv[s] * cbv[s]; }
  m1 /= 65536.0;
  const float cb_std = (float)std::sqrt(m2 / 65536.0 - m1 * m1);

  const uint64_t key_in = rng_key(seed, 0x1001), key_out = rng_key(seed, 0x1002);
  std::vector<float> sin_(n_in), sout(n_out), rscale(n_out);
  for (int64_t k = 0; k < n_in; k++) sin_[k] = (rng_at(key_in, k) >> 63) ? -1.f : 1.f;
  for (int64_t n = 0; n < n_out; n++) sout[n] = (rng_at(key_out, n) >> 63) ? -1.f : 1.f;

  std::vector<float> r((size_t)n_out * n_in);
  float* R = r.data();
  // normalise + sign + rotate along n_in
  parallel_for(n_out, 16, [&](int64_t lo, int64_t hi) {
    for (int64_t n = lo; n < hi; n++) {
      double ss = 0;
      for (int64_t k = 0; k < n_in; k++) ss += (double)w[n * n_in + k] * w[n * n_in + k];
      float rms = (float)std::sqrt(ss / (double)n_in);
      if (!(rms > 0.f)) rms = 1.f;
      // the stored scale is fp16; normalise with the value the decoder will really use
      const uint16_t sh = float_to_half(sout[n] * rms / cb_std);
      svh_f16[n] = sh;
      const float sv = half_to_float(sh) * cb_std;  // = sign * rms as stored
      rscale[n] = sv;
      float* row = R + n * n_in;
      for (int64_t k = 0; k < n_in; k++) row[k] = w[n * n_in + k] * sin_[k] / sv;
      for (int64_t g = 0; g < n_in; g += 128) fwht128(row + g, 1);
    }
  });
  for (int64_t k = 0; k < n_in; k++) suh_f16[k] = float_to_half(sin_[k]);
  // rotate along n_out
  parallel_for(n_in, 64, [&](int64_t lo, int64_t hi) {
    for (int64_t k = lo; k < hi; k++)
      for (int64_t g = 0; g < n_out; g += 128) fwht128(R + g * n_in + k, n_in);
  });

  const int64_t kt_n = n_in / 16, nt_n = n_out / 16;
  const int words = 16 * bits, total = 256 * bits;
  const float* cb = cbv.data();
  parallel_for(kt_n * nt_n, 64, [&](int64_t lo, int64_t hi) {
    std::vector<uint8_t> bitbuf(total);
    for (int64_t t = lo; t < hi; t++) {
      const int64_t kt = t / nt_n, nt = t % nt_n;
      float v[256];
      for (int i = 0; i < 256; i++)
        v[i] = R[(nt * 16 + (i >> 4)) * n_in + kt * 16 + (i & 15)] * cb_std;
      // first window: best of 1024 scattered candidates for weight 0
      uint32_t best_s = 0;
      float best_e = 1e30f;
      for (uint32_t c = 0; c < 1024; c++) {
        const uint32_t s = (c * 40503u + 12345u) & 0xFFFFu;
        const float e = std::fabs(cb[s] - v[0]);
        if (e < best_e) { best_e = e; best_s = s; }
      }
      for (int j = 0; j < 16; j++) bitbuf[j] = (best_s >> (15 - j)) & 1;
      uint32_t state = best_s;
      for (int i = 1; i < 256; i++) {
        const int p0 = 16 + (i - 1) * bits;           // first new bit of this step
        int nfree = std::min(bits, std::max(0, total - p0));
        uint32_t forced = 0;                          // wrapped bits come from the start
        for (int j = nfree; j < bits; j++) forced = (forced << 1) | bitbuf[(p0 + j) % total];
        const int nforced = bits - nfree;
        uint32_t pick = 0;
        float pe = 1e30f;
        for (uint32_t c = 0; c < (1u << nfree); c++) {
          const uint32_t nb = (c << nforced) | forced;
          const uint32_t s = ((state << bits) | nb) & 0xFFFFu;
          const float e = std::fabs(cb[s] - v[i]);
          if (e < pe) { pe = e; pick = c; }
        }
        for (int j = 0; j < nfree; j++) bitbuf[p0 + j] = (pick >> (nfree - 1 - j)) & 1;
        state = ((state << bits) | ((pick << nforced) | forced)) & 0xFFFFu;
      }
      uint16_t* tile = trellis + t * words;
      for (int wd = 0; wd < words; wd++) {
        uint32_t x = 0;
        for (int j = 0; j < 16; j++) x = (x << 1) | bitbuf[16 * wd + j];
        tile[wd] = (uint16_t)x;
      }
    }
  });
  return TTQ_OK;
}

}  // extern "C"
