// Prefill GEMM for Q4_K, Q6_K and Q8_0 weights on gfx950, producer/consumer form (kernel: ttq_gemm_pc.h):
// tile choice, split along K and its workspace, and the launchers behind ttq_gemm_* / ttq_linear_forward.
#include "ttq_gemm_pc.h"

namespace ttq {

// x: the activations, or (tile_if_packed >= 0) their packed copy and the tile's index for launch_gemm_packed
template <int FMT, int MB, int NJ, bool FUSE>
static hipError_t launch_pc_tile(const uint8_t* wb, const uint16_t* x, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int splits, int tile_if_packed,
                                 hipStream_t s, bool x_f16 = false, const float* row_scale = nullptr) {
  PcSplit sp{1, 0, nullptr, nullptr};
  if (!FUSE && splits > 1) {
    // (the chooser has checked that the blocks of a row divide evenly and that the counters suffice)
    constexpr int BO = NJ * 16, BM = pc_bm(MB);
    const size_t units = (size_t)((n_out + BO - 1) / BO) * (size_t)((m + BM - 1) / BM) * 4;
    void* part = nullptr;
    void* cnt = nullptr;
    hipError_t e = stream_workspace(kWsGemmPartials, s, units * splits * (size_t)(MB * NJ * 1024), &part);
    if (e == hipSuccess) e = stream_workspace(kWsGemmCounters, s, (size_t)kPcMaxCounters * 4, &cnt, true);
    if (e != hipSuccess) return e;
    sp.splits = splits;
    sp.partials = static_cast<float*>(part);
    sp.counters = static_cast<uint32_t*>(cnt);
  }
  if (tile_if_packed >= 0)
    return launch_gemm_packed(FMT, FUSE, tile_if_packed, wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s, x_f16, row_scale);
  return launch_pc_grid<FMT, MB, NJ, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, sp, s);
}

// Tile choice.  A workgroup owns 64*MB rows x 16*NJ columns (8*NJ outputs when fused); the grid
// should fill the 256 CUs without a nearly empty last round.  Cost model: rounds of workgroups x
// (64-k steps x time per step of the tile shape + a fixed cost per workgroup), both measured
// (microseconds; 14336 x 4096 and x 8192 at 2048 rows).  Smaller tiles are cheaper per step --
// down to the latency of the producers' load / dequantize / store / barrier chain, about 0.45 us
// -- but dequantize every weight for fewer rows.
struct PcTile { int mb, nj; float step_us; };
static const PcTile kPcTiles[] = {{4, 7, 0.87f}, {4, 4, 0.68f}, {2, 7, 0.585f}, {2, 4, 0.55f}, {1, 7, 0.46f}, {1, 4, 0.52f}};
constexpr float kPcFixedUs = 6.f;

// A grid that leaves most compute units idle (few columns x few rows: the attention output and down projections
// at a few hundred rows) is also split along K, 2 / 4 / 7 / 8 ways while all copies still fit one round: the
// length of a short round is the latency of its K loop.  What the meeting of the copies costs (measured, 1024 /
// 4096 / 14336 columns x 4096 / 14336 inputs at 128 .. 1024 rows): a consumer stores its partial sums, counts,
// and the last one loads the copies one after the other -- 2 + copies trips to the memory side (3 for two
// copies), each the longer the more accumulators a lane holds -- and the partial sums cross the memory system
// twice at about 4 TB/s.
struct PcChoice { int tile, splits; float cost_us; };

static float pc_split_us(const PcTile& t, int splits, int64_t padded_rows, int64_t padded_cols) {
  const float trip = 0.9f + 0.06f * (float)(t.mb * t.nj);
  const float trips = splits == 2 ? 3.f : 2.f + (float)splits;
  return trips * trip + 2.f * (float)splits * (float)padded_rows * (float)padded_cols * 4.f / 4.0e6f;
}

static PcChoice pc_choose(int64_t m, int64_t n_out, int64_t n_in, bool fuse) {
  static const int forced = dev_knob("TTQ_GEMM_TILE", -1);
  static const int forced_splits = dev_knob("TTQ_GEMM_SPLITS", 0);   // A/B: 1 = never split, n = n ways where possible
  static const int kSplits[] = {1, 2, 4, 7, 8};
  const int cus = device_num_cus();
  const int64_t blocks = n_in / 256;
  PcChoice best{0, 1, 1e30f};
  for (int pass = 0; pass < 2 && best.cost_us > 1e29f; pass++) {
    for (int i = 0; i < (int)(sizeof(kPcTiles) / sizeof(kPcTiles[0])); i++) {
      if (forced >= 0 && forced < (int)(sizeof(kPcTiles) / sizeof(kPcTiles[0])) && i != forced) continue;
      const PcTile& t = kPcTiles[i];
      const int64_t bo = fuse ? t.nj * 8 : t.nj * 16, bm = pc_bm(t.mb);
      const int64_t nt = (n_out + bo - 1) / bo, mt = (m + bm - 1) / bm, tiles = nt * mt;
      for (int sp : kSplits) {
        if (pass == 0 && forced_splits > 0 && sp != forced_splits) continue;
        if (pass == 1 && sp != 1) continue;
        if (sp > 1 && (fuse || blocks % sp != 0 || blocks / sp < 2 || tiles * sp > cus || tiles * 4 > kPcMaxCounters)) continue;
        const int64_t rounds = (tiles * sp + cus - 1) / cus;
        const float cost = (float)rounds * ((float)(n_in / 64 / sp) * t.step_us + kPcFixedUs) +
                           (sp > 1 ? pc_split_us(t, sp, mt * bm, nt * bo) : 0.f);
        if (cost < best.cost_us * 0.999f) best = PcChoice{i, sp, cost};
      }
    }
  }
  return best;
}

size_t gemm_pc_partials_bytes(int64_t m, int64_t n_out, int64_t n_in) {
  if (m <= 0 || n_out <= 0 || n_in < 256) return 0;
  const PcChoice c = pc_choose(m, n_out, n_in, false);
  if (c.splits <= 1) return 0;
  const PcTile& t = kPcTiles[c.tile];
  const int64_t nt = (n_out + t.nj * 16 - 1) / (t.nj * 16), mt = (m + pc_bm(t.mb) - 1) / pc_bm(t.mb);
  return (size_t)(nt * mt * 4) * (size_t)c.splits * (size_t)(t.mb * t.nj * 1024);
}

// Rough time of the GEMM for this shape (microseconds), for callers that can also run the
// operator as a few GEMV passes.  The Q6_K and Q8_0 producers are slower than the Q4_K one.
float gemm_pc_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in) {
  const float c = pc_choose(m, n_out, n_in, false).cost_us;
  return c * (format == kQ8_0 ? 1.9f : (format == kQ6_K ? 1.4f : 1.f)) + 2.f;
}

// Launches of 256-row tiles read the activations from a copy in fragment order (ttq_gemm_pcd.h), made by one pass
// over X into a workspace: with no X traffic through LDS their K loop is 6 % (64-column tiles) to 15 % (112-column
// tiles) shorter, which pays for the pass (2.5 us + the bytes at about 7 TB/s, they come out of the caches) on every
// shape measured from 50 us of GEMM on: 4096 x 14336 at 512 rows 90.4 -> 84.6 us, at 1024 rows 150.7 -> 142.2 us,
// 5120 x 13824 at 512 rows 102.1 -> 94.2 us, 4096 x 4096 at 1024 rows 53.8 -> 51.6 us.  Tiles of 128 and 64 rows
// move a half and a quarter of the activation bytes per step through LDS and gain nothing from the copy (-0.5 to
// -6 us on seven shapes, split along K or not).
constexpr int64_t kPackRows = 8192;         // rows packed (and multiplied) at a time
static bool pc_use_packed(const PcChoice& c) {
  static const int knob = dev_knob("TTQ_GEMM_PACKED", -1);      // A/B: 0 never, 1 always
  if (knob >= 0) return knob != 0;
  return kPcTiles[c.tile].mb == 4 && c.cost_us >= 45.f;
}

template <int FMT, bool FUSE>
static hipError_t launch_pc_rows(const PcChoice& c, int tile_if_packed, const uint8_t* wb, const uint16_t* x, void* y,
                                 int y_dtype, const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                 hipStream_t s, bool x_f16 = false, const float* row_scale = nullptr) {
  const int p = tile_if_packed;
  switch (c.tile) {
    case 0: return launch_pc_tile<FMT, 4, 7, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
    case 1: return launch_pc_tile<FMT, 4, 4, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
    case 2: return launch_pc_tile<FMT, 2, 7, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
    case 3: return launch_pc_tile<FMT, 2, 4, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
    case 4: return launch_pc_tile<FMT, 1, 7, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
    default: return launch_pc_tile<FMT, 1, 4, FUSE>(wb, x, y, y_dtype, bias, bias_dtype, m, n_out, n_in, c.splits, p, s, x_f16, row_scale);
  }
}

// x in x_dtype: bf16 for the direct form; any type when the launch goes through the packed copy (the packing pass
// rounds to bf16, or -- keep_f16 -- leaves fp16 activations as they are for the fp16 form of the kernel).
template <int FMT, bool FUSE>
static hipError_t launch_pc_fmt(const uint8_t* wb, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, bool force_packed, hipStream_t s,
                                int f16_mode = 0) {      // 1: fp16 activations stay fp16; 2: fp32 activations as scaled fp16
  const PcChoice whole = pc_choose(m, n_out, n_in, FUSE);
  // (the fused gate||up form keeps the LDS-staged kernel: beside the packed kernel's three steps of A fragments its
  // epilogue does not fit the registers, and a kernel that requests registers asynchronously must never spill them)
  if (FUSE || (!force_packed && !pc_use_packed(whole)))
    return launch_pc_rows<FMT, FUSE>(whole, -1, wb, static_cast<const uint16_t*>(x), y, y_dtype, bias, bias_dtype, m, n_out,
                                     n_in, s);
  const int64_t block_rows = m < kPackRows ? m : kPackRows;
  void* ws = nullptr;
  // (fp32 activations as scaled fp16: the rows' inverse factors follow the packed copy)
  const size_t copy_bytes = (gemm_packed_activation_bytes(block_rows, n_in) + 255) & ~(size_t)255;
  hipError_t e = stream_workspace(kWsPackedActivations, s, copy_bytes + (f16_mode == 2 ? (size_t)block_rows * 4 : 0), &ws);
  if (e != hipSuccess) return e;
  float* row_scale = f16_mode == 2 ? reinterpret_cast<float*>(static_cast<char*>(ws) + copy_bytes) : nullptr;
  const int64_t xsize = x_dtype == kF32 ? 4 : 2, ysize = y_dtype == kF32 ? 4 : 2;
  for (int64_t r0 = 0; r0 < m; r0 += kPackRows) {
    const int64_t rows = m - r0 < kPackRows ? m - r0 : kPackRows;
    if (f16_mode == 2)
      e = launch_gemm_pack_activations_scaled(static_cast<const float*>(x) + r0 * n_in, static_cast<uint16_t*>(ws), row_scale,
                                              rows, n_in, s);
    else
      e = launch_gemm_pack_activations(static_cast<const char*>(x) + r0 * n_in * xsize, x_dtype, static_cast<uint16_t*>(ws),
                                       rows, n_in, s, f16_mode == 1);
    if (e != hipSuccess) return e;
    const PcChoice c = rows == m ? whole : pc_choose(rows, n_out, n_in, FUSE);
    e = launch_pc_rows<FMT, FUSE>(c, c.tile, wb, static_cast<const uint16_t*>(ws), static_cast<char*>(y) + r0 * n_out * ysize,
                                  y_dtype, bias, bias_dtype, rows, n_out, n_in, s, f16_mode != 0, row_scale);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// 112- and 64-column tiles are built in this form: with 128 columns the consumers' 128
// accumulator registers plus the fragment rings do not fit the 168 registers a wavefront gets
// when twelve of them share a CU.
bool gemm_pc_supported(int format, int64_t m, int64_t n_out, int64_t n_in, int bn) {
  static const int disabled = dev_knob("TTQ_GEMM_NO_PC", 0);
  // activation byte offsets are 32-bit in the kernel; a step loop iteration is 256 k
  return !disabled && (format == kQ4_K || format == kQ6_K || format == kQ8_0) && bn == 112 &&
         m * n_in * 2 < ((int64_t)1 << 32) && n_out > 0 && n_in > 0 && n_in % 256 == 0;
}

// x: bf16 activations; or (x_dtype fp16 / fp32) activations that may be rounded to bf16: those always go through the
// packed copy, whose packing pass does the rounding; or (f16_native) the fp16 form of the kernel, which rounds the
// weights to fp16 and multiplies on the fp16 matrix cores: fp16 activations stay as they are in the packed copy, fp32
// activations become fp16 there after every row has been scaled by a power of two (undone in the epilogue).
hipError_t launch_gemm_pc_x(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                            const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s,
                            bool f16_native) {
  if (m == 0 || n_out == 0) return hipSuccess;
  if (y_dtype != kBF16 && y_dtype != kF32 && y_dtype != kF16) return hipErrorInvalidValue;
  if (f16_native && x_dtype != kF16 && x_dtype != kF32) return hipErrorInvalidValue;
  const PcChoice c = pc_choose(m, n_out, n_in, false);
  const bool packed = x_dtype != kBF16 || pc_use_packed(c);
  if (route_probe(f16_native ? (x_dtype == kF32 ? kRouteGemmPcF32ScaledF16 : kRouteGemmPcF16)
                             : (x_dtype != kBF16 ? kRouteGemmPcBf16Copy
                                                 : (c.splits > 1 ? (packed ? kRouteGemmPcPackedSplitK : kRouteGemmPcSplitK)
                                                                 : (packed ? kRouteGemmPcPacked : kRouteGemmPc)))))
    return hipSuccess;
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  const bool force = x_dtype != kBF16;
  switch (format) {
    case kQ4_K: return launch_pc_fmt<kQ4_K, false>(wb, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, force, s, f16_native ? (x_dtype == kF32 ? 2 : 1) : 0);
    case kQ6_K: return launch_pc_fmt<kQ6_K, false>(wb, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, force, s, f16_native ? (x_dtype == kF32 ? 2 : 1) : 0);
    case kQ8_0: return launch_pc_fmt<kQ8_0, false>(wb, x, x_dtype, y, y_dtype, bias, bias_dtype, m, n_out, n_in, force, s, f16_native ? (x_dtype == kF32 ? 2 : 1) : 0);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemm_pc(int format, const void* w, const uint16_t* x_bf16, void* y, int y_dtype,
                          const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                          hipStream_t s) {
  return launch_gemm_pc_x(format, w, x_bf16, kBF16, y, y_dtype, bias, bias_dtype, m, n_out, n_in, s);
}

// bytes of the packed copy a launch of this shape takes from the workspace (0: it reads X itself)
size_t gemm_pc_packed_bytes(int64_t m, int64_t n_out, int64_t n_in, int x_dtype) {
  if (m <= 0 || n_out <= 0 || n_in < 256) return 0;
  const bool packed = x_dtype != kBF16 || pc_use_packed(pc_choose(m, n_out, n_in, false));
  if (!packed) return 0;
  const int64_t rows = m < kPackRows ? m : kPackRows;
  // (fp32 activations: room for a factor per row behind the copy, whichever way they are narrowed)
  return ((gemm_packed_activation_bytes(rows, n_in) + 255) & ~(size_t)255) + (x_dtype == kF32 ? (size_t)rows * 4 : 0);
}


// gate||up projection + silu_and_mul in the GEMM epilogue: w holds 2*n_ff rows (gate rows first),
// y is (m, n_ff).  Q4_K weights.
hipError_t launch_gemm_pc_silu_mul(const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                                   int bias_dtype, int64_t m, int64_t n_ff, int64_t n_in, hipStream_t s) {
  if (m == 0 || n_ff == 0) return hipSuccess;
  if (y_dtype != kBF16 && y_dtype != kF32) return hipErrorInvalidValue;
  return launch_pc_fmt<kQ4_K, true>(static_cast<const uint8_t*>(w), x_bf16, kBF16, y, y_dtype, bias, bias_dtype, m, n_ff,
                                    n_in, false, s);
}

}  // namespace ttq
