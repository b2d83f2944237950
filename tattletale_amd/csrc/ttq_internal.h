// Internal launcher interface between the C-ABI layer (ttq_api.hip) and the kernel files.
// Every launcher assumes its arguments were validated by the caller and returns the
// hipError_t of the launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdlib.h>

#include <atomic>

namespace ttq {

// Which kernel family a dispatcher picks (values as ttq_route_id in ttq.h).  ttq_route runs the dispatch code of
// ttq_linear_forward itself with a probe bound to the calling thread: every dispatcher reports its choice through
// route_probe and, when a probe is bound, returns instead of launching.
enum : int {
  kRouteNone = 0,
  kRouteGemvQ4kStream = 1,
  kRouteGemvQ4kStream4 = 2,
  kRouteGemvQ4kSlice = 3,
  kRouteGemvQ4kBatch4 = 4,
  kRouteGemvQ4kBatch = 5,
  kRouteGemvQ4kMfma = 6,
  kRouteGemvQ6kStream = 7,
  kRouteGemvQ6kStream4 = 8,
  kRouteGemvQ8Stream = 9,
  kRouteGemvQ8Win = 10,
  kRouteGemvQ8Mfma = 11,
  kRouteGemvDot2 = 12,
  kRouteGemvDot2Multi = 13,
  kRouteGemvGeneric = 14,
  kRouteGemvLong = 15,
  kRouteGemmSkinnyF32ScaledF16 = 19,
  kRouteGemmPc = 20,
  kRouteGemmPcSplitK = 21,
  kRouteGemmSkinny = 22,
  kRouteGemmSkinnyChunked = 23,
  kRouteGemmQ4kTiles = 24,
  kRouteGemmPcBf16Copy = 25,
  kRouteGemmPcPacked = 26,
  kRouteGemmPcPackedSplitK = 27,
  kRouteGemmPcF16 = 28,
  kRouteGemmPcF32ScaledF16 = 29,
  kRouteExl3Gemv = 30,
  kRouteExl3GemvSliced = 31,
  kRouteExl3Gemm = 32,
  kRouteExl3GemvTwoLaunches = 33,
};
struct RouteProbe { int route; };
extern thread_local RouteProbe* t_route_probe;
inline bool route_probe(int id) {
  RouteProbe* p = t_route_probe;
  if (!p) return false;
  if (p->route == 0) p->route = id;
  return true;
}
#define TTQ_ROUTE(id, call)                      \
  do {                                           \
    if (::ttq::route_probe(id)) return hipSuccess; \
    return call;                                 \
  } while (0)

// Developer A/B switches.  They are read from the environment only in builds made with
// -DTTQ_DEV_KNOBS; the product build (tattletale_amd/build.py) leaves that off, so what the library
// does never depends on the process environment.
inline int dev_knob(const char* name, int dflt) {
#ifdef TTQ_DEV_KNOBS
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
#else
  (void)name;
  return dflt;
#endif
}

// dtype codes as in ttq.h (TTQ_F32 = 0, TTQ_F16 = 1, TTQ_BF16 = 2)
enum : int { kF32 = 0, kF16 = 1, kBF16 = 2 };
// format codes as in ttq.h
enum : int { kQ8_0 = 0, kQ4_K = 1, kQ6_K = 2, kEXL3 = 3 };

constexpr int64_t kMaxGemvInF32 = 16384;    // activations staged in 64 KiB of LDS
constexpr int64_t kMaxGemvIn16 = 65536;   // 16-bit activations as staged pairs: 128 KiB of the 160 KiB of LDS
// rows beyond what the staged decode kernels take (they go to the unstaged kernel of ttq_gemv.hip)
bool gemv_row_is_long(int format, int x_dtype, int64_t n_in);

hipError_t launch_dequant(int format, const void* w, void* out, int out_dtype, int64_t n_out,
                          int64_t n_in, hipStream_t s);

// y (m, n_out) in y_dtype = x (m, n_in) in x_dtype times W^T, optional bias (n_out).
hipError_t launch_gemv(int format, const void* w, const void* x, int x_dtype, void* y,
                       int y_dtype, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                       int64_t n_in, hipStream_t s);

// Packed-dot fast path for 16-bit activations (ttq_gemv_dot2.hip).
// Packed-dot GEMV for two or four activation rows per pass over the weights (Q4_K shapes the
// matrix-core few-row kernels do not take, Q6_K).
bool gemv_dot2_multi_supported(int format, int x_dtype, int64_t m, int64_t n_in);
hipError_t launch_gemv_dot2_multi(int format, const void* w, const void* x, int x_dtype, void* y,
                                  int y_dtype, const void* bias, int bias_dtype, int64_t m,
                                  int64_t n_out, int64_t n_in, hipStream_t s);
bool gemv_dot2_supported(int format, int x_dtype, int64_t n_in);
hipError_t launch_gemv_dot2(int format, const void* w, const void* x, int x_dtype, void* y,
                            int y_dtype, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                            int64_t n_in, hipStream_t s);

// int8 matrix-core path for Q4_K and 16-bit activations (ttq_gemv_mfma.hip).
bool gemv_mfma_supported(int format, int x_dtype, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_mfma(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                            const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                            hipStream_t s);

// The same arithmetic with the weights streamed through LDS as whole cache lines (ttq_gemv_q4k_stream.hip):
// 16-bit activations, n_in 2048 or 4096.
bool gemv_q4k_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q4k_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                  const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                  hipStream_t s);

// The streamed kernel for long rows (ttq_gemv_q4k_slice.hip): n_in 6144 .. 14336 in steps of 2048, the K
// dimension dealt to the wavefronts, each with its own activation tables.
bool gemv_q4k_slice_supported(int format, int x_dtype, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q4k_slice(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                 const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                 hipStream_t s);

// The streamed kernel for two to four activation rows (ttq_gemv_q4k_stream4.hip): the tokens share the matrix
// instructions of a super-block; n_in 2048 or 4096, at least 16 rows per compute unit.
bool gemv_q4k_stream4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q4k_stream4(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                   const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                   hipStream_t s);
// gate || up + silu_and_mul on the same kernel: n_ff outputs from 2 n_ff weight rows
bool gemv_q4k_stream4_fused_supported(int x_dtype, int64_t m, int64_t n_ff, int64_t n_in);
hipError_t launch_gemv_q4k_stream4_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                         int64_t n_ff, int64_t n_in, hipStream_t s);

// Q8_0 through the int8 matrix cores with the raw bytes of the rows as the K dimension, streamed through three LDS
// buffers (ttq_gemv_q8_stream.hip): n_in a multiple of 2048 up to 8192 (4096 for fp32 activations), whole groups of
// 16 rows, at least one per compute unit.
bool gemv_q8_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q8_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                 const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                 hipStream_t s);

// Q6_K through the int8 matrix cores, 16 rows at a time streamed linearly through two or three LDS buffers
// (ttq_gemv_q6k_stream.hip): 16-bit activations, n_in a multiple of 2048 up to 14336 (or another multiple of 256:
// two, four or eight consecutive rows streamed as one), whole groups of 16 rows, at least one per compute unit.
bool gemv_q6k_stream_supported(int format, int x_dtype, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q6k_stream(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                  const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                  hipStream_t s);

// The same stream for two or more activation rows, two or four to a pass (ttq_gemv_q6k_stream4.hip).
bool gemv_q6k_stream4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q6k_stream4(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                   const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                   hipStream_t s);

// int8 matrix-core path for Q8_0, any activation dtype (ttq_gemv_q8_mfma.hip).
// Q8_0 through the matrix cores, rows read as aligned 64-byte windows (ttq_gemv_q8_win.hip).
bool gemv_q8_win_supported(int format, int64_t n_out, int64_t n_in);
int gemv_q8_win_tokens(int x_dtype, int64_t m, int64_t n_in);
hipError_t launch_gemv_q8_win(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                              int64_t n_in, hipStream_t s);
bool gemv_q8_mfma_supported(int format, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q8_mfma(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                               const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                               hipStream_t s);

// Fused decode kernels for Q4_K (ttq_gemv_mfma.hip): optional RMSNorm of the activation row in
// front (norm_gamma != null; residual / outputs optional) and optional gate/up + silu_and_mul
// behind (w then holds 2*n_out rows, gate rows first).
bool gemv_fused_supported(int format, int x_dtype, int64_t n_out, int64_t n_in, bool silu_mul);
// gate || up + silu_and_mul on the LDS-streamed kernel (ttq_gemv_q4k_stream.hip): Q4_K, 16-bit activations
bool gemv_q4k_stream_fused_supported(int x_dtype, int64_t n_ff, int64_t n_in);
hipError_t launch_gemv_q4k_stream_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                        int64_t n_ff, int64_t n_in, hipStream_t s);
// add + RMSNorm in front of either form (the shapes the two predicates above accept)
hipError_t launch_gemv_q4k_stream_norm(const void* w, const void* x, int x_dtype, void* y, int y_dtype, int64_t m,
                                       int64_t n_out, int64_t n_in, bool silu_mul, const void* norm_residual,
                                       const void* norm_gamma, float norm_eps, void* new_residual_out,
                                       void* normed_out, hipStream_t s);
hipError_t launch_gemv_fused(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                             const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                             bool silu_mul, const void* norm_residual, const void* norm_gamma,
                             float norm_eps, void* new_residual_out, void* normed_out, hipStream_t s);
// RMSNorm alone (ttq_activations.hip): t = x (+ residual), normed = t * rsqrt(mean(t^2) + eps) * gamma.
hipError_t launch_rmsnorm(const void* x, const void* residual, const void* gamma, float eps, int dtype,
                          void* new_residual_out, void* normed_out, int64_t m, int64_t n, hipStream_t s);
// out (m, h) = silu(in[:, :h]) * in[:, h:], in (m, 2h), same dtype (ttq_activations.hip).
hipError_t launch_silu_and_mul(const void* in, void* out, int dtype, int64_t m, int64_t h, hipStream_t s);

// Q4_K decode GEMV for a few activation rows at once (ttq_gemv_q4k_batch.hip): the weights are
// read and unpacked once per 8 or 16 rows.
bool gemv_q4k_batch_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q4k_batch(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                 const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                                 int64_t n_in, hipStream_t s);

// The same with four rows per pass, for rows up to the GEMV limit (ttq_gemv_q4k_batch4.hip).
bool gemv_q4k_batch4_supported(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_q4k_batch4(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                                  const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                                  int64_t n_in, hipStream_t s);

// Rough times (microseconds) of the two ways to run a few activation rows.
float gemv_estimate_us(int format, int x_dtype, int64_t m, int64_t n_out, int64_t n_in);
float gemm_pc_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in);
int gemv_q4k_batch_tokens(int64_t m, int64_t n_in);

// Compute units of the current device (256 when the query fails); cached per device ordinal.
int device_num_cus();

// Kernels that use more than 64 KiB of dynamic LDS must be allowed to, once per device.  One
// LargeLds per kernel instantiation (a function-local static) remembers on which device ordinals
// that has been done.
struct LargeLds { std::atomic<uint64_t> done{0}; };
hipError_t allow_large_lds(const void* kernel, LargeLds& state);

// Q4_K / Q6_K / Q8_0 linear layer for up to 64 rows of 16-bit activations, weights dequantized in
// registers (ttq_gemm_skinny.hip).
bool gemm_skinny_supported(int format, int64_t m, int64_t n_out, int64_t n_in);
float gemm_skinny_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in);
// x: bf16 or fp16 activations (the weights are rounded once to the same type); y: bf16, fp16 or fp32.
// row_scale (fp16 activations only): a factor per row on the sums, before the bias.
hipError_t launch_gemm_skinny(int format, const void* w, const uint16_t* x, int x_dtype, void* y, int y_dtype,
                              const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                              hipStream_t s, const float* row_scale = nullptr);
// Any number of rows, 64 per launch.
hipError_t launch_gemm_skinny_chunked(int format, const void* w, const uint16_t* x, int x_dtype, void* y, int y_dtype,
                                      const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                                      hipStream_t s, const float* row_scale = nullptr);
// fp32 activations: a copy scaled row by row to fp16 range (a power of two per row, undone on the sums) in the
// stream's workspace, then the fp16 kernel, 64 rows per launch.
hipError_t launch_gemm_skinny_f32(int format, const void* w, const float* x, void* y, int y_dtype, const void* bias,
                                  int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s);

// The same kernel with the fused gate||up weight (2 * n_ff rows, gate rows first) and silu_and_mul
// in its epilogue: y is (m, n_ff).  Q4_K.
bool gemm_skinny_silu_mul_supported(int64_t m, int64_t n_ff, int64_t n_in);
float gemm_skinny_silu_mul_estimate_us(int64_t m, int64_t n_ff, int64_t n_in);
hipError_t launch_gemm_skinny_silu_mul(const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                                       int bias_dtype, int64_t m, int64_t n_ff, int64_t n_in, hipStream_t s);

// The multi-row operator for block formats and bf16 activations: the few-row kernel or the tiled
// GEMM, whichever is estimated to be faster for the shape (ttq_gemm_q4k.hip).
bool gemm_supported(int format, int64_t m, int64_t n_out, int64_t n_in);
float gemm_estimate_us(int format, int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemm(int format, const void* w, const uint16_t* x_bf16, void* y, int y_dtype, const void* bias,
                       int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s);

// Producer/consumer GEMM for Q4_K / Q6_K / Q8_0 weights and bf16 activations (ttq_gemm_pc.hip).
bool gemm_pc_supported(int format, int64_t m, int64_t n_out, int64_t n_in, int bn);
hipError_t launch_gemm_pc(int format, const void* w, const uint16_t* x_bf16, void* y, int y_dtype,
                          const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in,
                          hipStream_t s);

// The same GEMM with silu_and_mul in the epilogue: Q4_K weight of 2*n_ff rows (gate rows first).
hipError_t launch_gemm_pc_silu_mul(const void* w, const uint16_t* x_bf16, void* y, int y_dtype,
                                   const void* bias, int bias_dtype, int64_t m, int64_t n_ff,
                                   int64_t n_in, hipStream_t s);

hipError_t launch_dequant_exl3(const uint16_t* trellis, uint16_t* out_f16, int64_t n_out,
                               int64_t n_in, int bits, int cb, hipStream_t s);
hipError_t launch_gemv_exl3(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                            const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                            int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int bits,
                            int cb, hipStream_t s);
hipError_t launch_hadamard128(float* v, const uint16_t* pre, const uint16_t* post, int64_t n,
                              hipStream_t s);

// Workspaces the library keeps per (slot, device, stream), grown on demand (ttq_workspace.hip).
constexpr int kWsExl3Rotated = 0, kWsGemmPartials = 2, kWsGemmCounters = 3, kWsPackedActivations = 4;
// zeroed: a newly allocated buffer is cleared (on the stream) before it is handed out
hipError_t stream_workspace(int slot, hipStream_t s, size_t bytes, void** out, bool zeroed = false);
// Frees every library-owned workspace (nothing that uses one may be in flight or captured).
hipError_t release_stream_workspaces();
hipError_t exl3_release_workspaces();
// A caller-owned workspace, bound to the calling thread while the object lives: stream_workspace and
// exl3_workspace then serve every request from it and allocate nothing.
constexpr int kCwCounters = 0, kCwExl3Words = 1, kCwScratch = 2;
class CallerWsScope {
 public:
  CallerWsScope(void* ws, size_t bytes);
  ~CallerWsScope();
  CallerWsScope(const CallerWsScope&) = delete;
  CallerWsScope& operator=(const CallerWsScope&) = delete;
  bool too_small() const;      // some request did not fit (the call then failed with hipErrorOutOfMemory)
 private:
  alignas(8) unsigned char state_[40];
};
// false: no caller workspace is bound.  true: *out / *err say where the region lies or that it does not fit.
bool caller_workspace_region(int region, size_t bytes, void** out, hipError_t* err);
// bytes in front of the scratch part of a caller-owned workspace (arrival counters, trellis hand-off words)
size_t caller_workspace_header_bytes();
int64_t exl3_workspace_words();
// the prefill GEMM for activations of any type (fp16 / fp32 are rounded to bf16 by its packing pass), and the bytes
// of packed copy such a launch takes from the workspace
hipError_t launch_gemm_pc_x(int format, const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                            const void* bias, int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, hipStream_t s, bool f16_native = false);
size_t gemm_pc_packed_bytes(int64_t m, int64_t n_out, int64_t n_in, int x_dtype);
// exact size of the partial sums a split-K launch of the prefill GEMM takes for this shape (0: not split)
size_t gemm_pc_partials_bytes(int64_t m, int64_t n_out, int64_t n_in);
// how often the trellis GEMV's last slice polls a missing word before it gives the row up; returns the old value
int exl3_set_poll_limit(int limit);
// n fp16 or fp32 values (n a multiple of 8) rounded to bf16

// Trellis layer for many activation rows (ttq_exl3_prefill.hip): activations rotated once into a workspace
// the library keeps per (device, stream), then 64 rows per decoded weight.  y fp32.
bool gemm_exl3_preferred(int64_t m, int64_t n_out, int64_t n_in);
// a prefill GEMM launch split along K: copies of the tile grid that meet in a workspace (ttq_gemm_pc.h)
struct PcSplit {
  int splits;          // 1: none
  int tile_wgs;        // workgroups of one copy of the tile grid
  float* partials;
  uint32_t* counters;
};
constexpr int kPcMaxCounters = 16384;     // (tile, consumer) pairs a split launch may have
// bytes of partial sums the many-row trellis GEMM keeps in the workspace for this call (0: not split along K)
size_t gemm_exl3_partials_bytes(int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemm_exl3_pc(int bits, int cb, int mb, const uint16_t* trellis, const uint16_t* svh, const uint16_t* xp,
                               void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m, int64_t n_out,
                               int64_t n_in, PcSplit sp, hipStream_t s);
hipError_t launch_gemm_exl3(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, const void* x,
                            int x_dtype, void* y, int y_dtype, const void* bias, int bias_dtype, int64_t m,
                            int64_t n_out, int64_t n_in, int bits, int cb, hipStream_t s);

// Matrix-core trellis GEMV in one launch (ttq_exl3_mfma.hip).  The plan says how the reduction
// dimension is sliced and how many 64-bit accumulator words a sliced launch needs (zero before and
// after every launch).
struct Exl3Plan {
  int groups, row_groups, slices, slice_tiles;
  int64_t accum_words;
};
Exl3Plan exl3_mfma_plan(int64_t m, int64_t n_out, int64_t n_in);
hipError_t launch_gemv_exl3_mfma(const Exl3Plan& p, const uint16_t* trellis, const uint16_t* suh,
                                 const uint16_t* svh, const void* x, int x_dtype, void* y, int y_dtype, const void* bias,
                                 int bias_dtype, int64_t m, int64_t n_out, int64_t n_in, int bits, int cb,
                                 unsigned long long* accum, hipStream_t s);
// The library's own accumulator words for the calling thread's device and this stream, allocated and
// cleared on first use.
hipError_t exl3_workspace(hipStream_t s, unsigned long long** accum);
// The workspace that lives in the library's own device image (one per GPU, nothing allocated), and its size.
hipError_t exl3_resident_workspace(unsigned long long** accum);
int64_t exl3_resident_words();

}  // namespace ttq
