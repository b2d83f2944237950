/*
 * ttq.h -- C ABI of libttq_hip.so: quantized-weight linear layer for AMD MI355X (gfx950).
 *
 * Drop-in boundary for the linear layer of the tattletale inference framework.  The
 * reference operator is
 *     Linear{weight (out,in), bias?, in_features, out_features}, init(weight, bias),
 *     forward(x: (..., in)) -> (..., out)          workspace/transformers/src/layers/linear.nim:13-57
 * whose arithmetic is one FFI call
 *     torch::nn::functional::linear(input, weight[, bias])
 *                                                  workspace/libtorch/src/abi/neural_nets.nim:64-81
 * Each entry point below cites the reference interface it stands in for.  The reference
 * binds C libraries with `{.pragma: x, importc: "prefix_$1", cdecl, dynlib: lib.}`
 * (workspace/pcre2/pcre2.nim:376-384); every symbol here is plain C, `ttq_` prefixed and
 * takes raw pointers and sizes only, so it binds the same way.
 *
 * Conventions
 *   - All device pointers are HIP device memory on the current device; the library keeps
 *     no pointer to a caller's buffer after a call returns (work may still be in flight on `stream`).
 *   - Workspaces.  A few paths need device memory beyond inputs and outputs (partial sums of a
 *     launch split along K, the trellis GEMV's hand-off words, a bf16 or rotated copy of the
 *     activations).  The ttq_*_ws entry points take it from the caller -- the reference's
 *     convention, where the caller makes every tensor with from_blob / empty
 *     (workspace/libtorch/src/abi/torch_tensors.nim:250-289) -- allocate nothing, and can be
 *     captured into a HIP graph the first time they run.  The entry points without a workspace
 *     argument are the convenience form: the library allocates what the call needs on first use,
 *     one buffer per (device, stream), keeps it until ttq_release_workspaces, and such a first call
 *     must not happen under capture.  A graph captured with a library-owned workspace must be
 *     replayed on the stream it was captured on (another stream's launches use another buffer and
 *     would overlap it), and one host thread at a time may issue calls on a given stream.
 *   - `stream` is a hipStream_t passed as void*; NULL = the default stream.  Launches are
 *     asynchronous; the caller synchronises (same contract as a torch tensor op).
 *   - Return value: 0 on success, a negative ttq_status otherwise.  No C++ exception
 *     crosses this boundary.
 *   - Weights are (n_out, n_in) row-major; quantization blocks run along n_in.
 *   - Base pointers must be 16-byte aligned (torch allocations are).
 */
#ifndef TTQ_H
#define TTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTQ_VERSION 120 /* 0.1.2 */

/* Exported symbols: the library is built with hidden visibility by default. */
#if defined(TTQ_BUILD)
#define TTQ_API __attribute__((visibility("default")))
#else
#define TTQ_API
#endif

typedef enum {
  TTQ_OK = 0,
  TTQ_ERR_NULL = -1,        /* a required pointer is NULL */
  TTQ_ERR_SHAPE = -2,       /* dimension not positive / not a multiple of the block size */
  TTQ_ERR_ALIGN = -3,       /* base pointer not 16-byte aligned */
  TTQ_ERR_DTYPE = -4,       /* unknown or unsupported dtype code */
  TTQ_ERR_FORMAT = -5,      /* unknown format / bits / codebook */
  TTQ_ERR_UNSUPPORTED = -6, /* valid request outside what the kernels cover (size limits) */
  TTQ_ERR_HIP = -7,         /* a HIP runtime call failed; see ttq_last_hip_error() */
  TTQ_ERR_ALIAS = -8,       /* an output overlaps an input in a call that must run out of place */
  TTQ_ERR_WORKSPACE = -9    /* caller-owned workspace NULL, misaligned or smaller than ttq_workspace_bytes says */
} ttq_status;

/* Element types of activation / output / bias buffers.  They correspond to the
 * reference's ScalarKind members kFloat32, kFloat16, kBfloat16
 * (workspace/libtorch/src/abi/torch_tensors.nim:114-130). */
typedef enum { TTQ_F32 = 0, TTQ_F16 = 1, TTQ_BF16 = 2 } ttq_dtype;

typedef enum { TTQ_Q8_0 = 0, TTQ_Q4_K = 1, TTQ_Q6_K = 2, TTQ_EXL3 = 3 } ttq_format;

/* How ttq_linear_forward may trade accuracy for speed when there are several activation rows. */
typedef enum {
  TTQ_PRECISION_AUTO = 0,       /* from five rows on, whichever kernel of the activations' own type the shape makes cheaper */
  TTQ_PRECISION_F32_SCALES = 1, /* always the decode kernels: fp32 scales, rel-L2 <= 1e-3 whatever m is */
  TTQ_PRECISION_BF16_OK = 2     /* as AUTO, and fp32 activations may be rounded to bf16 for the matrix-core GEMM */
} ttq_precision;

/* Codebook functions of the trellis format. */
typedef enum { TTQ_CB_3INST = 0, TTQ_CB_MCG = 1 } ttq_codebook;

/* ---- library ---------------------------------------------------------------------- */

TTQ_API int ttq_version(void);
TTQ_API const char* ttq_strerror(int status);
/* hipError_t value of the most recent failed HIP call on this thread (0 if none). */
TTQ_API int ttq_last_hip_error(void);

/* Bytes of the packed weight buffer for an (n_out, n_in) matrix; negative status on bad
 * arguments.  `bits` is used by TTQ_EXL3 only (1..8).  Replaces weight.nbytes of the dense
 * tensor (workspace/libtorch/src/abi/torch_tensors.nim:192). */
TTQ_API int64_t ttq_packed_nbytes(int format, int64_t n_out, int64_t n_in, int bits);

/* ---- the operator ----------------------------------------------------------------- */

/* Plain-data description of one quantized linear layer: the quantized counterpart of the
 * reference's `Linear` object (linear.nim:13-27).  All pointers are device pointers owned
 * by the caller. */
typedef struct ttq_qlinear {
  int32_t format;        /* ttq_format */
  int32_t bits;          /* TTQ_EXL3: bits per weight (1..8); otherwise ignored */
  int32_t codebook;      /* TTQ_EXL3: ttq_codebook; otherwise ignored */
  int32_t bias_dtype;    /* ttq_dtype of `bias`; ignored when bias is NULL */
  int32_t precision;     /* ttq_precision */
  int32_t reserved;      /* 0 */
  int64_t n_out;         /* out_features */
  int64_t n_in;          /* in_features */
  const void* qweight;   /* packed blocks (Q8_0/Q4_K/Q6_K) or trellis words (EXL3) */
  const void* suh;       /* TTQ_EXL3: n_in fp16 input sign/scale vector, else NULL */
  const void* svh;       /* TTQ_EXL3: n_out fp16 output sign/scale vector, else NULL */
  const void* bias;      /* n_out values or NULL (linear.nim:26, Option[TorchTensor]) */
} ttq_qlinear;

/* y = x * W^T (+ bias) for x of shape (m, n_in), y of shape (m, n_out).
 * Replaces Linear.forward (linear.nim:45-57) and the F.linear call under it
 * (neural_nets.nim:64,73).  m == 1 runs the decode GEMV; m > 1 runs the prefill GEMM
 * (MFMA kernel for Q4_K with bf16 activations, a batched GEMV otherwise) -- the same
 * split the reference makes implicitly through x.size(1) (attn.nim:154-156).
 * Accuracy: up to four rows always run the decode kernels (fp32 scales; rel-L2 <= 1e-3 against the
 * canonical dequantized weights).  From five rows of bf16 (fp16) activations on, the library may
 * run matrix-core kernels that round each dequantized weight once to bf16 (fp16) -- the 2e-2 class
 * of the GEMM entry points -- when its cost estimate prefers them for the shape.  A layer with
 * precision == TTQ_PRECISION_F32_SCALES keeps the decode kernels, and with them the 1e-3 class,
 * for every m.  fp16 and fp32 activations stay in that 1e-3 class for every m by default: fp16
 * activations take the decode kernels, the fp16 few-row matrix-core kernel or, beyond 64 rows, the
 * fp16 form of the prefill GEMM (a packed fp16 copy of x in a workspace, weights rounded once to
 * fp16, fp16 matrix cores: about 2e-4 measured; a dequantized weight beyond the fp16 range becomes
 * an infinity there); fp32 activations take the decode kernels (which read them as 15-bit block
 * fixed point) or, from two rows on where that is cheaper, the same fp16 kernels (the few-row kernel, then the GEMM) over
 * a copy in which every row has been scaled by its own power of two (largest magnitude to 2^14) and
 * rounded to fp16, the factor undone on the sums (about 2e-4 measured for rows of any magnitude; a
 * non-finite value makes its own output row non-finite and no other).  Only a layer with precision == TTQ_PRECISION_BF16_OK lets
 * the library round 256 or more rows of fp32 activations to bf16 and run the bf16 GEMM on the copy
 * (2e-2 class).
 * Limits (TTQ_ERR_UNSUPPORTED beyond): every format takes any n_in (block formats: rows beyond
 * 65536 values for Q4_K / Q6_K with 16-bit activations, beyond 16384 otherwise, run a decode kernel
 * that stages nothing in LDS, at about half the rate of the staged ones); any m (rows are taken 65535 at a time where a
 * kernel needs that).  m == 0 or n_out == 0 returns TTQ_OK without touching a pointer. */
TTQ_API int ttq_linear_forward(const ttq_qlinear* layer, const void* x, int x_dtype, int64_t m,
                       void* y, int y_dtype, void* stream);

/* Bytes of caller-owned workspace that ttq_linear_forward_ws needs for this layer, row count and
 * activation type (0: none; negative status on bad arguments).  An upper bound that depends on the
 * device's compute-unit count; a pure host function.  No counterpart in the reference, where
 * F.linear allocates what it needs inside libtorch; the caller makes the buffer as it makes every
 * tensor (F.zeros / from_blob, torch_tensors.nim:250-289). */
TTQ_API int64_t ttq_workspace_bytes(const ttq_qlinear* layer, int64_t m, int x_dtype);

/* ttq_linear_forward with the workspace in the caller's hands: never allocates, safe to capture on
 * its first call.  `ws` is 16-byte aligned device memory of at least ttq_workspace_bytes(layer, m,
 * x_dtype) bytes (TTQ_ERR_WORKSPACE otherwise; ws may be NULL when that is 0), CLEARED TO ZERO ONCE
 * before its first use: the library keeps arrival counters and a generation count in its first
 * bytes and leaves them ready for the next call.  One workspace serves any sequence of calls for
 * any layers on one stream (each call sized by its own ttq_workspace_bytes); calls that may
 * overlap -- different streams -- need different workspaces. */
TTQ_API int ttq_linear_forward_ws(const ttq_qlinear* layer, const void* x, int x_dtype, int64_t m,
                          void* y, int y_dtype, void* ws, int64_t ws_bytes, void* stream);

/* Frees every workspace the library allocated for the entry points without a workspace argument.
 * Only when nothing that could use one is in flight, and no captured graph that was recorded
 * through such an entry point will be replayed again: synchronize the device first. */
TTQ_API int ttq_release_workspaces(void);

/* Which kernel family ttq_linear_forward launches for this layer, row count and types: a
 * ttq_route_id (>= 0) or a negative status.  It runs the dispatch code of ttq_linear_forward itself
 * with the launches switched off, touches no buffer and no device memory, and depends only on its
 * arguments and the current device's compute-unit count (256 when no device is visible).  No
 * counterpart in the reference: there F.linear chooses inside libtorch. */
typedef enum {
  TTQ_ROUTE_NONE = 0,
  TTQ_ROUTE_GEMV_Q4K_STREAM = 1,     /* Q4_K, weights streamed HBM -> LDS as whole cache lines */
  TTQ_ROUTE_GEMV_Q4K_STREAM4 = 2,    /* ... two to four activation rows per pass */
  TTQ_ROUTE_GEMV_Q4K_SLICE = 3,      /* ... long rows, K dealt to the wavefronts */
  TTQ_ROUTE_GEMV_Q4K_BATCH4 = 4,
  TTQ_ROUTE_GEMV_Q4K_BATCH = 5,
  TTQ_ROUTE_GEMV_Q4K_MFMA = 6,       /* register-streamed int8 matrix-core kernel */
  TTQ_ROUTE_GEMV_Q6K_STREAM = 7,
  TTQ_ROUTE_GEMV_Q6K_STREAM4 = 8,
  TTQ_ROUTE_GEMV_Q8_STREAM = 9,
  TTQ_ROUTE_GEMV_Q8_WIN = 10,
  TTQ_ROUTE_GEMV_Q8_MFMA = 11,
  TTQ_ROUTE_GEMV_DOT2 = 12,
  TTQ_ROUTE_GEMV_DOT2_MULTI = 13,
  TTQ_ROUTE_GEMV_GENERIC = 14,
  TTQ_ROUTE_GEMV_LONG = 15,          /* rows longer than the staged kernels take: nothing staged in LDS */
  TTQ_ROUTE_GEMM_SKINNY_F32_SCALED_F16 = 19, /* fp32 activations, few rows: the few-row kernel in fp16 over a copy scaled row by row */
  TTQ_ROUTE_GEMM_PC = 20,            /* producer / consumer prefill GEMM */
  TTQ_ROUTE_GEMM_PC_SPLIT_K = 21,    /* ... in several copies along K (takes a workspace) */
  TTQ_ROUTE_GEMM_SKINNY = 22,        /* 17-64 rows */
  TTQ_ROUTE_GEMM_SKINNY_CHUNKED = 23,
  TTQ_ROUTE_GEMM_Q4K_TILES = 24,     /* single-role tiled kernel: more than 4 GiB of activations */
  TTQ_ROUTE_GEMM_PC_BF16_COPY = 25,  /* TTQ_PRECISION_BF16_OK: fp32 activations rounded to bf16 by the packing pass */
  TTQ_ROUTE_GEMM_PC_PACKED = 26,     /* long launches: activations packed in fragment order first (takes a workspace) */
  TTQ_ROUTE_GEMM_PC_PACKED_SPLIT_K = 27,
  TTQ_ROUTE_GEMM_PC_F16 = 28,        /* fp16 activations: packed fp16 copy, weights rounded to fp16, fp16 matrix cores */
  TTQ_ROUTE_GEMM_PC_F32_SCALED_F16 = 29, /* fp32 activations: the same over a copy scaled row by row and rounded to fp16 */
  TTQ_ROUTE_EXL3_GEMV = 30,
  TTQ_ROUTE_EXL3_GEMV_SLICED = 31,   /* K sliced over workgroups that meet in a workspace */
  TTQ_ROUTE_EXL3_GEMM = 32,
  TTQ_ROUTE_EXL3_GEMV_TWO_LAUNCHES = 33
} ttq_route_id;
TTQ_API int ttq_route(const ttq_qlinear* layer, int64_t m, int x_dtype, int y_dtype);
TTQ_API const char* ttq_route_name(int route);

/* ---- decode GEMV, one entry per block format (m rows of x, normally m == 1) -------- */
/* y[m][n_out] (fp32) = x[m][n_in] * W^T.  Stand in for F.linear(x, weight) with a
 * (1, n_in) activation (neural_nets.nim:64).  Any n_in (rows beyond 65536 values for Q4_K / Q6_K
 * with 16-bit activations, beyond 16384 otherwise, take the unstaged kernel).  Two to four rows (a speculative step, a few sequences) of
 * 16-bit activations over a large Q4_K or Q6_K matrix cost about one pass over the weights, not
 * one per row; every row's result stays within the 1e-3 class of the single-row call.  A NaN or
 * an infinity among a row's activations, or in a block scale of a weight row, makes the outputs
 * they reach non-finite, as F.linear on the dequantized weight would; other outputs are unaffected. */
TTQ_API int ttq_gemv_q8_0(const void* w, const void* x, int x_dtype, float* y, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);
TTQ_API int ttq_gemv_q4_k(const void* w, const void* x, int x_dtype, float* y, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);
TTQ_API int ttq_gemv_q6_k(const void* w, const void* x, int x_dtype, float* y, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);

/* EXL3-style trellis GEMV: y = svh o H( T * H(suh o x) ), fp16 activations, fp32 output.
 * n_in and n_out must be multiples of 128 (Hadamard groups). */
TTQ_API int ttq_gemv_exl3(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                  const uint16_t* x_f16, float* y, int64_t m, int64_t n_out, int64_t n_in,
                  int bits, int codebook, void* stream);

/* ttq_gemv_exl3 for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments,
 * same results bit for bit; m <= 8.  Where ttq_gemv_exl3 takes its workspace (the words through which
 * the slices of the reduction meet) from hipMalloc on first use, this entry point uses a 4 MiB array
 * that is part of the library's device image: every GPU the library runs on holds one from the first
 * call there until the process ends.  It calls no allocating routine.  Returns TTQ_ERR_UNSUPPORTED
 * for m > 8 and for a launch that would need more than the 4 MiB (a device with more than 256
 * compute units).  All calls on one GPU share the array: calls that may overlap there (different
 * streams, different threads) race; calls on one stream do not.  Nothing is cleared between calls:
 * the words carry the tag of the launch that wrote them (the array's generation count + 1), and
 * every launch advances the count when its last group is done. */
TTQ_API int ttq_gemv_exl3_noalloc(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                  const uint16_t* x_f16, float* y, int64_t m, int64_t n_out, int64_t n_in,
                  int bits, int codebook, void* stream);

/* ---- prefill GEMM ------------------------------------------------------------------ */
/* Y[m][n_out] (bf16) = X[m][n_in] (bf16) * W^T, Q4_K weights dequantized to bf16 tiles and
 * multiplied with bf16 MFMA, fp32 accumulation.  Stands in for F.linear(x, weight) with a
 * (batch*seq, n_in) activation (neural_nets.nim:64; attn.nim:154-156 prefill case).
 * Up to 64 rows may run a kernel that dequantizes in registers instead of tiling W through LDS
 * (same arithmetic: weights rounded to bf16 once, fp32 accumulation); the library picks by shape.
 * Shapes with few output tiles and a long K are computed as up to eight partial products over slices
 * of K that meet in a workspace the library keeps per (device, stream) -- fp32, rows x columns x
 * slices, allocated on first use and grown on demand, so the first call of such a shape on a stream
 * must not happen under graph capture; the partial products are added in a fixed order (the same
 * bits on every call).  The same holds for ttq_gemm_q6_k, ttq_gemm_q8_0 and ttq_linear_forward. */
TTQ_API int ttq_gemm_q4_k(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);
/* The same operator for Q6_K and Q8_0 weights (a GGUF "Q4_K_M" file mixes Q4_K and Q6_K tensors;
 * every projection of attn.nim:154-156,189 and mlp.nim:56,60 sees seq_len > 1 at prefill).
 * n_in must be a multiple of 256. */
TTQ_API int ttq_gemm_q6_k(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);
TTQ_API int ttq_gemm_q8_0(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                  int64_t n_out, int64_t n_in, void* stream);
/* The three above with the workspace in the caller's hands (see ttq_linear_forward_ws for the
 * contract: cleared once, never allocates, capturable on the first call).  Size: ttq_workspace_bytes
 * of a ttq_qlinear with this format and shape, m and TTQ_BF16.  No counterpart in the reference. */
TTQ_API int ttq_gemm_q4_k_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                     int64_t n_out, int64_t n_in, void* ws, int64_t ws_bytes, void* stream);
TTQ_API int ttq_gemm_q6_k_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                     int64_t n_out, int64_t n_in, void* ws, int64_t ws_bytes, void* stream);
TTQ_API int ttq_gemm_q8_0_ws(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                     int64_t n_out, int64_t n_in, void* ws, int64_t ws_bytes, void* stream);
/* The operator for a trellis-coded weight and many activation rows (prefill: seq_len > 1 at every
 * projection, attn.nim:154-156): y (m, n_out) fp32 = svh o H( T * H(suh o x) ) for x (m, n_in) of any
 * dtype.  The activations are rotated once and rounded to fp16 (rel-L2 <= 2e-2 class, about 3e-4 in
 * practice); every weight is decoded once per 128 rows (tiled GEMM, split along K while compute
 * units are free).  The rotated activations and the partial sums of a split launch live in a workspace
 * the library allocates per (device, stream) on first use and grows on demand (up to 4096 rows of
 * n_in fp16 values), so the first call, and a call with more rows than any before, must not happen
 * under graph capture (ttq_gemm_exl3_ws has no such limit).  ttq_linear_forward takes this path by
 * itself from 9 to 48 rows on, depending on the matrix, unless the layer asks for
 * TTQ_PRECISION_F32_SCALES. */
TTQ_API int ttq_gemm_exl3(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                  const void* x, int x_dtype, float* y, int64_t m, int64_t n_out, int64_t n_in,
                  int bits, int codebook, void* stream);
/* ttq_gemm_exl3 and ttq_gemv_exl3 with the workspace in the caller's hands (contract of
 * ttq_linear_forward_ws; size: ttq_workspace_bytes of a TTQ_EXL3 ttq_qlinear of this shape).  No
 * counterpart in the reference. */
TTQ_API int ttq_gemm_exl3_ws(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                     const void* x, int x_dtype, float* y, int64_t m, int64_t n_out, int64_t n_in,
                     int bits, int codebook, void* ws, int64_t ws_bytes, void* stream);
TTQ_API int ttq_gemv_exl3_ws(const uint16_t* trellis, const uint16_t* suh_f16, const uint16_t* svh_f16,
                     const uint16_t* x_f16, float* y, int64_t m, int64_t n_out, int64_t n_in,
                     int bits, int codebook, void* ws, int64_t ws_bytes, void* stream);
/* Diagnostics: how many times the last slice of a sliced trellis GEMV looks at a hand-off word
 * that has not arrived before it gives the row up and writes NaN (default 65536; 0 = look once).
 * Process-wide; returns the previous value.  Exists so that the give-up path can be exercised from
 * the host with every kernel exiting normally.  No counterpart in the reference. */
TTQ_API int ttq_debug_set_exl3_poll_limit(int limit);
/* Prefill half of GatedMLP.forward in one kernel: y (m, n_ff) = silu(x Wg^T) * (x Wu^T) with the
 * fused gate||up weight of mlp.nim:39 (2*n_ff rows, gate rows first) -- gate_up_proj.forward
 * followed by silu_and_mul (mlp.nim:56-59, activations.nim:14-38), silu(g)*u formed in fp32 from
 * the fp32 accumulators and rounded once to bf16.  n_in a multiple of 256. 
 * Up to 64 rows may run the few-row kernel (see ttq_gemm_q4_k), same arithmetic. */
TTQ_API int ttq_gemm_q4_k_silu_mul(const void* w, const uint16_t* x_bf16, uint16_t* y_bf16, int64_t m,
                  int64_t n_ff, int64_t n_in, void* stream);

/* ---- device dequantizers (the bit-exactness contract made observable) -------------- */
/* out[n_out][n_in] in `out_dtype`: TTQ_F32 gives the canonical values; TTQ_BF16 gives them
 * rounded to nearest-even, i.e. exactly what the GEMM feeds to the matrix cores.  These
 * produce the dense weight the reference's Linear would have held (linear.nim:19). */
TTQ_API int ttq_dequant_q8_0(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream);
TTQ_API int ttq_dequant_q4_k(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream);
TTQ_API int ttq_dequant_q6_k(const void* w, void* out, int out_dtype, int64_t n_out, int64_t n_in, void* stream);
/* Decoded (unscaled, unrotated) trellis values as fp16, shape (n_out, n_in). */
TTQ_API int ttq_dequant_exl3(const uint16_t* trellis, uint16_t* out_f16, int64_t n_out, int64_t n_in,
                     int bits, int codebook, void* stream);
/* In-place orthonormal 128-group Hadamard transform of n fp32 values, optionally
 * multiplying by an fp16 vector before (pre) and/or after (post) the transform. */
TTQ_API int ttq_hadamard128_f32(float* v, const uint16_t* pre_f16, const uint16_t* post_f16,
                        int64_t n, void* stream);

/* ---- gated MLP: activation and its fusion into the decode GEMV ---------------------- */
/* out[m][h] = silu(in[m][0:h]) * in[m][h:2h], in and out of the same dtype.  Stands in for
 * silu_and_mul (workspace/transformers/src/kernels/activations.nim:14-38), applied by
 * GatedMLP.forward to the output of the fused gate/up projection (mlp.nim:56-60). */
TTQ_API int ttq_silu_and_mul(const void* in, void* out, int dtype, int64_t m, int64_t h, void* stream);
/* y[m][n_ff] = silu(x Wg^T) * (x Wu^T) in one kernel, W = [Wg; Wu] the (2*n_ff, n_in) Q4_K
 * matrix GatedMLP.init builds by row concatenation (mlp.nim:39).  Replaces
 * gate_up_proj.forward followed by silu_and_mul (mlp.nim:56-59) for decode.  16-bit
 * activations only; returns TTQ_ERR_UNSUPPORTED for shapes the fused kernel does not cover
 * (n_ff < 16, fp32 activations): call ttq_gemv_q4_k + ttq_silu_and_mul then. */
TTQ_API int ttq_gemv_q4_k_silu_mul(const void* w, const void* x, int x_dtype, void* y, int y_dtype,
                           int64_t m, int64_t n_ff, int64_t n_in, void* stream);

/* ---- RMSNorm and its fusion into the decode GEMV -------------------------------------- */
/* t = x (+ residual, rounded to dtype); normed = t * rsqrt(mean(t^2) + eps) * gamma, fp32
 * arithmetic, one rounding to dtype.  x, residual, new_residual_out, normed_out are (m, n);
 * gamma is (n).  Stands in for RmsNorm.forward (residual = NULL) and
 * RmsNorm.forward_with_residual, which returns (normalized, new_residual)
 * (workspace/transformers/src/layers/norm.nim:23-38; torch::rms_norm,
 * workspace/libtorch/src/abi/neural_nets.nim:144-146).  new_residual_out may be NULL.
 * The outputs may be the inputs (normed_out == x, new_residual_out == residual: the in-place
 * add of the residual stream); other overlaps are not allowed.  All pointers 16-byte aligned. */
TTQ_API int ttq_rmsnorm(const void* x, const void* residual, const void* gamma, float eps, int dtype,
                void* new_residual_out, void* normed_out, int64_t m, int64_t n, void* stream);
/* y = Linear(RmsNorm(x [, residual])) in one kernel for a Q4_K weight and 16-bit activations:
 * the "fused add + RMSNorm" that norm.nim:35 leaves as a TODO, placed in front of the decode
 * GEMV.  With silu_mul != 0 the weight is the (2*n_out, n_in) gate/up matrix and y is
 * silu_and_mul of the projection (mlp.nim:56-59).  residual, new_residual_out and normed_out
 * may be NULL; normed_out receives the normalized row the GEMV consumed (other projections of
 * the same block read it).  With two to four rows, normed_out given and a large matrix (rows of 2048 or
 * 4096 values, 4096 weight rows or more) the call is two launches -- the normalization, then one pass
 * over the weights for all rows -- which is faster than one weight pass per row; the results are those of
 * ttq_rmsnorm followed by ttq_gemv_q4_k / ttq_gemv_q4_k_silu_mul on normed_out.
 * Returns TTQ_ERR_UNSUPPORTED for fp32 activations or n_out < 16.
 * Out of place only: every workgroup re-reads x and residual while the outputs are written, so
 * new_residual_out and normed_out must not overlap x, residual or each other (TTQ_ERR_ALIAS);
 * use ttq_rmsnorm for the in-place form. */
TTQ_API int ttq_gemv_q4_k_rmsnorm(const void* w, const void* x, const void* residual, const void* gamma,
                          float eps, int x_dtype, void* new_residual_out, void* normed_out, void* y,
                          int y_dtype, int64_t m, int64_t n_out, int64_t n_in, int silu_mul, void* stream);

/* ---- host-side preparation (CPU code; no GPU needed) ------------------------------- */
/* Weight preparation happens once at load time, off the hot path; the reference's
 * counterpart is building the dense weight tensor handed to Linear.init (linear.nim:29-43,
 * mlp.nim:39-41).  All pointers here are HOST pointers. */

/* Counter-based normal generator: out[i] = sigma * N(0,1) drawn from (seed, stream, i).
 * Identical bytes on every machine with the same libm. */
TTQ_API int ttq_host_fill_normal(uint64_t seed, uint64_t stream, float sigma, float* out, int64_t n);

TTQ_API int ttq_host_quantize_q8_0(const float* w, void* out, int64_t n_out, int64_t n_in);
TTQ_API int ttq_host_quantize_q4_k(const float* w, void* out, int64_t n_out, int64_t n_in);
TTQ_API int ttq_host_quantize_q6_k(const float* w, void* out, int64_t n_out, int64_t n_in);
/* Rotates and trellis-encodes w (n_out, n_in).  Writes trellis words
 * [n_in/16][n_out/16][16*bits], suh (n_in fp16 signs drawn from `seed`) and svh (n_out
 * fp16: sign * per-channel scale).  Encoder is a greedy search; only the decoder is a
 * format contract. */
TTQ_API int ttq_host_quantize_exl3(const float* w, uint16_t* trellis, uint16_t* suh_f16,
                           uint16_t* svh_f16, int64_t n_out, int64_t n_in, int bits,
                           int codebook, uint64_t seed);

/* fp32 <-> 16-bit conversions, round-to-nearest-even. */
TTQ_API int ttq_host_f32_to_bf16(const float* in, uint16_t* out, int64_t n);
TTQ_API int ttq_host_f32_to_f16(const float* in, uint16_t* out, int64_t n);
TTQ_API int ttq_host_bf16_to_f32(const uint16_t* in, float* out, int64_t n);
TTQ_API int ttq_host_f16_to_f32(const uint16_t* in, float* out, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* TTQ_H */
