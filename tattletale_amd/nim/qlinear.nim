# Nim binding of libttq_hip.so and a QuantLinear layer shaped like the reference's Linear
# (workspace/transformers/src/layers/linear.nim:13-57).  Mechanically derived from
# include/ttq.h, in the reference's own FFI idiom for C libraries
# (workspace/pcre2/pcre2.nim:376-384: a pragma alias with importc "prefix_$1", cdecl, dynlib).
#
# NOT compiled in this repository: no Nim toolchain is available where it is built.  All
# testing goes through the same C ABI from Python (tattletale_amd/qlinear.py).

import std/options
import workspace/libtorch as F

const ttqlib = "libttq_hip.so"
{.pragma: ttq, importc: "ttq_$1", cdecl, dynlib: ttqlib.}

type
  QuantFormat* {.size: sizeof(cint).} = enum
    kQ8_0 = 0, kQ4_K = 1, kQ6_K = 2, kEXL3 = 3
  TtqDtype* {.size: sizeof(cint).} = enum
    kTtqF32 = 0, kTtqF16 = 1, kTtqBF16 = 2
  TtqPrecision* {.size: sizeof(cint).} = enum
    kTtqAuto = 0, kTtqF32Scales = 1, kTtqBf16Ok = 2
      ## kTtqF32Scales: decode kernels (fp32 scales) for every batch size
      ## kTtqBf16Ok: fp32 activations may be rounded to bf16 for the matrix-core GEMM (fp16 ones have their own)
  TtqQLinear* {.bycopy.} = object      ## struct ttq_qlinear
    format*, bits*, codebook*, bias_dtype*: int32
    precision*, reserved*: int32       ## ttq_precision, 0
    n_out*, n_in*: int64
    qweight*, suh*, svh*, bias*: pointer
  QuantLinearError* = object of ValueError

proc version*(): cint {.ttq.}
proc strerror*(status: cint): cstring {.ttq.}
proc last_hip_error*(): cint {.ttq.}
proc packed_nbytes*(format: cint, n_out, n_in: int64, bits: cint): int64 {.ttq.}
proc linear_forward*(layer: ptr TtqQLinear, x: pointer, x_dtype: cint, m: int64,
                     y: pointer, y_dtype: cint, stream: pointer): cint {.ttq.}
proc workspace_bytes*(layer: ptr TtqQLinear, m: int64, x_dtype: cint): int64 {.ttq.}
proc linear_forward_ws*(layer: ptr TtqQLinear, x: pointer, x_dtype: cint, m: int64,
                        y: pointer, y_dtype: cint, ws: pointer, ws_bytes: int64, stream: pointer): cint {.ttq.}
proc release_workspaces*(): cint {.ttq.}
proc route*(layer: ptr TtqQLinear, m: int64, x_dtype, y_dtype: cint): cint {.ttq.}
proc route_name*(route: cint): cstring {.ttq.}
proc gemv_q8_0*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_q4_k*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_q6_k*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_exl3*(trellis, suh, svh, x: ptr uint16, y: ptr cfloat, m, n_out, n_in: int64,
                bits, codebook: cint, stream: pointer): cint {.ttq.}
proc gemv_exl3_noalloc*(trellis, suh, svh, x: ptr uint16, y: ptr cfloat, m, n_out, n_in: int64,
                        bits, codebook: cint, stream: pointer): cint {.ttq.}
proc gemm_exl3*(trellis, suh, svh: ptr uint16, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64,
                bits, codebook: cint, stream: pointer): cint {.ttq.}
proc gemv_exl3_ws*(trellis, suh, svh, x: ptr uint16, y: ptr cfloat, m, n_out, n_in: int64,
                   bits, codebook: cint, ws: pointer, ws_bytes: int64, stream: pointer): cint {.ttq.}
proc gemm_exl3_ws*(trellis, suh, svh: ptr uint16, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64,
                   bits, codebook: cint, ws: pointer, ws_bytes: int64, stream: pointer): cint {.ttq.}
proc debug_set_exl3_poll_limit*(limit: cint): cint {.ttq.}
proc gemm_q4_k_ws*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, ws: pointer, ws_bytes: int64,
                   stream: pointer): cint {.ttq.}
proc gemm_q6_k_ws*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, ws: pointer, ws_bytes: int64,
                   stream: pointer): cint {.ttq.}
proc gemm_q8_0_ws*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, ws: pointer, ws_bytes: int64,
                   stream: pointer): cint {.ttq.}
proc gemm_q4_k*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemm_q6_k*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemm_q8_0*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q8_0*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q4_k*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q6_k*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_exl3*(trellis, dst: ptr uint16, n_out, n_in: int64, bits, codebook: cint, stream: pointer): cint {.ttq.}
proc hadamard128_f32*(v: ptr cfloat, pre_f16, post_f16: ptr uint16, n: int64, stream: pointer): cint {.ttq.}
proc silu_and_mul*(src, dst: pointer, dtype: cint, m, h: int64, stream: pointer): cint {.ttq.}
proc gemm_q4_k_silu_mul*(w: pointer, x, y: ptr uint16, m, n_ff, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_q4_k_silu_mul*(w, x: pointer, x_dtype: cint, y: pointer, y_dtype: cint, m, n_ff, n_in: int64,
                         stream: pointer): cint {.ttq.}
proc rmsnorm*(x, residual, gamma: pointer, eps: cfloat, dtype: cint, new_residual_out, normed_out: pointer,
              m, n: int64, stream: pointer): cint {.ttq.}
proc gemv_q4_k_rmsnorm*(w, x, residual, gamma: pointer, eps: cfloat, x_dtype: cint,
                        new_residual_out, normed_out, y: pointer, y_dtype: cint, m, n_out, n_in: int64,
                        silu_mul: cint, stream: pointer): cint {.ttq.}
# host-side preparation (CPU code)
proc host_fill_normal*(seed, stream: uint64, sigma: cfloat, dst: ptr cfloat, n: int64): cint {.ttq.}
proc host_quantize_q8_0*(w: ptr cfloat, dst: pointer, n_out, n_in: int64): cint {.ttq.}
proc host_quantize_q4_k*(w: ptr cfloat, dst: pointer, n_out, n_in: int64): cint {.ttq.}
proc host_quantize_q6_k*(w: ptr cfloat, dst: pointer, n_out, n_in: int64): cint {.ttq.}
proc host_quantize_exl3*(w: ptr cfloat, trellis, suh_f16, svh_f16: ptr uint16, n_out, n_in: int64,
                         bits, codebook: cint, seed: uint64): cint {.ttq.}
proc host_f32_to_bf16*(src: ptr cfloat, dst: ptr uint16, n: int64): cint {.ttq.}
proc host_f32_to_f16*(src: ptr cfloat, dst: ptr uint16, n: int64): cint {.ttq.}
proc host_bf16_to_f32*(src: ptr uint16, dst: ptr cfloat, n: int64): cint {.ttq.}
proc host_f16_to_f32*(src: ptr uint16, dst: ptr cfloat, n: int64): cint {.ttq.}

# The stream torch's own kernels of this thread run on, so that a layer keeps its place in the
# caller's stream order (a ROCm build of libtorch names its HIP streams c10::cuda as well).
proc currentStream*(): pointer {.importcpp: "((void*)c10::cuda::getCurrentCUDAStream().stream())",
                                 header: "<c10/cuda/CUDAStream.h>".}

func ttqDtype(k: ScalarKind): cint =
  case k
  of kFloat32: 0
  of kFloat16: 1
  of kBfloat16: 2
  else: raise newException(QuantLinearError, "unsupported dtype " & $k)

type
  QuantLinear* = object
    ## Quantized counterpart of Linear: packed weight instead of a dense tensor.
    qweight*: TorchTensor           ## kUint8 packed blocks / kInt16 trellis words, on the GPU
    format*: QuantFormat
    bias*: Option[TorchTensor]
    suh*, svh*: Option[TorchTensor] ## EXL3 only, kFloat16
    bits*, codebook*: int
    in_features*, out_features*: int
    precision*: TtqPrecision

func init*(_: type QuantLinear, qweight: TorchTensor, format: QuantFormat,
           in_features, out_features: int, bias = none(TorchTensor),
           suh = none(TorchTensor), svh = none(TorchTensor),
           bits = 0, codebook = 1, precision = kTtqAuto): QuantLinear =
  ## Creates the layer from existing packed weights (no copy), as Linear.init does.
  let need = packed_nbytes(format.cint, out_features, in_features, bits.cint)
  if need < 0 or need != qweight.nbytes.int64:
    raise newException(QuantLinearError, "packed buffer size does not match the dimensions")
  QuantLinear(qweight: qweight, format: format, bias: bias, suh: suh, svh: svh, bits: bits,
              codebook: codebook, in_features: in_features, out_features: out_features,
              precision: precision)

func descriptor(self: QuantLinear): TtqQLinear =
  TtqQLinear(
    format: self.format.int32, bits: self.bits.int32, codebook: self.codebook.int32,
    bias_dtype: (if self.bias.isSome: ttqDtype(self.bias.get().scalarType()).int32 else: 0),
    precision: self.precision.int32, reserved: 0,
    n_out: self.out_features, n_in: self.in_features,
    qweight: self.qweight.data_ptr(byte),
    suh: (if self.suh.isSome: self.suh.get().data_ptr(byte) else: nil),
    svh: (if self.svh.isSome: self.svh.get().data_ptr(byte) else: nil),
    bias: (if self.bias.isSome: self.bias.get().data_ptr(byte) else: nil))

proc workspaceBytes*(self: QuantLinear, m: int, dtype: ScalarKind): int64 =
  ## What forward(x, workspace) needs for m rows: make it with F.zeros (cleared once, then reusable).
  var desc = self.descriptor()
  result = workspace_bytes(addr desc, m, ttqDtype(dtype))
  if result < 0:
    raise newException(QuantLinearError, "ttq_workspace_bytes: " & $strerror(result.cint))

proc forward*(self: QuantLinear, x: TorchTensor, workspace = none(TorchTensor)): TorchTensor =
  ## x: (..., in_features) -> (..., out_features); launches on torch's current stream.  With a workspace
  ## (a kUint8 tensor from F.zeros of at least workspaceBytes, torch_tensors.nim:280-289) the library
  ## allocates nothing and the call can be captured into a graph the first time it runs.
  var shape = x.sizes().asNimView().toSeq()      # (..., in) -> (..., out)
  shape[^1] = self.out_features
  let m = x.numel() div self.in_features
  result = F.empty(shape, x.options())
  var desc = self.descriptor()
  let rc =
    if workspace.isSome:
      linear_forward_ws(addr desc, x.data_ptr(byte), ttqDtype(x.scalarType()), m, result.data_ptr(byte),
                        ttqDtype(x.scalarType()), workspace.get().data_ptr(byte), workspace.get().nbytes.int64,
                        currentStream())
    else:
      linear_forward(addr desc, x.data_ptr(byte), ttqDtype(x.scalarType()), m,
                     result.data_ptr(byte), ttqDtype(x.scalarType()), currentStream())
  if rc != 0:
    raise newException(QuantLinearError, "ttq_linear_forward: " & $strerror(rc))

# ---------------------------------------------------------------------------- gated MLP
# Shaped like GatedMLP (workspace/transformers/src/layers/mlp.nim:25-60): one fused gate/up
# projection, silu_and_mul (workspace/transformers/src/kernels/activations.nim:14-38), down.

const kTtqErrUnsupported = -6
const kFusedGemmMinRows = 2048   # below it the plain GEMM (packed activations) + silu_and_mul are 4 to 6 % faster
const kFusedFewRowsMin = 17     # 17..64 rows: the few-row kernel with silu_and_mul in its epilogue
const kFusedFewRowsMax = 64

type
  QuantGatedMLP* = object
    gate_up_proj*: QuantLinear    ## (2 * intermediate, hidden), gate rows first (mlp.nim:39)
    down_proj*: QuantLinear       ## (hidden, intermediate)

func init*(_: type QuantGatedMLP, gate_up_proj, down_proj: QuantLinear): QuantGatedMLP =
  ## Row-wise block formats concatenate as bytes, so the caller builds gate_up_proj.qweight
  ## with F.cat([gate_packed, up_packed], 0) exactly as mlp.nim:39 does for dense weights.
  if gate_up_proj.out_features != 2 * down_proj.in_features or
     gate_up_proj.in_features != down_proj.out_features:
    raise newException(QuantLinearError, "gate_up / down shapes do not form a gated MLP")
  QuantGatedMLP(gate_up_proj: gate_up_proj, down_proj: down_proj)

proc quant_silu_and_mul*(x: TorchTensor): TorchTensor =
  ## (..., 2h) -> (..., h), drop-in for silu_and_mul.
  var shape = x.sizes().asNimView().toSeq()
  let h = shape[^1] div 2
  shape[^1] = h
  result = F.empty(shape, x.options())
  let rc = silu_and_mul(x.data_ptr(byte), result.data_ptr(byte), ttqDtype(x.scalarType()),
                        x.numel() div (2 * h), h, currentStream())
  if rc != 0: raise newException(QuantLinearError, "ttq_silu_and_mul: " & $strerror(rc))

proc forward*(self: QuantGatedMLP, x: TorchTensor): TorchTensor =
  ## x (..., hidden) -> (..., hidden).  Decode on Q4_K weights takes the fused kernel.
  let gu = self.gate_up_proj
  let nff = self.down_proj.in_features
  let m = x.numel() div gu.in_features
  # one row, or two to four rows on the shapes whose fused kernel reads the weights once for all of them
  let few = m >= 2 and m <= 4 and (gu.in_features == 2048 or gu.in_features == 4096) and nff mod 8 == 0 and
            nff >= 2048 and nff <= 16384
  if gu.format == kQ4_K and gu.bias.isNone and (m == 1 or few):
    var shape = x.sizes().asNimView().toSeq()
    shape[^1] = nff
    let act = F.empty(shape, x.options())
    let rc = gemv_q4_k_silu_mul(gu.qweight.data_ptr(byte), x.data_ptr(byte), ttqDtype(x.scalarType()),
                                act.data_ptr(byte), ttqDtype(x.scalarType()), m, nff, gu.in_features, currentStream())
    if rc == 0: return self.down_proj.forward(act)
    if rc != kTtqErrUnsupported:
      raise newException(QuantLinearError, "ttq_gemv_q4_k_silu_mul: " & $strerror(rc))
  elif gu.format == kQ4_K and gu.bias.isNone and x.scalarType() == kBfloat16 and
       (m >= kFusedGemmMinRows or (m >= kFusedFewRowsMin and m <= kFusedFewRowsMax)):
    # prefill: silu_and_mul in the GEMM epilogue (breaks even at 512 rows, 15 % faster at 2048);
    # 17..64 rows: the same entry point runs the few-row kernel
    var shape = x.sizes().asNimView().toSeq()
    shape[^1] = nff
    let act = F.empty(shape, x.options())
    let rc = gemm_q4_k_silu_mul(gu.qweight.data_ptr(byte), cast[ptr uint16](x.data_ptr(byte)),
                                cast[ptr uint16](act.data_ptr(byte)), m, nff, gu.in_features, currentStream())
    if rc == 0: return self.down_proj.forward(act)
    if rc != kTtqErrUnsupported:
      raise newException(QuantLinearError, "ttq_gemm_q4_k_silu_mul: " & $strerror(rc))
  result = self.down_proj.forward(quant_silu_and_mul(gu.forward(x)))

# ------------------------------------------------------------------------------ RMSNorm
# Shaped like RmsNorm (workspace/transformers/src/layers/norm.nim:13-38).

type
  QuantRmsNorm* = object
    weight*: TorchTensor
    eps*: float
    hidden_size*: int

func init*(_: type QuantRmsNorm, weight: TorchTensor, eps: float = 1e-6): QuantRmsNorm =
  QuantRmsNorm(weight: weight, eps: eps, hidden_size: weight.size(0))

proc forward_with_residual*(self: QuantRmsNorm, hidden_state, residual: TorchTensor): (TorchTensor, TorchTensor) =
  ## (normalized, new_residual), one kernel instead of an add and an rms_norm (the TODO of norm.nim:35).
  let normalized = F.empty(hidden_state.sizes(), hidden_state.options())
  let new_residual = F.empty(hidden_state.sizes(), hidden_state.options())
  let rc = rmsnorm(hidden_state.data_ptr(byte), residual.data_ptr(byte), self.weight.data_ptr(byte),
                   self.eps.cfloat, ttqDtype(hidden_state.scalarType()), new_residual.data_ptr(byte),
                   normalized.data_ptr(byte), hidden_state.numel() div self.hidden_size, self.hidden_size, currentStream())
  if rc != 0: raise newException(QuantLinearError, "ttq_rmsnorm: " & $strerror(rc))
  (normalized, new_residual)

proc forward_norm_gate_up*(norm: QuantRmsNorm, mlp: QuantGatedMLP,
                           hidden_state, residual: TorchTensor): (TorchTensor, TorchTensor) =
  ## Decode: add + RMSNorm + gate/up projection + silu_and_mul in ONE launch, then the down
  ## projection.  Returns (mlp output, new_residual).
  let gu = mlp.gate_up_proj
  let nff = mlp.down_proj.in_features
  var shape = hidden_state.sizes().asNimView().toSeq()
  shape[^1] = nff
  let act = F.empty(shape, hidden_state.options())
  let new_residual = F.empty(hidden_state.sizes(), hidden_state.options())
  let rc = gemv_q4_k_rmsnorm(gu.qweight.data_ptr(byte), hidden_state.data_ptr(byte), residual.data_ptr(byte),
                             norm.weight.data_ptr(byte), norm.eps.cfloat, ttqDtype(hidden_state.scalarType()),
                             new_residual.data_ptr(byte), nil, act.data_ptr(byte),
                             ttqDtype(hidden_state.scalarType()), hidden_state.numel() div gu.in_features,
                             nff, gu.in_features, 1, currentStream())
  if rc != 0: raise newException(QuantLinearError, "ttq_gemv_q4_k_rmsnorm: " & $strerror(rc))
  (mlp.down_proj.forward(act), new_residual)
