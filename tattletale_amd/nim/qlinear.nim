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
  TtqQLinear* {.bycopy.} = object      ## struct ttq_qlinear
    format*, bits*, codebook*, bias_dtype*: int32
    n_out*, n_in*: int64
    qweight*, suh*, svh*, bias*: pointer
  QuantLinearError* = object of ValueError

proc version*(): cint {.ttq.}
proc strerror*(status: cint): cstring {.ttq.}
proc last_hip_error*(): cint {.ttq.}
proc packed_nbytes*(format: cint, n_out, n_in: int64, bits: cint): int64 {.ttq.}
proc linear_forward*(layer: ptr TtqQLinear, x: pointer, x_dtype: cint, m: int64,
                     y: pointer, y_dtype: cint, stream: pointer): cint {.ttq.}
proc gemv_q8_0*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_q4_k*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_q6_k*(w, x: pointer, x_dtype: cint, y: ptr cfloat, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc gemv_exl3*(trellis, suh, svh, x: ptr uint16, y: ptr cfloat, m, n_out, n_in: int64,
                bits, codebook: cint, stream: pointer): cint {.ttq.}
proc gemm_q4_k*(w: pointer, x, y: ptr uint16, m, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q8_0*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q4_k*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_q6_k*(w, dst: pointer, out_dtype: cint, n_out, n_in: int64, stream: pointer): cint {.ttq.}
proc dequant_exl3*(trellis, dst: ptr uint16, n_out, n_in: int64, bits, codebook: cint, stream: pointer): cint {.ttq.}

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

func init*(_: type QuantLinear, qweight: TorchTensor, format: QuantFormat,
           in_features, out_features: int, bias = none(TorchTensor),
           suh = none(TorchTensor), svh = none(TorchTensor),
           bits = 0, codebook = 1): QuantLinear =
  ## Creates the layer from existing packed weights (no copy), as Linear.init does.
  let need = packed_nbytes(format.cint, out_features, in_features, bits.cint)
  if need < 0 or need != qweight.nbytes.int64:
    raise newException(QuantLinearError, "packed buffer size does not match the dimensions")
  QuantLinear(qweight: qweight, format: format, bias: bias, suh: suh, svh: svh, bits: bits,
              codebook: codebook, in_features: in_features, out_features: out_features)

proc forward*(self: QuantLinear, x: TorchTensor): TorchTensor =
  ## x: (..., in_features) -> (..., out_features); launches on the current stream.
  var shape = x.sizes().asNimView().toSeq()      # (..., in) -> (..., out)
  shape[^1] = self.out_features
  let m = x.numel() div self.in_features
  let outKind = if self.format == kEXL3: kFloat32 else: x.scalarType()
  result = F.empty(shape, x.options().dtype(outKind))
  var desc = TtqQLinear(
    format: self.format.int32, bits: self.bits.int32, codebook: self.codebook.int32,
    bias_dtype: (if self.bias.isSome: ttqDtype(self.bias.get().scalarType()).int32 else: 0),
    n_out: self.out_features, n_in: self.in_features,
    qweight: self.qweight.data_ptr(byte),
    suh: (if self.suh.isSome: self.suh.get().data_ptr(byte) else: nil),
    svh: (if self.svh.isSome: self.svh.get().data_ptr(byte) else: nil),
    bias: (if self.bias.isSome: self.bias.get().data_ptr(byte) else: nil))
  let rc = linear_forward(addr desc, x.data_ptr(byte), ttqDtype(x.scalarType()), m,
                          result.data_ptr(byte), ttqDtype(outKind), nil)
  if rc != 0:
    raise newException(QuantLinearError, "ttq_linear_forward: " & $strerror(rc))
  if outKind != x.scalarType(): result = result.to(x.scalarType())
