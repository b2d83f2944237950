"""Packed weights from disk: a minimal GGUF (v2/v3) reader and writer, and the ``U8``-tensor
convention for safetensors files.

The reference's container is safetensors, memory-mapped and handed to libtorch without a copy
(workspace/safetensors/src/safetensors.nim:256-274,
workspace/transformers/src/safetensors_libtorch.nim:57-107); its comments anticipate loading
straight to the GPU (safetensors.nim:11-15).  The quantized layer needs no new dtype there:
packed blocks travel as ``U8`` tensors (safetensors_libtorch.nim:44), and the same bytes are the
tensor-data section of a GGUF file, whose Q8_0 / Q4_K / Q6_K block layouts are the ones
``libttq_hip.so`` consumes (rows of blocks along the input dimension, no repacking).

Only what the linear layer needs is implemented: header, metadata key/values, tensor directory,
and zero-copy (memory-mapped) views of tensor data.  No file produced by another GGUF writer was
available to check against, so compatibility with such files is by specification only.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Any, BinaryIO, Dict, Iterable, List, Optional, Tuple

import numpy as np

from . import _lib

GGUF_MAGIC = 0x46554747          # "GGUF" little-endian
DEFAULT_ALIGNMENT = 32

# ggml tensor types this library understands -> (format code or numpy dtype, block elements, block bytes)
GGML_F32, GGML_F16, GGML_Q8_0, GGML_Q4_K, GGML_Q6_K, GGML_BF16 = 0, 1, 8, 12, 14, 30
_BLOCK = {GGML_Q8_0: (_lib.Q8_0, 32, 34), GGML_Q4_K: (_lib.Q4_K, 256, 144), GGML_Q6_K: (_lib.Q6_K, 256, 210)}
_PLAIN = {GGML_F32: (np.float32, 4), GGML_F16: (np.float16, 2), GGML_BF16: (np.uint16, 2)}
_FORMAT_TO_GGML = {_lib.Q8_0: GGML_Q8_0, _lib.Q4_K: GGML_Q4_K, _lib.Q6_K: GGML_Q6_K}

# metadata value types
_U8, _I8, _U16, _I16, _U32, _I32, _F32, _BOOL, _STR, _ARR, _U64, _I64, _F64 = range(13)
_SCALAR = {_U8: "<B", _I8: "<b", _U16: "<H", _I16: "<h", _U32: "<I", _I32: "<i", _F32: "<f", _BOOL: "<?",
           _U64: "<Q", _I64: "<q", _F64: "<d"}


class GGUFError(ValueError):
    """Malformed or unsupported GGUF content."""


@dataclass(frozen=True)
class TensorInfo:
    name: str
    shape: Tuple[int, ...]        # torch order: (n_out, n_in) for a weight matrix
    ggml_type: int
    offset: int                   # absolute file offset of the data
    nbytes: int

    @property
    def format(self) -> Optional[int]:
        """Library format code for block-quantized tensors, None for plain ones."""
        return _BLOCK[self.ggml_type][0] if self.ggml_type in _BLOCK else None


class _Reader:
    def __init__(self, buf, size: int):
        self.buf, self.size, self.pos = buf, size, 0

    def take(self, fmt: str):
        n = struct.calcsize(fmt)
        if self.pos + n > self.size:
            raise GGUFError("truncated file (offset %d)" % self.pos)
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += n
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if n > self.size - self.pos:
            raise GGUFError("truncated string (offset %d)" % self.pos)
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8")
        self.pos += n
        return s

    def value(self, vt: int, depth: int = 0):
        if vt in _SCALAR:
            return self.take(_SCALAR[vt])
        if vt == _STR:
            return self.string()
        if vt == _ARR and depth == 0:
            et, n = self.take("<I"), self.take("<Q")
            if n > self.size:
                raise GGUFError("array length out of range")
            return [self.value(et, 1) for _ in range(n)]
        raise GGUFError("unknown metadata value type %d" % vt)


def tensor_nbytes(ggml_type: int, shape: Tuple[int, ...]) -> int:
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    if ggml_type in _BLOCK:
        _, be, bb = _BLOCK[ggml_type]
        if not shape or shape[-1] % be:
            raise GGUFError("row length %s is not a multiple of the block size %d" % (shape[-1:] or 0, be))
        return n // be * bb
    if ggml_type in _PLAIN:
        return n * _PLAIN[ggml_type][1]
    raise GGUFError("unsupported ggml tensor type %d" % ggml_type)


class GGUFFile:
    """Read-only view of a GGUF file: ``metadata`` (dict), ``tensors`` (name -> TensorInfo) and
    zero-copy ``data(name)``.  The file stays memory-mapped until ``close``."""

    def __init__(self, path: str):
        self.path = path
        self._f: Optional[BinaryIO] = open(path, "rb")
        try:
            size = os.fstat(self._f.fileno()).st_size
            if size < 24:
                raise GGUFError("file too short for a GGUF header")
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
            r = _Reader(self._mm, size)
            if r.take("<I") != GGUF_MAGIC:
                raise GGUFError("not a GGUF file (bad magic)")
            self.version = r.take("<I")
            if self.version not in (2, 3):
                raise GGUFError("unsupported GGUF version %d" % self.version)
            n_tensors, n_kv = r.take("<Q"), r.take("<Q")
            if n_tensors > size or n_kv > size:
                raise GGUFError("implausible tensor / metadata counts")
            self.metadata: Dict[str, Any] = {}
            for _ in range(n_kv):
                key = r.string()
                self.metadata[key] = r.value(r.take("<I"))
            infos = []
            for _ in range(n_tensors):
                name = r.string()
                nd = r.take("<I")
                if nd > 4:
                    raise GGUFError("tensor %r has %d dimensions" % (name, nd))
                ne = [r.take("<Q") for _ in range(nd)]
                infos.append((name, tuple(reversed(ne)), r.take("<I"), r.take("<Q")))
            self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
            if self.alignment <= 0 or self.alignment & (self.alignment - 1):
                raise GGUFError("alignment %d is not a power of two" % self.alignment)
            self.data_offset = (r.pos + self.alignment - 1) // self.alignment * self.alignment
            self.tensors: Dict[str, TensorInfo] = {}
            for name, shape, gt, rel in infos:
                nb = tensor_nbytes(gt, shape) if (gt in _BLOCK or gt in _PLAIN) else -1
                off = self.data_offset + rel
                if rel % self.alignment:
                    raise GGUFError("tensor %r is not aligned to %d bytes" % (name, self.alignment))
                if nb >= 0 and off + nb > size:
                    raise GGUFError("tensor %r runs past the end of the file" % name)
                self.tensors[name] = TensorInfo(name, shape, gt, off, nb)
        except Exception:
            self.close()
            raise

    def close(self) -> None:
        mm = getattr(self, "_mm", None)
        if mm is not None:
            try:
                mm.close()
            except BufferError:      # a view returned by data() is still alive; it keeps the map open
                pass
            self._mm = None
        if self._f is not None:
            self._f.close()
            self._f = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def data(self, name: str) -> np.ndarray:
        """The tensor's bytes as a read-only uint8 view of the mapping (no copy)."""
        t = self.tensors[name]
        if t.nbytes < 0:
            raise GGUFError("tensor %r has unsupported ggml type %d" % (name, t.ggml_type))
        return np.frombuffer(self._mm, dtype=np.uint8, count=t.nbytes, offset=t.offset)


# ---------------------------------------------------------------------------------- writer
def _w_string(out: List[bytes], s: str) -> None:
    b = s.encode("utf-8")
    out.append(struct.pack("<Q", len(b)) + b)


def _w_value(out: List[bytes], v: Any) -> None:
    if isinstance(v, bool):
        out.append(struct.pack("<I?", _BOOL, v))
    elif isinstance(v, int):
        if 0 <= v < 2 ** 32:
            out.append(struct.pack("<II", _U32, v))
        else:
            out.append(struct.pack("<Iq", _I64, v))
    elif isinstance(v, float):
        out.append(struct.pack("<If", _F32, v))
    elif isinstance(v, str):
        out.append(struct.pack("<I", _STR))
        _w_string(out, v)
    elif isinstance(v, (list, tuple)) and all(isinstance(e, str) for e in v):
        out.append(struct.pack("<IIQ", _ARR, _STR, len(v)))
        for e in v:
            _w_string(out, e)
    elif isinstance(v, (list, tuple)) and all(isinstance(e, int) and not isinstance(e, bool) for e in v):
        out.append(struct.pack("<IIQ", _ARR, _I32, len(v)))
        out.append(struct.pack("<%di" % len(v), *v))
    else:
        raise GGUFError("cannot encode metadata value %r" % (v,))


def write_gguf(path: str, tensors: Iterable[Tuple[str, int, Tuple[int, ...], np.ndarray]],
               metadata: Optional[Dict[str, Any]] = None, alignment: int = DEFAULT_ALIGNMENT) -> None:
    """Writes a GGUF v3 file.  ``tensors``: (name, ggml_type, shape in torch order, raw bytes)."""
    tensors = list(tensors)
    md = dict(metadata or {})
    md.setdefault("general.alignment", alignment)
    head: List[bytes] = [struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(md))]
    for k, v in md.items():
        _w_string(head, k)
        _w_value(head, v)
    rel = 0
    blobs = []
    for name, gt, shape, raw in tensors:
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        if raw.size != tensor_nbytes(gt, tuple(shape)):
            raise GGUFError("tensor %r: %d bytes given, %d expected" % (name, raw.size, tensor_nbytes(gt, tuple(shape))))
        _w_string(head, name)
        head.append(struct.pack("<I", len(shape)))
        head.append(struct.pack("<%dQ" % len(shape), *reversed(shape)))
        head.append(struct.pack("<IQ", gt, rel))
        blobs.append((rel, raw))
        rel = (rel + raw.size + alignment - 1) // alignment * alignment
    header = b"".join(head)
    pad = (-len(header)) % alignment
    with open(path, "wb") as f:
        f.write(header + b"\0" * pad)
        pos = 0
        for off, raw in blobs:
            f.write(b"\0" * (off - pos))
            f.write(raw.tobytes())
            pos = off + raw.size


# ------------------------------------------------------------------------- layer loading
def load_quant_linear(gguf: GGUFFile, name: str, device, bias_name: Optional[str] = None):
    """``QuantLinear`` from a block-quantized 2-D tensor of an open GGUF file: the mapped bytes are
    copied to ``device`` once, unchanged (the role of safetensors_libtorch.nim:57-107 for dense
    weights)."""
    import torch
    from .qlinear import QuantLinear
    t = gguf.tensors[name]
    if t.format is None or len(t.shape) != 2:
        raise GGUFError("tensor %r is not a block-quantized matrix this library runs (type %d, shape %s)"
                        % (name, t.ggml_type, t.shape))
    n_out, n_in = t.shape
    # the mapping is read-only and torch only reads from it during the copy
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", UserWarning)
        src = torch.frombuffer(memoryview(gguf.data(name)), dtype=torch.uint8)
    qweight = src.to(device)
    bias = None
    if bias_name is not None:
        b = gguf.tensors[bias_name]
        if b.ggml_type not in _PLAIN or b.shape != (n_out,):
            raise GGUFError("bias %r does not match %r" % (bias_name, name))
        arr = gguf.data(bias_name).view(_PLAIN[b.ggml_type][0])
        tb = torch.from_numpy(np.array(arr))
        bias = (tb.view(torch.bfloat16) if b.ggml_type == GGML_BF16 else tb).to(device)
    return QuantLinear.init(qweight, t.format, n_in, n_out, bias=bias)


def ggml_type_of(fmt: int) -> int:
    return _FORMAT_TO_GGML[fmt]


# ---------------------------------------------------------------- safetensors convention
# Packed blocks as a 1-D ``U8`` tensor named <name>.qweight, with the layer's format and
# dimensions in the file's ``__metadata__`` under "ttq.<name>" as JSON.

def safetensors_entry(name: str, fmt: int, n_out: int, n_in: int) -> Tuple[str, str]:
    """(metadata key, metadata value) describing a packed weight stored as ``<name>.qweight``."""
    return "ttq." + name, json.dumps({"format": int(fmt), "n_out": int(n_out), "n_in": int(n_in)})


def load_quant_linear_safetensors(path: str, name: str, device):
    """``QuantLinear`` from a safetensors file that follows the convention above."""
    from safetensors import safe_open
    from .qlinear import QuantLinear
    with safe_open(path, framework="pt", device="cpu") as f:
        md = f.metadata() or {}
        key = "ttq." + name
        if key not in md:
            raise GGUFError("safetensors metadata has no entry %r" % key)
        info = json.loads(md[key])
        q = f.get_tensor(name + ".qweight")
    return QuantLinear.init(q.to(device), int(info["format"]), int(info["n_in"]), int(info["n_out"]))
