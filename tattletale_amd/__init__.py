"""Quantized-weight linear layer for AMD MI355X (gfx950): hand-written HIP kernels behind a
C ABI (``include/ttq.h`` -> ``libttq_hip.so``), with a thin host-side mirror of the
reference's ``Linear`` operator.

    from tattletale_amd import QuantLinear, quantize, formats
"""
import importlib

from . import _lib as formats  # format / dtype / status codes
from ._lib import TtqError, TtqLibraryError, lib

__all__ = ["formats", "TtqError", "TtqLibraryError", "lib", "QuantLinear", "QuantGatedMLP", "quantize", "qlinear", "gguf"]


def __getattr__(name):
    # torch is only needed by the device-facing half; keep `import tattletale_amd` light
    if name in ("quantize", "qlinear", "gguf"):
        return importlib.import_module("." + name, __name__)
    if name in ("QuantLinear", "QuantGatedMLP"):
        return getattr(importlib.import_module(".qlinear", __name__), name)
    raise AttributeError(name)
