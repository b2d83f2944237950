"""Builds ``libttq_hip.so`` (gfx950 only) with hipcc.  ``python -m tattletale_amd.build``.

hipcc cross-compiles without a GPU, so this runs on any host with ROCm installed.  The
library is written in-tree, next to this file.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libttq_hip.so")
LADDER_LIB = os.path.join(HERE, "libttq_ladder.so")      # bench.py's measurement ladders, built on demand

SOURCES = [
    "ttq_api.hip",
    "ttq_dequant.hip",
    "ttq_gemv.hip",
    "ttq_gemv_dot2.hip",
    "ttq_gemv_mfma.hip",
    "ttq_gemv_q4k_stream.hip",
    "ttq_gemv_q4k_slice.hip",
    "ttq_gemv_q4k_stream4.hip",
    "ttq_gemv_q6k_stream.hip",
    "ttq_gemv_q6k_stream4.hip",
    "ttq_gemv_q8_stream.hip",
    "ttq_gemv_q8_mfma.hip",
    "ttq_gemv_q8_win.hip",
    "ttq_gemv_q4k_batch.hip",
    "ttq_gemv_q4k_batch4.hip",
    "ttq_gemm_q4k.hip",
    "ttq_gemm_pc.hip",
    "ttq_gemm_pcd.hip",
    "ttq_gemm_skinny.hip",
    "ttq_exl3.hip",
    "ttq_exl3_mfma.hip",
    "ttq_exl3_prefill.hip",
    "ttq_gemm_exl3_pc.hip",
    "ttq_activations.hip",
    "ttq_workspace.hip",
    "ttq_host.cpp",
]

# -ffp-contract=off: float expressions round per operation, as the canonical dequantizer
# does; fused multiply-adds are written explicitly in the kernels.
# packed-fp32-ops is switched off so the compiler never forms v_pk_*_f32 instructions.
COMMON = ["-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-fvisibility=hidden",
          "-Wall", "-Wno-unused-function"]
# kernarg-preload-count: the first 16 dwords of a kernel's arguments arrive in scalar registers with the wavefront
# instead of through a scalar load at its start (the headline GEMV launch is 0.06 us shorter; firmware that does not
# preload runs the compiler's fallback prologue, which loads them as before).
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build libttq_hip.so")
    return exe


# Kernels whose consumers request registers asynchronously (inline-asm buffer loads that the compiler takes for
# complete): a register the compiler spills is stored before its data has landed, so these must not spill at all.
# The build reads the compiler's own resource report for them and fails otherwise.
NO_SPILL_KERNELS = {
    "ttq_gemm_pcd.hip": ("gemm_pcd_kernel",),
    "ttq_gemm_exl3_pc.hip": ("gemm_exl3_pc_kernel",),
}


def spilling_kernels(report: str, names) -> list:
    """Kernels named in `names` for which a -Rpass-analysis=kernel-resource-usage report shows vector register
    spills, as (mangled name, spilled registers) pairs."""
    bad, current = [], None
    for line in report.splitlines():
        if "Function Name:" in line:
            current = line.split("Function Name:")[1].split()[0]
        elif "VGPRs Spill:" in line and current is not None:
            n = int(line.split("VGPRs Spill:")[1].split()[0])
            if n > 0 and any(k in current for k in names):
                bad.append((current, n))
    return bad


def _compile(src: str, obj: str) -> None:
    cmd = [hipcc()] + COMMON
    if src.endswith(".hip"):
        cmd += DEVICE
    watched = NO_SPILL_KERNELS.get(os.path.basename(src))
    if watched:
        cmd += ["-Rpass-analysis=kernel-resource-usage"]
    cmd += ["-DTTQ_BUILD", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    if watched:
        bad = spilling_kernels(r.stderr, watched)
        if bad:
            raise RuntimeError("%s: kernels with asynchronously loaded registers must not spill: %s"
                               % (os.path.basename(src), ", ".join("%s (%d)" % b for b in bad)))


def build_library(force: bool = True, verbose: bool = False) -> str:
    """Compile every source and link the shared library.  Returns its path."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    deps = srcs + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".h")]
    deps.append(os.path.join(HERE, "..", "include", "ttq.h"))
    if not force and os.path.exists(LIB):
        newest = max(os.path.getmtime(d) for d in deps)
        if os.path.getmtime(LIB) >= newest:
            return LIB
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.basename(s) + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(lambda so: _compile(*so), zip(srcs, objs)))
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LIB)
    return LIB


LADDER_SOURCES = ["ttq_ladder.hip", "ttq_ladder_gemm.hip"]


def build_ladder(force: bool = False, verbose: bool = False) -> str:
    """Compile the measurement-only ladder kernels (bench.py --only ladder*) into ``libttq_ladder.so``.
    Not part of the product library and not built by ``build_library``."""
    srcs = [os.path.join(CSRC, s) for s in LADDER_SOURCES]
    deps = srcs + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".h")]
    if not force and os.path.exists(LADDER_LIB) and os.path.getmtime(LADDER_LIB) >= max(os.path.getmtime(d) for d in deps):
        return LADDER_LIB
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.basename(s) + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=len(srcs)) as ex:
        list(ex.map(lambda so: _compile(*so), zip(srcs, objs)))
    r = subprocess.run([hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LADDER_LIB] + objs,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LADDER_LIB)
    return LADDER_LIB


if __name__ == "__main__":
    if "--ladder" in sys.argv:
        build_ladder(force=True, verbose=True)
        sys.exit(0)
    build_library(force="--if-stale" not in sys.argv, verbose=True)
