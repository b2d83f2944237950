#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--replays R] [--only NAME] [--no-cpu] [--no-extra]

Headline workload (`value`): Q4_K decode GEMV, W 14336x4096, batch 1, bf16 activations, fp32
output -- weight-stream GB/s.  One step = one GEMV call.  Steps rotate through enough distinct
copies of the packed weight (> 2 x 256 MiB in total) that the Infinity Cache cannot serve the
stream.  All inputs are resident in HBM before the timed region.

Launch: K >= 200 steps are captured into one HIP graph and replayed; fewer steps are launched one
by one through the C ABI (ctypes, no Python wrapper in the loop).  A graph launch costs about one
kernel duration (7 us) per replay on this runtime whatever K is, which a 20-step region cannot
amortize; plain launches cost about 0.15 us more per step but nothing per region.  --graph and
--eager force either way; `config.launch` says which one ran.

Timing: W untimed warm-up steps, a fixed untimed conditioning phase (the same K steps repeated
for about 0.4 s, so that a short run is not timed on clocks that have not ramped yet), then R
timed passes of exactly K steps.  A timed pass is bracketed by synchronization on both sides and
by HIP events on the stream the kernels run on; two untimed passes are queued in front of the first
event, so that the K timed steps follow them back to back and the host's submission is not part of a
20-step measurement (a plain launch takes the host about as long to submit as the headline kernel runs).  `ms_per_step` is the median timed pass divided by K; minimum and maximum
are reported beside it.

The same line carries the other configurations (Q8_0 / Q6_K / EXL3 GEMV, Q4_K GEMM at
M = 64 / 512 / 2048, attention-shaped GEMVs) under "extra", a roofline object for the GEMV and one
for the GEMM, and a CPU baseline timed on this machine's host cores.

    python bench.py --only ladder     the roofline ladder of the headline kernel (see csrc/ttq_ladder.hip);
                                      --only ladder_14336x4096 runs one shape (for a kernel trace);
                                      --only ladder_q6k the stages of the Q6_K streamed GEMV;
                                      --only ladder_gemm the roles of the prefill GEMM kernel, alone and together
                                      (the ladder kernels are compiled on demand into libttq_ladder.so)
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MALL_BYTES = 256 << 20
CONDITIONING_S = 0.4
FRONT_PASSES = 2          # untimed passes of K steps queued in front of every timed pass
GRAPH_MIN_STEPS = 200     # fewer timed steps than this are launched one by one (a graph launch costs ~7 us per replay)
METRIC = "Q4_K GEMV weight GB/s (% of HBM peak); Q4_K GEMM M=512 TFLOP/s"
FMT_NAME = {0: "Q8_0", 1: "Q4_K", 2: "Q6_K", 3: "EXL3"}
# what the kernels compute in (not a precision claim)
GEMV_DTYPE = ("i8 (bf16 activations as 15-bit block fixed point in two int8 planes, 4-bit weights, "
              "int32 MFMA accumulate; fp32 scales and row sums)")
GEMM_DTYPE = "bf16 (weights dequantized in fp32 and rounded once to bf16; fp32 MFMA accumulate)"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_brand() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--replays", type=int, default=7, help="timed replays of the K-step graph (median reported)")
    ap.add_argument("--only", default=None, help="run a single configuration (name in tattletale_amd.configs), "
                                                 "or one of: ladder, ladder_<n_out>x<n_in>, ladder_q6k, ladder_gemm, "
                                                 "ladder_gemm_m<rows>, widened, q4_k_gate_up_silu_gemv, dense_reference")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--eager", action="store_true", help="always time plain launches")
    ap.add_argument("--graph", action="store_true", help="always time replays of a HIP graph of K launches")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain device copy of 256 MiB a few times and exit (reference point for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU; --gpus %d is not supported (the operator shards by "
              "output rows with no exchange; nothing here uses a second device)" % args.gpus, file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from tattletale_amd import configs as CFG
    from tattletale_amd import formats as F
    from tattletale_amd import qlinear as QL
    from tattletale_amd import quantize as Q
    from tattletale_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    TD = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": 256 << 20, "launches": 10}))
        return 0

    def to_dev(a: "np.ndarray", kind: str | None = None):
        if a.dtype == np.uint16:
            t = torch.from_numpy(a.view(np.int16)).to(dev)
            return t.view(TD[kind]) if kind in ("f16", "bf16") else t
        return torch.from_numpy(a).to(dev)

    def time_steps(step_fn, steps: int, warmup: int, use_graph: bool = True, replays: int | None = None,
                   direct_fn=None):
        """`warmup` untimed calls of step_fn(i), a graph of exactly `steps` calls (or, for few steps and
        when a `direct_fn(i)` that goes straight to the C ABI is given, plain launches), an untimed
        conditioning phase, then `replays` timed passes.  Returns a dict with the per-step times
        (milliseconds, HIP events on the launch stream): median, min, max over the passes."""
        replays = args.replays if replays is None else replays
        stream = torch.cuda.current_stream(dev)
        for i in range(warmup):
            step_fn(i)
        torch.cuda.synchronize()
        graph = None
        if args.eager or (direct_fn is not None and steps < GRAPH_MIN_STEPS and not args.graph):
            use_graph = False
            if direct_fn is not None:
                step_fn = direct_fn
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream(dev)
            side.wait_stream(stream)
            with torch.cuda.stream(side):
                step_fn(0)
                torch.cuda.synchronize()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(steps):
                        step_fn(i)
            stream.wait_stream(side)
            torch.cuda.synchronize()

        def run_once():
            if graph is not None:
                graph.replay()
            else:
                for i in range(steps):
                    step_fn(i)

        # conditioning: same launches, untimed, a fixed wall-clock budget
        run_once()
        torch.cuda.synchronize()
        t_end = time.perf_counter() + CONDITIONING_S
        n_cond = 1
        while time.perf_counter() < t_end:
            run_once()
            torch.cuda.synchronize()
            n_cond += 1
        per = []
        wall = []
        for _ in range(max(1, replays)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            # untimed passes run while the host submits the timed one, so that the K timed steps start back to
            # back with the first event instead of waiting for the submission.  Two of them: submitting a plain
            # launch through the C ABI takes about as long as the 7 us headline kernel runs, and with one pass in
            # front the stream still ran dry (7.04 us per step against 6.90 with two, four or eight)
            for _ in range(FRONT_PASSES):
                run_once()
            e0.record(stream)
            run_once()
            e1.record(stream)
            torch.cuda.synchronize()
            wall.append((time.perf_counter() - t0) * 1e3 / ((FRONT_PASSES + 1) * steps))
            per.append(e0.elapsed_time(e1) / steps)
        per.sort()
        wall.sort()
        return {"ms": per[len(per) // 2], "ms_min": per[0], "ms_max": per[-1], "wall_ms": wall[len(wall) // 2],
                "replays": len(per), "conditioning_replays": n_cond,
                "launch": ("hip-graph replay of %d launches" % steps) if graph is not None else
                          ("%d plain stream launches through the C ABI" % steps if step_fn is direct_fn else
                           "%d plain stream launches through the Python wrapper" % steps)}

    def rotated(nbytes: int) -> int:
        """Copies of a weight of nbytes to rotate through so that the Infinity Cache cannot serve it."""
        return 1 if nbytes > MALL_BYTES else min(96, max(2, -(-2 * MALL_BYTES // nbytes)))

    def run_config(name: str, steps: int, warmup: int):
        cfg = CFG.CONFIGS[name]
        t0 = time.time()
        packed = CFG.packed_weights(cfg)
        xh = CFG.activations(cfg)
        log("[%s] inputs generated in %.1f s" % (name, time.time() - t0))
        x = to_dev(xh, cfg.x_dtype)
        direct = None
        if cfg.fmt == F.EXL3:
            trellis, suh, svh = packed
            wbytes = trellis.nbytes
            ncopies = rotated(wbytes)
            tr = [to_dev(trellis) for _ in range(ncopies)]
            suh_d, svh_d = to_dev(suh, "f16"), to_dev(svh, "f16")
            y = torch.empty((cfg.m, cfg.n_out), dtype=torch.float32, device=dev)

            def step(i):
                QL.gemv_exl3(tr[i % ncopies], suh_d, svh_d, x, cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG, out=y)
        else:
            wbytes = packed.nbytes
            ncopies = rotated(wbytes)
            ws = [to_dev(packed) for _ in range(ncopies)]
            if cfg.m == 1:
                y = torch.empty((1, cfg.n_out), dtype=torch.float32, device=dev)

                def step(i):
                    QL.gemv(cfg.fmt, ws[i % ncopies], x, cfg.n_out, cfg.n_in, out=y)
                entry = getattr(_lib.lib(), {F.Q8_0: "ttq_gemv_q8_0", F.Q4_K: "ttq_gemv_q4_k",
                                             F.Q6_K: "ttq_gemv_q6_k"}[cfg.fmt])
                wp, xp, yp = [w.data_ptr() for w in ws], x.data_ptr(), y.data_ptr()
                xcode = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16}[cfg.x_dtype]
                sp = torch.cuda.current_stream(dev).cuda_stream

                def direct(i):
                    rc = entry(wp[i % ncopies], xp, xcode, yp, 1, cfg.n_out, cfg.n_in, sp)
                    if rc:
                        raise RuntimeError("%s returned %d" % (name, rc))
            else:
                y = torch.empty((cfg.m, cfg.n_out), dtype=torch.bfloat16, device=dev)

                def step(i):
                    QL.gemm_q4_k(ws[i % ncopies], x, cfg.n_out, cfg.n_in, out=y)
        t = time_steps(step, steps, warmup, direct_fn=direct)
        flops = 2.0 * cfg.m * cfg.n_out * cfg.n_in
        res = {
            "name": name, "steps": steps, "replays": t["replays"], "launch": t["launch"], "weight_bytes": int(wbytes),
            "weight_copies": ncopies,
            "ms_per_step": t["ms"], "ms_per_step_min": t["ms_min"], "ms_per_step_max": t["ms_max"],
            "wall_ms_per_step": t["wall_ms"],
            "weight_GBps": wbytes / (t["ms"] * 1e-3) / 1e9,
            "TFLOPs": flops / (t["ms"] * 1e-3) / 1e12,
        }
        if cfg.m == 1:
            res["hbm_frac"] = res["weight_GBps"] / HBM_PEAK_GBPS
        else:
            res["mfma_frac"] = res["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS
        log("[%s] %.3f us/step (min %.3f, max %.3f over %d replays)  %.0f GB/s  %.1f TFLOP/s" % (
            name, t["ms"] * 1e3, t["ms_min"] * 1e3, t["ms_max"] * 1e3, t["replays"], res["weight_GBps"],
            res["TFLOPs"]))
        del y
        torch.cuda.empty_cache()
        return res

    def random_packed(rng, fmt, n_out, n_in):
        """Random packed bytes with finite scale fields (timing only)."""
        nbytes, wpb, scale_hi = {F.Q8_0: (34, 32, [1]), F.Q4_K: (144, 256, [1, 3]), F.Q6_K: (210, 256, [209])}[fmt]
        raw = rng.integers(0, 256, (n_out * (n_in // wpb), nbytes), dtype=np.uint8)
        for off in scale_hi:
            raw[:, off] &= 0x3F            # |fp16 scale| < 2
        return raw.reshape(-1)

    def cpu_baseline():
        """The same operator on this machine's host cores, in the probes-table style of the reference
        (workspace/probes/src/reports.nim:27-46: name, calls, time per call, rate).

        kind "port": the oracle's fused packed-weight GEMV (plain C, OpenMP), all host cores and one
        thread, for the four GEMV configurations; plus ATen's dense bf16 linear on dequantized weights
        for the headline shape, which is what the reference's Linear.forward runs on a CPU."""
        import oracle
        ncores = os.cpu_count() or 1
        table = []

        def timed(label, fn, nbytes, flops, threads, budget_s):
            fn()
            n, t0 = 0, time.perf_counter()
            while True:
                fn()
                n += 1
                dt = time.perf_counter() - t0
                if dt >= budget_s:
                    break
            per = dt / n
            row = {"name": label, "threads": threads, "calls": n, "us_per_call": per * 1e6,
                   "weight_GBps": nbytes / per / 1e9, "GFLOPs": flops / per / 1e9}
            table.append(row)
            log("  %-34s %3d thr %5d calls %12.1f us/call %8.2f GB/s %8.2f GFLOP/s" % (
                label, threads, n, row["us_per_call"], row["weight_GBps"], row["GFLOPs"]))
            return row

        log("[cpu_baseline] %s, %d logical cores" % (cpu_brand(), ncores))
        head_all = head_one = None
        for name, budget in (("q4_k_gemv", 3.0), ("q8_0_gemv", 1.5), ("q6_k_gemv", 3.0)):
            cfg = CFG.CONFIGS[name]
            packed = CFG.packed_weights(cfg)
            xh = CFG.activations(cfg)
            xf = (oracle.bf16_to_f32(xh) if cfg.x_dtype == "bf16" else np.asarray(xh, np.float32))[0]
            flops = 2.0 * cfg.n_out * cfg.n_in
            for thr in (ncores, 1):
                r = timed("%s %dx%d" % (name, cfg.n_out, cfg.n_in),
                          lambda: oracle.gemv_fused(cfg.fmt, packed, xf, cfg.n_out, cfg.n_in, thr),
                          packed.nbytes, flops, thr, budget)
                if name == "q4_k_gemv":
                    if thr == ncores:
                        head_all = r
                    else:
                        head_one = r
        # EXL3: decode the trellis and multiply (the oracle has no fused form; one thread)
        cfg = CFG.CONFIGS["exl3_gemv"]
        trellis, suh, svh = CFG.packed_weights(cfg)
        xh = CFG.activations(cfg)

        def exl3_once():
            t = oracle.exl3_decode(trellis, cfg.n_out, cfg.n_in, cfg.bits, oracle.CB_MCG)
            oracle.exl3_gemv_f64(t, suh, svh, xh[0])

        timed("exl3_gemv %dx%d (decode + multiply)" % (cfg.n_out, cfg.n_in), exl3_once, trellis.nbytes,
              2.0 * cfg.n_out * cfg.n_in, 1, 2.0)
        # reference CPU path: dense linear on the dequantized weight (ATen), headline shape
        cfg = CFG.CONFIGS["q4_k_gemv"]
        packed = CFG.packed_weights(cfg)
        what = torch.from_numpy(oracle.dequant(cfg.fmt, packed, cfg.n_out, cfg.n_in)).to(torch.bfloat16)
        xb = torch.from_numpy(oracle.bf16_to_f32(CFG.activations(cfg))[0]).to(torch.bfloat16)[None, :]
        for thr in (ncores, 1):
            torch.set_num_threads(thr)
            timed("aten dense bf16 linear 14336x4096", lambda: torch.nn.functional.linear(xb, what),
                  what.numel() * 2, 2.0 * cfg.n_out * cfg.n_in, thr, 2.0)
        torch.set_num_threads(ncores)
        return {"value": head_all["weight_GBps"], "unit": "GB/s", "cores": ncores, "kind": "port",
                "sample": "%d calls of the full 14336x4096 Q4_K GEMV (the oracle's fused C restatement, OpenMP, "
                          "%d threads); the table has one thread and the other GEMV configurations"
                          % (head_all["calls"], ncores),
                "us_per_call": head_all["us_per_call"],
                "single_thread_value": head_one["weight_GBps"], "cpu": cpu_brand(), "table": table}

    def run_gate_up(steps: int, warmup: int):
        """Llama-3-8B FFN decode: the 28672 x 4096 gate/up matrix, silu_and_mul fused into the GEMV
        (one launch) against the GEMV followed by ttq_silu_and_mul (two launches)."""
        n_ff, n_in = 14336, 4096
        cfg = CFG.CONFIGS["q4_k_gemv"]
        t0 = time.time()
        w = Q.fill_normal(cfg.seed + 50, 0, 0.02, 2 * n_ff * n_in).reshape(2 * n_ff, n_in)
        packed = Q.quantize(F.Q4_K, w)
        del w
        log("[q4_k_gate_up_silu_gemv] inputs generated in %.1f s" % (time.time() - t0))
        x = to_dev(CFG.activations(cfg), "bf16")
        ncopies = rotated(packed.nbytes)
        ws = [to_dev(packed) for _ in range(ncopies)]
        y = torch.empty((1, n_ff), dtype=torch.bfloat16, device=dev)
        L = _lib.lib()

        def fused(i):
            _lib.check(L.ttq_gemv_q4_k_silu_mul(ws[i % ncopies].data_ptr(), x.data_ptr(), F.BF16, y.data_ptr(),
                                                F.BF16, 1, n_ff, n_in, torch.cuda.current_stream(dev).cuda_stream),
                       "ttq_gemv_q4_k_silu_mul")

        gu16 = torch.empty((1, 2 * n_ff), dtype=torch.bfloat16, device=dev)
        st = _lib.QLinearStruct(format=F.Q4_K, n_out=2 * n_ff, n_in=n_in)

        def unfused(i):
            cur = torch.cuda.current_stream(dev).cuda_stream
            st.qweight = ws[i % ncopies].data_ptr()
            _lib.check(L.ttq_linear_forward(C.byref(st), x.data_ptr(), F.BF16, 1, gu16.data_ptr(), F.BF16, cur),
                       "ttq_linear_forward")
            _lib.check(L.ttq_silu_and_mul(gu16.data_ptr(), y.data_ptr(), F.BF16, 1, n_ff, cur), "ttq_silu_and_mul")

        # the same with the block's add + RMSNorm in front: one launch against three
        res_in = torch.randn((1, n_in), device=dev).to(torch.bfloat16)
        gamma = torch.ones(n_in, dtype=torch.bfloat16, device=dev)
        new_res = torch.empty_like(res_in)
        normed = torch.empty_like(res_in)

        def norm_fused(i):
            cur = torch.cuda.current_stream(dev).cuda_stream
            _lib.check(L.ttq_gemv_q4_k_rmsnorm(ws[i % ncopies].data_ptr(), x.data_ptr(), res_in.data_ptr(),
                                               gamma.data_ptr(), 1e-5, F.BF16, new_res.data_ptr(), None,
                                               y.data_ptr(), F.BF16, 1, n_ff, n_in, 1, cur), "ttq_gemv_q4_k_rmsnorm")

        def norm_unfused(i):
            cur = torch.cuda.current_stream(dev).cuda_stream
            _lib.check(L.ttq_rmsnorm(x.data_ptr(), res_in.data_ptr(), gamma.data_ptr(), 1e-5, F.BF16,
                                     new_res.data_ptr(), normed.data_ptr(), 1, n_in, cur), "ttq_rmsnorm")
            st.qweight = ws[i % ncopies].data_ptr()
            _lib.check(L.ttq_linear_forward(C.byref(st), normed.data_ptr(), F.BF16, 1, gu16.data_ptr(), F.BF16, cur),
                       "ttq_linear_forward")
            _lib.check(L.ttq_silu_and_mul(gu16.data_ptr(), y.data_ptr(), F.BF16, 1, n_ff, cur), "ttq_silu_and_mul")

        f_ms = time_steps(fused, steps, warmup)["ms"]
        u_ms = time_steps(unfused, steps, warmup)["ms"]
        nf_ms = time_steps(norm_fused, steps, warmup)["ms"]
        nu_ms = time_steps(norm_unfused, steps, warmup)["ms"]
        res = {"name": "q4_k_gate_up_silu_gemv", "steps": steps, "weight_bytes": int(packed.nbytes),
               "weight_copies": ncopies, "ms_per_step": f_ms, "weight_GBps": packed.nbytes / (f_ms * 1e-3) / 1e9,
               "hbm_frac": packed.nbytes / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
               "unfused_two_launches_ms_per_step": u_ms,
               "with_add_rmsnorm_fused_ms_per_step": nf_ms, "with_add_rmsnorm_three_launches_ms_per_step": nu_ms}
        log("[q4_k_gate_up_silu_gemv] fused %.3f us/step (%.0f GB/s), GEMV + silu_and_mul %.3f us/step; "
            "with add+RMSNorm in front: one launch %.3f us/step, three launches %.3f us/step"
            % (f_ms * 1e3, res["weight_GBps"], u_ms * 1e3, nf_ms * 1e3, nu_ms * 1e3))
        # prefill, M = 2048: silu_and_mul in the GEMM epilogue against GEMM + ttq_silu_and_mul
        xm = torch.randn((2048, n_in), device=dev).mul_(0.05).to(torch.bfloat16)

        def pre_fused(i):
            QL.gemm_q4_k_silu_mul(ws[i % ncopies], xm, n_ff, n_in)

        def pre_unfused(i):
            QL.silu_and_mul(QL.gemm_q4_k(ws[i % ncopies], xm, 2 * n_ff, n_in))

        pf_ms = time_steps(pre_fused, 20, 3, replays=3)["ms"]
        pu_ms = time_steps(pre_unfused, 20, 3, replays=3)["ms"]
        res["prefill_m2048_fused_gemm_ms_per_step"] = pf_ms
        res["prefill_m2048_gemm_plus_silu_ms_per_step"] = pu_ms
        res["prefill_m2048_fused_TFLOPs"] = 2.0 * 2048 * 2 * n_ff * n_in / (pf_ms * 1e-3) / 1e12
        log("[q4_k_gate_up_silu_gemm M=2048] fused %.1f us/step (%.0f TFLOP/s), GEMM + silu_and_mul %.1f us/step"
            % (pf_ms * 1e3, res["prefill_m2048_fused_TFLOPs"], pu_ms * 1e3))
        return res

    def run_widened(steps: int, warmup: int):
        """Rows next to the headline ones, on random packed bytes with finite scale fields (timing
        only): the attention projections as decode GEMVs (q/o 4096x4096, k/v 1024x4096, reference call
        sites workspace/transformers/src/layers/attn.nim:113-116,154-156,189), the LM-head-sized Q4_K
        stream, a Q6_K down projection (mlp.nim:60), the Q6_K LM head for 1, 2 and 4 tokens (128256x4096) and for 1 and 4 (151936x1024), the few-row decode GEMV (2, 4, 8 and 16 activation rows at once), the few-row form of the
        prefill operator (32 rows), the prefill GEMM for Q6_K and Q8_0 weights and for fp16 activations, 14336 x 4096 unless
        named otherwise; the down projection at 128 and 512 rows (K split over copies of the tile grid);
        add + RMSNorm on rows of 4096."""
        n_out, n_in = 14336, 4096
        rng = np.random.default_rng(1234)
        res = {}

        def timed(name, fmt, m, fn_of, n_out=n_out, n_in=n_in, steps=steps):
            packed = random_packed(rng, fmt, n_out, n_in)
            ncopies = rotated(packed.nbytes)
            ws = [to_dev(packed) for _ in range(ncopies)]
            x = torch.randn((m, n_in), device=dev).to(torch.bfloat16)
            step = fn_of(ws, x, ncopies)
            ms = time_steps(step, steps, warmup)["ms"]
            res[name] = {"us_per_step": ms * 1e3, "weight_GBps": packed.nbytes / (ms * 1e-3) / 1e9,
                         "hbm_frac": packed.nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                         "TFLOPs": 2.0 * m * n_out * n_in / (ms * 1e-3) / 1e12}
            log("[%s] %.2f us/step  %.0f GB/s  %.1f TFLOP/s" % (name, ms * 1e3, res[name]["weight_GBps"],
                                                              res[name]["TFLOPs"]))
            del ws
            torch.cuda.empty_cache()

        for nm, (no, ni) in (("q4_k_gemv_o_4096x4096", (4096, 4096)), ("q4_k_gemv_kv_1024x4096", (1024, 4096)),
                             ("q4_k_gemv_down_4096x14336", (4096, 14336)),
                             ("q4_k_gemv_lm_head_128256x4096", (128256, 4096))):
            y = torch.empty((1, no), dtype=torch.float32, device=dev)
            timed(nm, F.Q4_K, 1,
                  lambda ws, x, nc, y=y, no=no, ni=ni: (lambda i: QL.gemv(F.Q4_K, ws[i % nc], x, no, ni, out=y)),
                  n_out=no, n_in=ni, steps=steps if no < 100000 else max(20, steps // 10))
        # Q6_K decode beside the LM head: the down projection of the layers that a "Q4_K_M" file stores as Q6_K
        y = torch.empty((1, 4096), dtype=torch.float32, device=dev)
        timed("q6_k_gemv_down_4096x14336", F.Q6_K, 1,
              lambda ws, x, nc, y=y: (lambda i: QL.gemv(F.Q6_K, ws[i % nc], x, 4096, 14336, out=y)),
              n_out=4096, n_in=14336)
        # the LM head as a "Q4_K_M" file stores it (Q6_K), for one token and for the two and four tokens of a
        # speculative step (one pass over the weights for all of them)
        for m in (1, 2, 4):
            y = torch.empty((m, 128256), dtype=torch.float32, device=dev)
            timed("q6_k_gemv_lm_head_128256x4096" + ("" if m == 1 else "_m%d" % m), F.Q6_K, m,
                  lambda ws, x, nc, y=y: (lambda i: QL.gemv(F.Q6_K, ws[i % nc], x, 128256, 4096, out=y)),
                  n_out=128256, n_in=4096, steps=max(20, steps // 10))
        # the same for a small model (hidden size 1024, vocabulary 151936): rows of 1024 values, streamed two at a time
        for m in (1, 4):
            y = torch.empty((m, 151936), dtype=torch.float32, device=dev)
            timed("q6_k_gemv_lm_head_151936x1024" + ("" if m == 1 else "_m%d" % m), F.Q6_K, m,
                  lambda ws, x, nc, y=y: (lambda i: QL.gemv(F.Q6_K, ws[i % nc], x, 151936, 1024, out=y)),
                  n_out=151936, n_in=1024, steps=max(20, steps // 4))
        # Q8_0 decode on the headline shape (every projection of a Q8_0 file is a Q8_0 stream)
        y = torch.empty((1, n_out), dtype=torch.float32, device=dev)
        timed("q8_0_gemv_14336x4096", F.Q8_0, 1,
              lambda ws, x, nc, y=y: (lambda i: QL.gemv(F.Q8_0, ws[i % nc], x, n_out, n_in, out=y)))
        for m in (2, 4, 8, 16):
            y = torch.empty((m, n_out), dtype=torch.float32, device=dev)
            timed("q4_k_gemv_m%d" % m, F.Q4_K, m,
                  lambda ws, x, nc, y=y: (lambda i: QL.gemv(F.Q4_K, ws[i % nc], x, n_out, n_in, out=y)))
        # 17..64 rows: the prefill operator's few-row kernel (weights dequantized in registers), on the
        # up/gate shape and on the down projection (few weight rows, long K)
        for nm, (no, ni) in (("q4_k_gemm_m32", (n_out, n_in)), ("q4_k_gemm_m32_down_4096x14336", (n_in, n_out))):
            y = torch.empty((32, no), dtype=torch.bfloat16, device=dev)
            timed(nm, F.Q4_K, 32,
                  lambda ws, x, nc, y=y, no=no, ni=ni: (lambda i: QL.gemm(F.Q4_K, ws[i % nc], x, no, ni, out=y)),
                  n_out=no, n_in=ni)
        for fmt, nm in ((F.Q6_K, "q6_k_gemm_m512"), (F.Q8_0, "q8_0_gemm_m512")):
            y = torch.empty((512, n_out), dtype=torch.bfloat16, device=dev)
            timed(nm, fmt, 512,
                  lambda ws, x, nc, y=y, fmt=fmt: (lambda i: QL.gemm(fmt, ws[i % nc], x, n_out, n_in, out=y)),
                  steps=max(20, steps // 4))
        # fp16 activations through the operator (ttq_linear_forward): the fp16 form of the prefill GEMM -- a packed
        # fp16 copy of the activations, weights rounded once to fp16, fp16 matrix cores
        def f16_forward(ws, x, nc):
            xh = (x.float() * 0.05).to(torch.float16)
            layers = [QL.QuantLinear.init(w, F.Q4_K, n_in, n_out) for w in ws]
            return lambda i: layers[i % nc].forward(xh)
        timed("q4_k_forward_f16_m512", F.Q4_K, 512, f16_forward, steps=max(20, steps // 4))

        # fp32 activations through the operator: the same GEMM over a copy scaled row by row and rounded to fp16
        def f32_forward(ws, x, nc):
            xf = x.float() * 0.05
            layers = [QL.QuantLinear.init(w, F.Q4_K, n_in, n_out) for w in ws]
            return lambda i: layers[i % nc].forward(xf)
        timed("q4_k_forward_f32_m512", F.Q4_K, 512, f32_forward, steps=max(20, steps // 4))
        # a few fp32 rows through the operator: the few-row kernel in fp16 over a row-major copy scaled the same way
        # (Q6_K has no decode kernel of several fp32 rows: four rows take it as well)
        timed("q4_k_forward_f32_m8", F.Q4_K, 8, f32_forward)

        def f32_forward_q6(ws, x, nc):
            xf = x.float() * 0.05
            layers = [QL.QuantLinear.init(w, F.Q6_K, n_in, n_out) for w in ws]
            return lambda i: layers[i % nc].forward(xf)
        timed("q6_k_forward_f32_m4", F.Q6_K, 4, f32_forward_q6)
        # trellis weights, 4096 x 4096 at 3 bits: 8 rows through the decode kernel (one decode of the weights
        # for all 8), 512 rows through the prefill path, and the Q4_K GEMM at the same shape beside it
        ecfg = CFG.CONFIGS["exl3_gemv"]
        etr, esuh, esvh = CFG.packed_weights(ecfg)
        enc = rotated(etr.nbytes)
        etrs = [to_dev(etr) for _ in range(enc)]
        esu, esv = to_dev(esuh, "f16"), to_dev(esvh, "f16")
        for m in (8, 512):
            xe = torch.randn((m, ecfg.n_in), device=dev).to(torch.float16)
            if m == 8:
                ye = torch.empty((m, ecfg.n_out), dtype=torch.float32, device=dev)

                def estep(i, xe=xe, ye=ye):
                    QL.gemv_exl3(etrs[i % enc], esu, esv, xe, ecfg.n_out, ecfg.n_in, ecfg.bits, F.CB_MCG, out=ye)
            else:
                def estep(i, xe=xe):
                    QL.gemm_exl3(etrs[i % enc], esu, esv, xe, ecfg.n_out, ecfg.n_in, ecfg.bits, F.CB_MCG)
            ms = time_steps(estep, steps if m == 8 else max(20, steps // 4), warmup)["ms"]
            nm = "exl3_gemv_m8_4096x4096" if m == 8 else "exl3_prefill_m512_4096x4096"
            res[nm] = {"us_per_step": ms * 1e3, "weight_GBps": etr.nbytes / (ms * 1e-3) / 1e9,
                       "TFLOPs": 2.0 * m * ecfg.n_out * ecfg.n_in / (ms * 1e-3) / 1e12}
            log("[%s] %.2f us/step  %.1f TFLOP/s" % (nm, ms * 1e3, res[nm]["TFLOPs"]))
        del etrs
        torch.cuda.empty_cache()
        y = torch.empty((512, 4096), dtype=torch.bfloat16, device=dev)
        timed("q4_k_gemm_m512_4096x4096", F.Q4_K, 512,
              lambda ws, x, nc, y=y: (lambda i: QL.gemm(F.Q4_K, ws[i % nc], x, 4096, 4096, out=y)),
              n_out=4096, n_in=4096, steps=max(20, steps // 4))
        # the fused gate||up weight as a plain GEMM at 2048 rows: eight full rounds of 256 x 112 tiles
        y = torch.empty((2048, 2 * n_out), dtype=torch.bfloat16, device=dev)
        timed("q4_k_gemm_m2048_gate_up_28672x4096", F.Q4_K, 2048,
              lambda ws, x, nc, y=y: (lambda i: QL.gemm(F.Q4_K, ws[i % nc], x, 2 * n_out, n_in, out=y)),
              n_out=2 * n_out, n_in=n_in, steps=max(10, steps // 10))
        del y
        torch.cuda.empty_cache()
        # the down projection of a prefill chunk: few output tiles, long K -- the launches that split K
        for m in (128, 512):
            y = torch.empty((m, 4096), dtype=torch.bfloat16, device=dev)
            timed("q4_k_gemm_m%d_down_4096x14336" % m, F.Q4_K, m,
                  lambda ws, x, nc, y=y: (lambda i: QL.gemm(F.Q4_K, ws[i % nc], x, 4096, 14336, out=y)),
                  n_out=4096, n_in=14336, steps=max(20, steps // 4))
        # add + RMSNorm alone (ttq_rmsnorm with a residual): one decode row and a prefill block.
        # Algorithmic bytes: x and residual read, new residual and normalized row written.
        L = _lib.lib()
        gamma = torch.ones(n_in, dtype=torch.bfloat16, device=dev)
        for m in (1, 2048):
            nbuf = max(2, -(-2 * MALL_BYTES // (4 * m * n_in * 2))) if m > 1 else 2
            xs = [torch.randn((m, n_in), device=dev).to(torch.bfloat16) for _ in range(nbuf)]
            rs = [torch.randn((m, n_in), device=dev).to(torch.bfloat16) for _ in range(nbuf)]
            new_res, normed = torch.empty_like(xs[0]), torch.empty_like(xs[0])

            def norm_step(i, m=m, xs=xs, rs=rs, new_res=new_res, normed=normed, nbuf=nbuf):
                _lib.check(L.ttq_rmsnorm(xs[i % nbuf].data_ptr(), rs[i % nbuf].data_ptr(), gamma.data_ptr(), 1e-5,
                                         F.BF16, new_res.data_ptr(), normed.data_ptr(), m, n_in,
                                         torch.cuda.current_stream(dev).cuda_stream), "ttq_rmsnorm")

            ms = time_steps(norm_step, steps, warmup)["ms"]
            nm = "add_rmsnorm_m%d" % m
            res[nm] = {"us_per_step": ms * 1e3, "GBps": 4.0 * m * n_in * 2 / (ms * 1e-3) / 1e9}
            log("[%s] %.2f us/step  %.0f GB/s" % (nm, ms * 1e3, res[nm]["GBps"]))
            del xs, rs
            torch.cuda.empty_cache()
        return res

    def run_dense_reference(steps: int, warmup: int):
        """Context, not the product: the vendor library's plain bf16 linear (torch -> hipBLASLt) on
        dense 14336 x 4096 weights, i.e. what the reference's Linear.forward would run on this GPU
        after dequantizing once.  Same timing method, weight copies rotated past the cache."""
        n_out, n_in = 14336, 4096
        ncopies = rotated(n_out * n_in * 2)
        ws = [torch.randn((n_out, n_in), device=dev).mul_(0.02).to(torch.bfloat16) for _ in range(ncopies)]
        res = {}
        for m in (1, 64, 512, 2048):
            x = torch.randn((m, n_in), device=dev).to(torch.bfloat16)
            y = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
            n = max(10, steps // (1 if m <= 64 else 4))
            ms = time_steps(lambda i: torch.matmul(x, ws[i % ncopies].t(), out=y), n, warmup)["ms"]
            res["m%d" % m] = {"us_per_step": ms * 1e3, "TFLOPs": 2.0 * m * n_out * n_in / (ms * 1e-3) / 1e12,
                              "weight_GBps": n_out * n_in * 2 / (ms * 1e-3) / 1e9}
            log("[dense_bf16_library m=%d] %.2f us/step  %.1f TFLOP/s  %.0f GB/s of bf16 weights" % (
                m, ms * 1e3, res["m%d" % m]["TFLOPs"], res["m%d" % m]["weight_GBps"]))
        del ws
        torch.cuda.empty_cache()
        return res

    def ladder_lib():
        """libttq_ladder.so, compiled on demand (measurement-only kernels, not part of the product build)."""
        from tattletale_amd import build as B
        return C.CDLL(B.build_ladder())

    def run_ladder(steps: int, warmup: int, shapes=((14336, 4096), (128256, 4096))):
        """What each stage of the headline kernel costs on its own (tattletale_amd/csrc/ttq_ladder.hip):
        empty launch, the kernel's requests alone, + the y store, the kernel without arithmetic, the
        kernel; at the headline shape and on a 295 MB Q4_K matrix (128256 x 4096)."""
        LAD = ladder_lib()
        LAD.ttq_ladder_launch.restype = C.c_int
        LAD.ttq_ladder_launch.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        L = _lib.lib()
        rng = np.random.default_rng(99)
        names = ["0 empty launch (grid, workgroup and LDS of the GEMV)", "1 requests only (HBM -> LDS, all at once)",
                 "2 requests + y store", "3 GEMV without arithmetic", "4 GEMV (ttq_gemv_q4_k)"]
        out = {}
        for n_out, n_in in shapes:
            st = steps if n_out < 100000 else max(20, steps // 10)
            packed = random_packed(rng, F.Q4_K, n_out, n_in)
            ncopies = rotated(packed.nbytes)
            ws = [to_dev(packed) for _ in range(ncopies)]
            x = torch.randn((1, n_in), device=dev).to(torch.bfloat16)
            y = torch.empty((1, n_out), dtype=torch.float32, device=dev)
            rows = []
            for rung in range(5):
                if rung < 4:
                    def step(i, rung=rung):
                        rc = LAD.ttq_ladder_launch(rung, ws[i % ncopies].data_ptr(), x.data_ptr(), y.data_ptr(), n_out,
                                                   n_in, torch.cuda.current_stream(dev).cuda_stream)
                        if rc != 0:
                            raise RuntimeError("ttq_ladder_launch(%d) returned %d" % (rung, rc))
                else:
                    def step(i):
                        _lib.check(L.ttq_gemv_q4_k(ws[i % ncopies].data_ptr(), x.data_ptr(), F.BF16, y.data_ptr(), 1,
                                                   n_out, n_in, torch.cuda.current_stream(dev).cuda_stream),
                                   "ttq_gemv_q4_k")
                t = time_steps(step, st, warmup)
                gbps = packed.nbytes / (t["ms"] * 1e-3) / 1e9
                rows.append({"rung": names[rung], "us_per_launch": t["ms"] * 1e3, "us_min": t["ms_min"] * 1e3,
                             "us_max": t["ms_max"] * 1e3, "weight_GBps": gbps if rung else None,
                             "hbm_frac": gbps / HBM_PEAK_GBPS if rung else None})
                log("[ladder %dx%d] %-58s %8.3f us  %s" % (n_out, n_in, names[rung], t["ms"] * 1e3,
                                                          ("%.0f GB/s (%.3f of peak)" % (gbps, gbps / HBM_PEAK_GBPS))
                                                          if rung else ""))
            out["%dx%d" % (n_out, n_in)] = {"weight_bytes": int(packed.nbytes), "weight_copies": ncopies,
                                           "steps": st, "rungs": rows}
            del ws
            torch.cuda.empty_cache()
        return out

    def run_ladder_q6k(steps: int, warmup: int, shapes=((128256, 4096), (4096, 14336))):
        """The stages of the Q6_K streamed GEMV (tattletale_amd/csrc/ttq_gemv_q6k_stream.h): its requests, waits and
        barriers alone; with the operand reads from LDS; the GEMV -- on the LM-head shape (two workgroups per
        compute unit) and on a down projection (one workgroup, three buffers)."""
        LAD = ladder_lib()
        LAD.ttq_ladder_q6k_launch.restype = C.c_int
        LAD.ttq_ladder_q6k_launch.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        L = _lib.lib()
        rng = np.random.default_rng(98)
        names = {2: "requests, waits and barriers", 1: "+ operand reads from LDS", 0: "GEMV (ttq_gemv_q6_k)"}
        out = {}
        for n_out, n_in in shapes:
            st = steps if n_out < 100000 else max(20, steps // 4)
            packed = random_packed(rng, F.Q6_K, n_out, n_in)
            ncopies = rotated(packed.nbytes)
            ws = [to_dev(packed) for _ in range(ncopies)]
            x = torch.randn((1, n_in), device=dev).to(torch.bfloat16)
            y = torch.empty((1, n_out), dtype=torch.float32, device=dev)
            rows = []
            for stage in (2, 1, 0):
                if stage:
                    def step(i, stage=stage):
                        rc = LAD.ttq_ladder_q6k_launch(stage, ws[i % ncopies].data_ptr(), x.data_ptr(), y.data_ptr(), n_out,
                                                       n_in, torch.cuda.current_stream(dev).cuda_stream)
                        if rc != 0:
                            raise RuntimeError("ttq_ladder_q6k_launch(%d) returned %d" % (stage, rc))
                else:
                    def step(i):
                        _lib.check(L.ttq_gemv_q6_k(ws[i % ncopies].data_ptr(), x.data_ptr(), F.BF16, y.data_ptr(), 1,
                                                   n_out, n_in, torch.cuda.current_stream(dev).cuda_stream),
                                   "ttq_gemv_q6_k")
                t = time_steps(step, st, warmup)
                gbps = packed.nbytes / (t["ms"] * 1e-3) / 1e9
                rows.append({"stage": names[stage], "us_per_launch": t["ms"] * 1e3, "us_min": t["ms_min"] * 1e3,
                             "us_max": t["ms_max"] * 1e3, "weight_GBps": gbps, "hbm_frac": gbps / HBM_PEAK_GBPS})
                log("[q6k stages %dx%d] %-32s %8.3f us  %.0f GB/s (%.3f of peak)"
                    % (n_out, n_in, names[stage], t["ms"] * 1e3, gbps, gbps / HBM_PEAK_GBPS))
            out["%dx%d" % (n_out, n_in)] = {"weight_bytes": int(packed.nbytes), "weight_copies": ncopies,
                                           "steps": st, "stages": rows}
            del ws
            torch.cuda.empty_cache()
        return out

    def run_ladder_gemm(steps: int, warmup: int, ms_=(512, 2048), n_out=14336, n_in=4096):
        """What each role of the prefill GEMM kernel costs alone and together
        (tattletale_amd/csrc/ttq_ladder_gemm.hip), 256 x 112 tiles, Q4_K 14336 x 4096."""
        LAD = ladder_lib()
        LAD.ttq_ladder_gemm_launch.restype = C.c_int
        LAD.ttq_ladder_gemm_launch.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                               C.c_int64, C.c_int64, C.c_void_p]
        rng = np.random.default_rng(97)
        # (kernel, ABL, what runs); kernel 0 = X straight into the consumers' registers, 1 = X staged through LDS
        rungs = [(0, 31, "packed X: barriers, prologue, epilogue only"),
                 (0, 4124, "packed X: consumers alone (A requests, B reads, MFMA; real values in the W tile)"),
                 (0, 4104, "packed X: + W loads and LDS stores, no dequantization"),
                 (0, 0, "packed X: whole kernel"),
                 (0, 3, "packed X: W producers alone"),
                 (0, 2, "packed X: consumers without A requests + W producers"),
                 (0, 1024, "packed X: whole kernel without barriers (roles free-running)"),
                 (2, 0, "packed X: whole kernel as a persistent workgroup per CU, LDS counters for barriers"),
                 (-1, 0, "packed X: the packing pass alone"),
                 (-2, 0, "for scale: the vendor library's dense bf16 GEMM (torch F.linear), random bf16 W, same x"),
                 (-3, 0, "for scale: the same with W = 0 and x = 0 (the matrix cores clock higher on zeros)"),
                 (1, 31, "LDS-staged X: barriers, prologue, epilogue only"),
                 (1, 4126, "LDS-staged X: consumers alone (real values in LDS)"),
                 (1, 4124, "LDS-staged X: consumers + X movers"),
                 (1, 0, "LDS-staged X: whole kernel"),
                 (1, 29, "LDS-staged X: X movers alone"),
                 (1, 1024, "LDS-staged X: whole kernel without barriers"),
                 (1, 2048, "LDS-staged X by global_load_lds: whole kernel")]
        LAD.ttq_ladder_gemm_pack.restype = C.c_int
        LAD.ttq_ladder_gemm_pack.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        packed = random_packed(rng, F.Q4_K, n_out, n_in)
        ncopies = rotated(packed.nbytes)
        ws = [to_dev(packed) for _ in range(ncopies)]
        w_dense = [torch.randn((n_out, n_in), device=dev).mul_(0.02).to(torch.bfloat16)
                   for _ in range(rotated(n_out * n_in * 2))]
        w_zero = torch.zeros((n_out, n_in), dtype=torch.bfloat16, device=dev)
        out = {}
        for m in ms_:
            x = torch.randn((m, n_in), device=dev).to(torch.bfloat16)
            x_zero = torch.zeros_like(x)
            y = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
            flop = 2.0 * m * n_out * n_in
            rows = []
            xp = torch.empty(((m + 15) // 16 * 16, n_in), dtype=torch.bfloat16, device=dev)
            if LAD.ttq_ladder_gemm_pack(x.data_ptr(), xp.data_ptr(), m, n_in, torch.cuda.current_stream(dev).cuda_stream):
                raise RuntimeError("ttq_ladder_gemm_pack failed")
            for kern, abl, what in rungs:
                def step(i, kern=kern, abl=abl):
                    sh = torch.cuda.current_stream(dev).cuda_stream
                    if kern == -2:
                        torch.matmul(x, w_dense[i % len(w_dense)].t(), out=y)
                        rc = 0
                    elif kern == -3:
                        torch.matmul(x_zero, w_zero.t(), out=y)
                        rc = 0
                    elif kern < 0:
                        rc = LAD.ttq_ladder_gemm_pack(x.data_ptr(), xp.data_ptr(), m, n_in, sh)
                    else:
                        rc = LAD.ttq_ladder_gemm_launch(kern, abl, ws[i % ncopies].data_ptr(),
                                                        (x if kern == 1 else xp).data_ptr(), y.data_ptr(), m, n_out, n_in, sh)
                    if rc != 0:
                        raise RuntimeError("ttq_ladder_gemm_launch(%d, %d) returned %d" % (kern, abl, rc))
                t = time_steps(step, max(20, steps // (10 if m <= 512 else 40)), max(3, warmup // 10))
                rows.append({"kernel": kern, "abl": abl, "rung": what, "us_per_launch": t["ms"] * 1e3,
                             "us_min": t["ms_min"] * 1e3, "us_max": t["ms_max"] * 1e3,
                             "mfma_frac_if_full_flops": flop / (t["ms"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS})
                log("[ladder gemm m=%d] k%d abl %-5d %-72s %8.2f us" % (m, kern, abl, what, t["ms"] * 1e3))
            # the persistent kernel is measured only: check here that it still computes what the product kernel does
            sh = torch.cuda.current_stream(dev).cuda_stream
            y2 = torch.empty_like(y)
            rc0 = LAD.ttq_ladder_gemm_launch(0, 0, ws[0].data_ptr(), xp.data_ptr(), y.data_ptr(), m, n_out, n_in, sh)
            rc2 = LAD.ttq_ladder_gemm_launch(2, 0, ws[0].data_ptr(), xp.data_ptr(), y2.data_ptr(), m, n_out, n_in, sh)
            torch.cuda.synchronize(dev)
            same = rc0 == 0 and rc2 == 0 and bool(torch.equal(y, y2))
            log("[ladder gemm m=%d] persistent kernel output identical to the product kernel's: %s" % (m, same))
            out["m%d" % m] = {"n_out": n_out, "n_in": n_in, "flop": flop, "rungs": rows,
                              "persistent_kernel_matches_product_kernel": same}
        del ws, w_dense, w_zero
        torch.cuda.empty_cache()
        return out

    if args.only == "ladder_gemm":
        print(json.dumps(run_ladder_gemm(args.steps, args.warmup)), flush=True)
        return 0
    if args.only and args.only.startswith("ladder_gemm_m"):      # one row count (for a kernel trace)
        print(json.dumps(run_ladder_gemm(args.steps, args.warmup, ms_=(int(args.only[len("ladder_gemm_m"):]),))), flush=True)
        return 0
    if args.only == "ladder_q6k":
        print(json.dumps(run_ladder_q6k(args.steps, args.warmup)), flush=True)
        return 0
    if args.only == "ladder":
        print(json.dumps(run_ladder(args.steps, args.warmup)), flush=True)
        return 0
    if args.only and args.only.startswith("ladder_"):      # one shape, e.g. ladder_14336x4096 (for a kernel trace)
        no, ni = (int(v) for v in args.only[len("ladder_"):].split("x"))
        print(json.dumps(run_ladder(args.steps, args.warmup, shapes=((no, ni),))), flush=True)
        return 0
    if args.only == "dense_reference":
        print(json.dumps(run_dense_reference(max(20, args.steps // 10), max(3, args.warmup // 10))), flush=True)
        return 0
    if args.only == "widened":
        print(json.dumps(run_widened(max(GRAPH_MIN_STEPS, args.steps // 4), max(3, args.warmup // 4))), flush=True)
        return 0
    if args.only == "q4_k_gate_up_silu_gemv":
        print(json.dumps(run_gate_up(max(GRAPH_MIN_STEPS, args.steps // 4), max(3, args.warmup // 4))), flush=True)
        return 0
    names = [args.only] if args.only else ["q4_k_gemv"]
    if not args.only and not args.no_extra:
        names += ["q4_k_gemm_m512", "q8_0_gemv", "q6_k_gemv", "exl3_gemv", "q4_k_gemm_m64", "q4_k_gemm_m2048"]
    results = {}
    for nme in names:
        cfg = CFG.CONFIGS[nme]
        steps = args.steps
        if nme != names[0]:
            # the other rows: fewer launches for longer kernels (the headline keeps K as passed)
            if cfg.m > 1 or nme == "q6_k_gemv":
                steps = max(20, args.steps // 10)
            else:
                steps = max(GRAPH_MIN_STEPS, args.steps)     # microsecond kernels: enough to amortize the graph launch
            if cfg.m >= 2048:
                steps = max(10, args.steps // 40)
        results[nme] = run_config(nme, steps, max(3, args.warmup * steps // max(1, args.steps)) if nme != names[0]
                                  else args.warmup)
    head = results[names[0]]
    hc = CFG.CONFIGS[names[0]]

    line = {
        "metric": METRIC,
        "value": head["weight_GBps"] if hc.m == 1 else head["TFLOPs"],
        "unit": "GB/s" if hc.m == 1 else "TFLOP/s",
        "n_gpus": 1, "steps": head["steps"], "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "ms_per_step_min": head["ms_per_step_min"], "ms_per_step_max": head["ms_per_step_max"],
        "replays": head["replays"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": GEMV_DTYPE if hc.m == 1 else GEMM_DTYPE, "data": "synthetic",
        "config": {"workload": "%s: W %dx%d %s, x %dx%d %s, y %s" % (
            hc.name, hc.n_out, hc.n_in, FMT_NAME[hc.fmt], hc.m, hc.n_in, hc.x_dtype, hc.y_dtype),
            "launch": head["launch"],
            "timing": "median of %d timed passes of K steps; each is bracketed by synchronization and by "
                      "HIP events on the launch stream, with two untimed passes queued in front of the first event"
                      % head["replays"],
            "conditioning": "%.1f s of untimed passes of the same K steps before the timed ones" % CONDITIONING_S,
            "weight_copies_rotated": head["weight_copies"]},
    }
    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (committed summary)
    traffic = {}
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            traffic = json.load(f)
    except (OSError, ValueError):
        pass

    def traffic_of(name):
        t = traffic.get(name)
        return t["hbm_read_bytes"] + t["hbm_write_bytes"] if t else None

    def gemv_roofline(r, name):
        return {"bound": "hbm", "kernel": name, "achieved": r["weight_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": r["weight_GBps"] / HBM_PEAK_GBPS, "traffic": traffic_of(name),
                "algorithmic_bytes": r["weight_bytes"]}

    def gemm_roofline(r, name):
        c = CFG.CONFIGS[name]
        return {"bound": "mfma", "kernel": name, "achieved": r["TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": r["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic_of(name),
                "algorithmic_flops": 2.0 * c.m * c.n_out * c.n_in, "dtype": GEMM_DTYPE}

    line["roofline"] = gemv_roofline(head, hc.name) if hc.m == 1 else gemm_roofline(head, hc.name)
    if "q4_k_gemm_m512" in results and names[0] != "q4_k_gemm_m512":
        g = results["q4_k_gemm_m512"]
        line["roofline_gemm"] = gemm_roofline(g, "q4_k_gemm_m512")
        line["gemm_m512_TFLOPs"] = g["TFLOPs"]
        line["gemm_m512_mfma_frac"] = g["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    line["extra"] = {k: v for k, v in results.items() if k != names[0]}
    if not args.only and not args.no_extra:
        line["extra"]["q4_k_gate_up_silu_gemv"] = run_gate_up(max(GRAPH_MIN_STEPS, args.steps // 4), max(3, args.warmup // 4))
        line["extra"]["widened"] = run_widened(max(GRAPH_MIN_STEPS, args.steps // 4), max(3, args.warmup // 4))
        line["extra"]["dense_bf16_library_14336x4096"] = run_dense_reference(max(20, args.steps // 10),
                                                                             max(3, args.warmup // 10))
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
