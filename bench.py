#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME] [--no-cpu] [--no-extra]

Headline workload (`value`): Q4_K decode GEMV, W 14336x4096, batch 1, bf16 activations, fp32
output -- weight-stream GB/s.  One step = one GEMV call.  Steps rotate through enough distinct
copies of the packed weight (> 256 MiB in total) that the Infinity Cache cannot serve the
stream, and are replayed from a HIP graph so that host launch cost does not starve a kernel
that runs for a few microseconds.  All inputs are resident in HBM before the timed region.

The same line carries the other configurations (Q8_0 / Q6_K / EXL3 GEMV, Q4_K GEMM at
M = 64 / 512 / 2048) under "extra", the roofline of the dominant kernel and a CPU baseline
timed on this machine's host cores.
"""
from __future__ import annotations

import argparse
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
METRIC = "Q4_K GEMV weight GB/s (% of HBM peak); Q4_K GEMM M=512 TFLOP/s"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--only", default=None, help="run a single configuration (name in tattletale_amd.configs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--eager", action="store_true", help="time plain launches instead of a HIP graph")
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

    def time_steps(step_fn, steps: int, warmup: int, use_graph: bool):
        """Runs `warmup` untimed and exactly `steps` timed calls of step_fn(i).
        Returns (wall ms per step, HIP-event ms per step)."""
        stream = torch.cuda.current_stream(dev)
        for i in range(warmup):
            step_fn(i)
        torch.cuda.synchronize()
        graph = None
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
            graph.replay()            # untimed replay: uploads the graph
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                step_fn(i)
        e1.record(stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps

    def run_config(name: str, steps: int, warmup: int):
        cfg = CFG.CONFIGS[name]
        t0 = time.time()
        packed = CFG.packed_weights(cfg)
        xh = CFG.activations(cfg)
        log("[%s] inputs generated in %.1f s" % (name, time.time() - t0))
        x = to_dev(xh, cfg.x_dtype)
        if cfg.fmt == F.EXL3:
            trellis, suh, svh = packed
            wbytes = trellis.nbytes
            ncopies = max(2, -(-2 * MALL_BYTES // wbytes))
            ncopies = min(ncopies, 96)
            tr = [to_dev(trellis) for _ in range(ncopies)]
            suh_d, svh_d = to_dev(suh, "f16"), to_dev(svh, "f16")
            y = torch.empty((cfg.m, cfg.n_out), dtype=torch.float32, device=dev)

            def step(i):
                QL.gemv_exl3(tr[i % ncopies], suh_d, svh_d, x, cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG, out=y)
        else:
            wbytes = packed.nbytes
            ncopies = 1 if wbytes > MALL_BYTES else max(2, -(-2 * MALL_BYTES // wbytes))
            ws = [to_dev(packed) for _ in range(ncopies)]
            if cfg.m == 1:
                y = torch.empty((1, cfg.n_out), dtype=torch.float32, device=dev)

                def step(i):
                    QL.gemv(cfg.fmt, ws[i % ncopies], x, cfg.n_out, cfg.n_in, out=y)
            else:
                y = torch.empty((cfg.m, cfg.n_out), dtype=torch.bfloat16, device=dev)

                def step(i):
                    QL.gemm_q4_k(ws[i % ncopies], x, cfg.n_out, cfg.n_in, out=y)
        wall_ms, ev_ms = time_steps(step, steps, warmup, use_graph=not args.eager)
        flops = 2.0 * cfg.m * cfg.n_out * cfg.n_in
        res = {
            "name": name, "steps": steps, "weight_bytes": int(wbytes), "weight_copies": ncopies,
            "ms_per_step": ev_ms, "wall_ms_per_step": wall_ms,
            "weight_GBps": wbytes / (ev_ms * 1e-3) / 1e9,
            "TFLOPs": flops / (ev_ms * 1e-3) / 1e12,
        }
        if cfg.m == 1:
            res["hbm_frac"] = res["weight_GBps"] / HBM_PEAK_GBPS
        else:
            res["mfma_frac"] = res["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS
        log("[%s] %.3f us/step  %.0f GB/s  %.1f TFLOP/s" % (name, ev_ms * 1e3, res["weight_GBps"], res["TFLOPs"]))
        del y
        torch.cuda.empty_cache()
        return res

    def cpu_baseline():
        """The oracle's fused packed-weight GEMV (a port of the same op to plain C) on the host
        cores, plus ATen's dense linear on dequantized weights (what the reference runs on CPU)."""
        import oracle
        cfg = CFG.CONFIGS["q4_k_gemv"]
        packed = CFG.packed_weights(cfg)
        xf = oracle.bf16_to_f32(CFG.activations(cfg))[0]
        threads = min(os.cpu_count() or 1, 16)
        oracle.gemv_fused(cfg.fmt, packed, xf, cfg.n_out, cfg.n_in, threads)
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 8.0:
            oracle.gemv_fused(cfg.fmt, packed, xf, cfg.n_out, cfg.n_in, threads)
            n += 1
        dt = (time.perf_counter() - t0) / n
        out = {"value": packed.nbytes / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "%d calls of the full 14336x4096 Q4_K GEMV (fused C port, OpenMP)" % n,
               "us_per_call": dt * 1e6}
        # reference CPU path: dense linear on the dequantized weight (ATen)
        what = torch.from_numpy(oracle.dequant(cfg.fmt, packed, cfg.n_out, cfg.n_in)).to(torch.bfloat16)
        xb = torch.from_numpy(xf).to(torch.bfloat16)[None, :]
        torch.set_num_threads(threads)
        torch.nn.functional.linear(xb, what)
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 6.0:
            torch.nn.functional.linear(xb, what)
            n += 1
        dt2 = (time.perf_counter() - t0) / n
        out["aten_dense_bf16_us_per_call"] = dt2 * 1e6
        out["aten_dense_bf16_weight_GBps"] = what.numel() * 2 / dt2 / 1e9
        return out

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
        ncopies = max(2, -(-2 * MALL_BYTES // packed.nbytes))
        ws = [to_dev(packed) for _ in range(ncopies)]
        y = torch.empty((1, n_ff), dtype=torch.bfloat16, device=dev)
        gu = torch.empty((1, 2 * n_ff), dtype=torch.float32, device=dev)
        L = _lib.lib()
        sp = torch.cuda.current_stream(dev).cuda_stream

        def fused(i):
            _lib.check(L.ttq_gemv_q4_k_silu_mul(ws[i % ncopies].data_ptr(), x.data_ptr(), F.BF16, y.data_ptr(),
                                                F.BF16, 1, n_ff, n_in, torch.cuda.current_stream(dev).cuda_stream),
                       "ttq_gemv_q4_k_silu_mul")

        gu16 = torch.empty((1, 2 * n_ff), dtype=torch.bfloat16, device=dev)
        st = _lib.QLinearStruct(format=F.Q4_K, n_out=2 * n_ff, n_in=n_in)
        import ctypes as C

        def unfused(i):
            cur = torch.cuda.current_stream(dev).cuda_stream
            st.qweight = ws[i % ncopies].data_ptr()
            _lib.check(L.ttq_linear_forward(C.byref(st), x.data_ptr(), F.BF16, 1, gu16.data_ptr(), F.BF16, cur),
                       "ttq_linear_forward")
            _lib.check(L.ttq_silu_and_mul(gu16.data_ptr(), y.data_ptr(), F.BF16, 1, n_ff, cur), "ttq_silu_and_mul")

        # the same with the block's add + RMSNorm in front: one launch against four
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

        _, f_ms = time_steps(fused, steps, warmup, use_graph=not args.eager)
        _, u_ms = time_steps(unfused, steps, warmup, use_graph=not args.eager)
        _, nf_ms = time_steps(norm_fused, steps, warmup, use_graph=not args.eager)
        _, nu_ms = time_steps(norm_unfused, steps, warmup, use_graph=not args.eager)
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

        _, pf_ms = time_steps(pre_fused, 20, 3, use_graph=not args.eager)
        _, pu_ms = time_steps(pre_unfused, 20, 3, use_graph=not args.eager)
        res["prefill_m2048_fused_gemm_ms_per_step"] = pf_ms
        res["prefill_m2048_gemm_plus_silu_ms_per_step"] = pu_ms
        res["prefill_m2048_fused_TFLOPs"] = 2.0 * 2048 * 2 * n_ff * n_in / (pf_ms * 1e-3) / 1e12
        log("[q4_k_gate_up_silu_gemm M=2048] fused %.1f us/step (%.0f TFLOP/s), GEMM + silu_and_mul %.1f us/step"
            % (pf_ms * 1e3, res["prefill_m2048_fused_TFLOPs"], pu_ms * 1e3))
        return res

    def run_widened(steps: int, warmup: int):
        """Rows next to the headline ones, on random packed bytes with finite scale fields (timing
        only): the few-row decode GEMV (8 and 16 activation rows at once), the few-row form of the
        prefill operator (32 rows) and the prefill GEMM for Q6_K and Q8_0 weights, 14336 x 4096 unless
        named otherwise; add + RMSNorm on rows of 4096."""
        n_out, n_in = 14336, 4096
        rng = np.random.default_rng(1234)
        res = {}

        def random_packed(fmt, n_out=n_out, n_in=n_in):
            nbytes, wpb, scale_hi = {F.Q8_0: (34, 32, [1]), F.Q4_K: (144, 256, [1, 3]), F.Q6_K: (210, 256, [209])}[fmt]
            raw = rng.integers(0, 256, (n_out * (n_in // wpb), nbytes), dtype=np.uint8)
            for off in scale_hi:
                raw[:, off] &= 0x3F            # |fp16 scale| < 2
            return raw.reshape(-1)

        def timed(name, fmt, m, fn_of, n_out=n_out, n_in=n_in):
            packed = random_packed(fmt, n_out, n_in)
            ncopies = max(2, -(-2 * MALL_BYTES // packed.nbytes))
            ws = [to_dev(packed) for _ in range(ncopies)]
            x = torch.randn((m, n_in), device=dev).to(torch.bfloat16)
            step = fn_of(ws, x, ncopies)
            _, ev_ms = time_steps(step, steps, warmup, use_graph=not args.eager)
            res[name] = {"us_per_step": ev_ms * 1e3, "weight_GBps": packed.nbytes / (ev_ms * 1e-3) / 1e9,
                         "TFLOPs": 2.0 * m * n_out * n_in / (ev_ms * 1e-3) / 1e12}
            log("[%s] %.2f us/step  %.0f GB/s  %.1f TFLOP/s" % (name, ev_ms * 1e3, res[name]["weight_GBps"],
                                                              res[name]["TFLOPs"]))
            del ws
            torch.cuda.empty_cache()

        for m in (8, 16):
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
                  lambda ws, x, nc, y=y, fmt=fmt: (lambda i: QL.gemm(fmt, ws[i % nc], x, n_out, n_in, out=y)))
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

            _, ev_ms = time_steps(norm_step, steps, warmup, use_graph=not args.eager)
            nm = "add_rmsnorm_m%d" % m
            res[nm] = {"us_per_step": ev_ms * 1e3, "GBps": 4.0 * m * n_in * 2 / (ev_ms * 1e-3) / 1e9}
            log("[%s] %.2f us/step  %.0f GB/s" % (nm, ev_ms * 1e3, res[nm]["GBps"]))
            del xs, rs
            torch.cuda.empty_cache()
        return res

    def run_dense_reference(steps: int, warmup: int):
        """Context, not the product: the vendor library's plain bf16 linear (torch -> hipBLASLt) on
        dense 14336 x 4096 weights, i.e. what the reference's Linear.forward would run on this GPU
        after dequantizing once.  Same timing method, weight copies rotated past the cache."""
        n_out, n_in = 14336, 4096
        ncopies = max(2, -(-2 * MALL_BYTES // (n_out * n_in * 2)))
        ws = [torch.randn((n_out, n_in), device=dev).mul_(0.02).to(torch.bfloat16) for _ in range(ncopies)]
        res = {}
        for m in (1, 64, 512, 2048):
            x = torch.randn((m, n_in), device=dev).to(torch.bfloat16)
            y = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
            n = max(10, steps // (1 if m <= 64 else 4))
            _, ev_ms = time_steps(lambda i: torch.matmul(x, ws[i % ncopies].t(), out=y), n, warmup,
                                  use_graph=not args.eager)
            res["m%d" % m] = {"us_per_step": ev_ms * 1e3, "TFLOPs": 2.0 * m * n_out * n_in / (ev_ms * 1e-3) / 1e12,
                              "weight_GBps": n_out * n_in * 2 / (ev_ms * 1e-3) / 1e9}
            log("[dense_bf16_library m=%d] %.2f us/step  %.1f TFLOP/s  %.0f GB/s of bf16 weights" % (
                m, ev_ms * 1e3, res["m%d" % m]["TFLOPs"], res["m%d" % m]["weight_GBps"]))
        del ws
        torch.cuda.empty_cache()
        return res

    if args.only == "dense_reference":
        print(json.dumps(run_dense_reference(max(20, args.steps // 10), max(3, args.warmup // 10))), flush=True)
        return 0
    if args.only == "widened":
        print(json.dumps(run_widened(max(20, args.steps // 4), max(3, args.warmup // 4))), flush=True)
        return 0
    if args.only == "q4_k_gate_up_silu_gemv":
        print(json.dumps(run_gate_up(max(20, args.steps // 4), max(3, args.warmup // 4))), flush=True)
        return 0
    names = [args.only] if args.only else ["q4_k_gemv"]
    if not args.only and not args.no_extra:
        names += ["q4_k_gemm_m512", "q8_0_gemv", "q6_k_gemv", "exl3_gemv", "q4_k_gemm_m64", "q4_k_gemm_m2048"]
    results = {}
    for nme in names:
        cfg = CFG.CONFIGS[nme]
        steps = args.steps
        if cfg.m > 1 or nme == "q6_k_gemv":
            steps = max(20, args.steps // 10)     # longer kernels need fewer launches
        if cfg.m >= 2048:
            steps = max(10, args.steps // 40)
        results[nme] = run_config(nme, steps, max(3, args.warmup * steps // max(1, args.steps)))
    head = results[names[0]]
    hc = CFG.CONFIGS[names[0]]

    line = {
        "metric": METRIC,
        "value": head["weight_GBps"] if hc.m == 1 else head["TFLOPs"],
        "unit": "GB/s" if hc.m == 1 else "TFLOP/s",
        "n_gpus": 1, "steps": head["steps"], "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s: W %dx%d %s, x %dx%d %s, y %s" % (
            hc.name, hc.n_out, hc.n_in, {0: "Q8_0", 1: "Q4_K", 2: "Q6_K", 3: "EXL3"}[hc.fmt], hc.m, hc.n_in,
            hc.x_dtype, hc.y_dtype),
            "launch": "eager" if args.eager else "hip-graph replay of %d launches" % head["steps"],
            "weight_copies_rotated": head["weight_copies"]},
    }
    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (committed summary)
    traffic = None
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f).get(hc.name)
        if t:
            traffic = t["hbm_read_bytes"] + t["hbm_write_bytes"]
    except (OSError, ValueError):
        pass
    if hc.m == 1:
        line["roofline"] = {"bound": "hbm", "achieved": head["weight_GBps"], "peak": HBM_PEAK_GBPS,
                            "unit": "GB/s", "frac": head["weight_GBps"] / HBM_PEAK_GBPS, "traffic": traffic,
                            "algorithmic_bytes": head["weight_bytes"]}
    else:
        line["roofline"] = {"bound": "mfma", "achieved": head["TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS,
                            "unit": "TFLOP/s", "frac": head["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic}
    if "q4_k_gemm_m512" in results:
        g = results["q4_k_gemm_m512"]
        line["gemm_m512_TFLOPs"] = g["TFLOPs"]
        line["gemm_m512_mfma_frac"] = g["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    line["extra"] = {k: v for k, v in results.items() if k != names[0]}
    if not args.only and not args.no_extra:
        line["extra"]["q4_k_gate_up_silu_gemv"] = run_gate_up(max(20, args.steps // 4), max(3, args.warmup // 4))
        line["extra"]["widened"] = run_widened(max(20, args.steps // 4), max(3, args.warmup // 4))
        line["extra"]["dense_bf16_library_14336x4096"] = run_dense_reference(max(20, args.steps // 10),
                                                                             max(3, args.warmup // 10))
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
