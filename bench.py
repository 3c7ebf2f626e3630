#!/usr/bin/env python3
"""Benchmark of the fused P-way gradient reduce + optimizer update on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload adam_f32]

A "step" is one launch of the hot path over the whole shard with inputs resident in HBM.  The default
workload is benchmark configuration 2: fused reduce + bias-corrected Adam, fp32, N = 2^28 parameters, P = 8
rank-gradient buffers.  One JSON line is printed: whole-job algorithmic GB/s (56 B/param for Adam), the
roofline of the dominant kernel from HIP events recorded on the launch stream, and the CPU restatement of the
reference checker loop timed on a bounded sample on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

METRIC = "fused reduce+Adam GB/s & % HBM roofline, N=2^28 P=8; params/s"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="adam_f32",
                    choices=["adam_f32", "adam_f32_scattered", "sgd_f32", "adam_f16g", "adam_bf16g", "lamb_f32",
                             "lamb_nccl_f16g", "mlp_outproj", "matmul_bf16", "matmul_bf16_c16", "copy", "copy_stream"])
    ap.add_argument("--log2n", type=int, default=None, help="override log2 of the parameter count")
    ap.add_argument("--ranks", type=int, default=None, help="override P")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true",
                    help="default run only: leave out the short runs of the other benchmark configurations")
    ap.add_argument("--graph-steps", type=int, default=0,
                    help="record this many steps once (ccn_graph_*) and time replays of the recording: for launch-bound "
                         "sizes such as config 1; a recorded step keeps its step number")
    ap.add_argument("--allocator", default="ccn", choices=["ccn", "torch"],
                    help="ccn: buffers from ccn_malloc (channel-staggered); torch: plain torch allocations")
    return ap.parse_args()


class Buffers:
    """Device buffers from the library's own allocator (ccn_malloc), the one the generated driver uses.  It
    staggers buffer starts so that the P+3 arrays walked in lock step do not collide on HBM channels;
    --allocator torch uses plain torch allocations (same-sized blocks, starts a power of two apart) instead."""

    def __init__(self, capi, torch, use_torch):
        self.capi, self.torch, self.use_torch, self.keep = capi, torch, use_torch, []

    def from_tensor(self, t):
        if self.use_torch:
            self.keep.append(t)
            return t
        nbytes = t.numel() * t.element_size()
        a = self.capi.malloc(nbytes)
        self.capi.memcpy_d2d(a, t, nbytes)
        self.torch.cuda.synchronize()
        self.keep.append(a)
        return a


def source_sha256(rel):
    import hashlib
    with open(os.path.join(ROOT, rel), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def traffic_from_profiles(name):
    """HBM bytes per launch measured with rocprofv3 --pmc, from the committed summary of this workload -- or None when
    there is none, or when the kernel's source file has changed since the summary was taken (every summary records the
    SHA-256 of the source file its kernel is compiled from: a stale figure is not passed on)."""
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    vals, fresh = {}, False
    for line in open(path):
        if line.startswith("SOURCE_SHA256="):
            digest, rel = line.split("=", 1)[1].split()[:2]
            try:
                fresh = source_sha256(rel) == digest
            except OSError:
                fresh = False
        if "=" in line and line.split("=")[0].strip() in ("FETCH_BYTES_PER_LAUNCH", "WRITE_BYTES_PER_LAUNCH"):
            k, v = line.split("=", 1)
            try:
                vals[k.strip()] = float(v.split()[0])
            except ValueError:
                pass
    if len(vals) == 2 and fresh:
        return vals["FETCH_BYTES_PER_LAUNCH"] + vals["WRITE_BYTES_PER_LAUNCH"]
    return None


def cpu_baseline(wl, P, budget_s=8.0):
    """The oracle's restatement of the reference loops (for Adam: multi-process-adam-scattered.cpp:112-136 with a
    fixed-order P-way sum), C compiled -O2 -ffp-contract=off -fopenmp, on a bounded sample of the same workload: once on
    one thread, as the reference runs its checker, and once as an OpenMP parallel-for over the elements (whole segments
    for LAMB, rows for the MLP) on the host threads this box gives a job.  Same arithmetic and results either way."""
    import oracle as orc
    threads = max(1, min(16, os.cpu_count() or 1))     # a one-GPU box gives a job 16 host threads
    r = np.random.Generator(np.random.Philox(key=[5, 0]))
    f32 = np.float32
    if wl in ("mlp_outproj", "matmul_bf16", "matmul_bf16_c16"):
        # a band of rows of the 8192 x 1024 x 8192 product with its 7 partial buffers
        rows, Nn, Kd, nP = 8 * threads, 8192, 1024, (7 if wl == "mlp_outproj" else 0)
        X = orc.f32_to_bf16(r.standard_normal((rows, Kd), dtype=f32))
        Wm = orc.f32_to_bf16(r.standard_normal((Kd, Nn), dtype=f32) * f32(0.02))
        parts = [r.standard_normal((rows, Nn), dtype=f32) for _ in range(nP)]
        bias = r.standard_normal(Nn, dtype=f32)
        resid = orc.f32_to_bf16(r.standard_normal((rows, Nn), dtype=f32))
        units, per_unit = rows * Nn, (nP * 4 + 2 + 2) + (Kd * 2 * 2.0) / 8192   # bytes per output, X and W amortised
        what = f"oracle orc_mlp_outproj (a float64 brute-force product, a checker and not a tuned CPU GEMM) on {rows} of the 8192 rows (K=1024, {nP} partials)"

        def piece(t):
            orc.mlp_outproj(X, Wm, parts, bias, resid, rows, Nn, Kd, 0.1 if nP else 0.0, 0)
    else:
        # the headline workload on a quarter of its elements (2^26: 3 GB of host memory), the others on 2^24
        n = 1 << (26 if wl in ("adam_f32", "adam_f32_scattered") else 24)
        nseg = 16
        segs = [k * (n // nseg) for k in range(nseg + 1)]
        half = wl in ("adam_f16g", "adam_bf16g", "lamb_nccl_f16g")
        scale = f32(2.0 ** 7 if wl == "adam_bf16g" else 2.0 ** 16 if wl == "adam_f16g" else 1.0)
        base = r.standard_normal(n, dtype=f32) * f32(1e-3)
        g = [np.roll(base, 1000003 * p) for p in range(P)]      # one draw, shifted per rank: distinct arrays, same statistics
        del base
        if half:
            g = [(orc.f32_to_bf16 if wl == "adam_bf16g" else orc.f32_to_f16)(x * scale) for x in g]
        w = r.uniform(-0.05, 0.05, n).astype(f32)
        m = np.zeros(n, f32)
        v = np.full(n, 1e-6, f32) if wl == "lamb_nccl_f16g" else np.zeros(n, f32)
        w16 = np.zeros(n, np.uint16)
        units = n
        per_unit = {"sgd_f32": (P + 1) * 4 + 4, "adam_f32": (P + 3) * 4 + 12, "adam_f32_scattered": (P + 3) * 4 + 12,
                    "lamb_f32": (P + 3) * 4 + 12}.get(wl, P * 2 + 12 + 12 + 2)
        what = (f"oracle loop of {wl}, P={P}, N=2^{int(np.log2(n))} sample of the 2^28 workload"
                + (" in 16 segments" if "lamb" in wl else ""))

        def piece(t):
            if wl == "sgd_f32":
                orc.sgd_f32(g, w, 0.01)
            elif wl in ("adam_f32", "adam_f32_scattered"):
                orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
            elif wl == "adam_f16g":
                orc.adam_f16g(g, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, t, f32(1.0) / scale)
            elif wl == "adam_bf16g":
                orc.adam_bf16g(g, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, t, f32(1.0) / scale)
            elif wl == "lamb_f32":
                orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
            else:
                orc.lamb_nccl_f16g(g, w, w16, m, v, segs, 1e-3, 0.9, 0.999, 1.0)
    orc.set_num_threads(threads)
    piece(1)          # warm the pages

    def timed(nthreads):
        orc.set_num_threads(nthreads)
        t0 = time.perf_counter()
        reps = 0
        while True:
            piece(reps + 2)
            reps += 1
            el = time.perf_counter() - t0
            if el > budget_s or reps >= 400:
                return el / (reps * units), reps

    many, repsT = timed(threads)
    one, reps1 = timed(1)
    orc.set_num_threads(1)
    return {
        "value": round(per_unit / many / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "params_per_s": round(1.0 / many, 1),
        "single_thread": {"value": round(per_unit / one / 1e9, 3), "unit": "GB/s", "params_per_s": round(1.0 / one, 1)},
        "sample": f"{what}; C loop (-O2 -ffp-contract=off -fopenmp): {repsT} steps as an OpenMP parallel-for on {threads} threads, "
                  f"{reps1} steps on 1 thread as the reference runs it ({os.cpu_count()} host cpus visible)",
    }


def build_workload(a, wl, capi, torch, stream, allocator):
    """Allocates the synthetic inputs of one workload in HBM.  Returns (step, alg_bytes, units, kernel, config, flops, P, keep)
    where step(t) enqueues one pass of the hot path on `stream` and `keep` holds what must stay alive."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    flops = None
    P = 8
    keep = []
    if wl == "adam_f32_scattered":
        # the same step with gradients and weights in 256 separate buffers (one per "parameter tensor")
        P = a.ranks or 8
        N = 1 << (a.log2n or 28)
        nbuff = 256
        per = N // nbuff
        bufs = Buffers(capi, torch, allocator == "torch")
        mk = lambda scale: bufs.from_tensor(torch.empty(per, device="cuda").normal_(0.0, scale, generator=gen))
        g = [[mk(1e-3) for _ in range(nbuff)] for _ in range(P)]
        w = [mk(0.05) for _ in range(nbuff)]
        m = bufs.from_tensor(torch.zeros(N, device="cuda"))
        v = bufs.from_tensor(torch.zeros(N, device="cuda"))
        plan = capi.ScatterPlan([per] * nbuff)
        per_param = (P + 3) * 4 + 3 * 4
        step = lambda t: plan.adam(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t, stream)
        kernel = "scattered_stream_kernel<AdamMath, %d>" % (P if P <= 8 else 0)
        alg_bytes = float(per_param) * N
        units = N
        config = {"workload": f"adam_f32 over {nbuff} scattered buffers, N=2^{int(np.log2(N))}, P={P}", "N": N, "P": P,
                  "algorithmic_bytes_per_param": per_param, "allocator": allocator}
        keep = [bufs, plan]
    elif wl in ("adam_f32", "sgd_f32", "lamb_f32", "adam_f16g", "adam_bf16g", "lamb_nccl_f16g", "sgd_f32_large"):
        large_sgd = wl == "sgd_f32_large"       # configuration 1's shape at a size that leaves the caches
        if large_sgd:
            wl = "sgd_f32"
        P = a.ranks or (4 if wl == "sgd_f32" else 8)
        N = 1 << (a.log2n or (28 if large_sgd else 20 if wl == "sgd_f32" else 28))
        gbytes = 2 if wl in ("adam_f16g", "adam_bf16g", "lamb_nccl_f16g") else 4
        half = torch.bfloat16 if wl == "adam_bf16g" else torch.float16
        gscale = 2.0 ** 7 if wl == "adam_bf16g" else 2.0 ** 16
        bufs = Buffers(capi, torch, allocator == "torch")
        g = []
        for p in range(P):
            if gbytes == 2:
                t = (torch.randn(N, device="cuda", generator=gen) * (1e-3 * gscale)).to(half)
                if p == 0 and wl != "lamb_nccl_f16g":
                    t[::1 << 20] = float("inf")        # benchmark configuration 3: one entry in 2^20 overflows
            else:
                t = torch.empty(N, device="cuda").normal_(0.0, 1e-3 if wl != "sgd_f32" else 1e-2, generator=gen)
            g.append(bufs.from_tensor(t))
            del t
        w = bufs.from_tensor(torch.empty(N, device="cuda").uniform_(-0.05, 0.05, generator=gen))
        m = bufs.from_tensor(torch.zeros(N, device="cuda"))
        v = bufs.from_tensor(torch.zeros(N, device="cuda"))
        keep = [bufs]
        if wl == "adam_f32":
            per_param = (P + 3) * 4 + 3 * 4
            step = lambda t: capi.adam_f32(g, w, m, v, N, 1e-3, 0.9, 0.999, 1e-6, t, stream)
            kernel = "fused_stream_kernel<AdamMath, %d, 4, 1, 64>" % (P if P <= 8 else 0)
        elif wl == "sgd_f32":
            per_param = (P + 1) * 4 + 4
            step = lambda t: capi.sgd_f32(g, w, N, 0.01, stream)
            kernel = "fused_stream_kernel<SgdMath, %d, 4, 1, %d>" % (P if P <= 8 else 0, 256 if P + 2 <= 3 else 64)
        elif wl == "lamb_nccl_f16g":
            # the modified NCCL's mixed-precision LAMB, 256 segments
            w16 = bufs.from_tensor(torch.empty(N, dtype=torch.float16, device="cuda"))
            nseg = 256 if N >= (1 << 20) * 256 else max(1, N >> 20)
            plan = capi.LambPlan([i * (N // nseg) for i in range(nseg + 1)])
            keep.append(plan)
            per_param = P * 2 + 12 + 12 + 2
            step = lambda t: plan.step_nccl_f16g(g, w, w16, m, v, 1e-3, 0.9, 0.999, 1.0, stream)
            kernel = "lamb_reset_kernel + lamb_oneshot_kernel<%d, 256, 8, false, uint16_t> + lamb_deferred_kernel<256, 8, false, true>" % (P if P <= 8 else 0)
        elif gbytes == 2:
            w16 = bufs.from_tensor(torch.empty(N, dtype=half, device="cuda"))
            flag = torch.zeros(1, dtype=torch.int32, device="cuda")
            keep.append(flag)
            per_param = P * 2 + 12 + 12 + 2
            call = capi.adam_bf16g if wl == "adam_bf16g" else capi.adam_f16g
            step = lambda t: call(g, w, m, v, w16, N, 1e-3, 0.9, 0.999, 1e-6, t, 1.0 / gscale, flag, stream)
            kernel = "fused_stream_kernel<Adam16MathT<%s>, %d, 4, 1, 64>" % ("true" if wl == "adam_bf16g" else "false",
                                                                             P if P <= 8 else 0)
        else:
            nseg = 256 if N >= (1 << 20) * 256 else max(1, N >> 20)
            plan = capi.LambPlan([i * (N // nseg) for i in range(nseg + 1)])
            keep.append(plan)
            per_param = (P + 3) * 4 + 3 * 4
            step = lambda t: plan.step(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, capi.LAMB_TRUST_RATIO, stream)
            kernel = "lamb_reset_kernel + lamb_oneshot_kernel<%d, 256, 8> + lamb_deferred_kernel<256, 8>" % (P if P <= 8 else 0)
        alg_bytes = float(per_param) * N
        units = N
        config = {"workload": f"{wl} fused reduce+update, N=2^{int(np.log2(N))}, P={P}", "N": N, "P": P,
                  "algorithmic_bytes_per_param": per_param, "allocator": allocator}
    elif wl == "mlp_outproj":
        M = Nn = 8192
        Kd = 1024
        X = torch.randn(M, Kd, device="cuda", generator=gen).to(torch.bfloat16)
        Wm = (torch.randn(Kd, Nn, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
        parts = [torch.randn(M, Nn, device="cuda", generator=gen) for _ in range(7)]
        bias = torch.randn(Nn, device="cuda", generator=gen)
        resid = torch.randn(M, Nn, device="cuda", generator=gen).to(torch.bfloat16)
        out = torch.empty(M, Nn, dtype=torch.bfloat16, device="cuda")
        step = lambda t: capi.mlp_outproj_bf16(X, Wm, parts, bias, resid, out, M, Nn, Kd, 0.1, 0, stream)
        alg_bytes = float(7 * M * Nn * 4 + M * Kd * 2 + Kd * Nn * 2 + Nn * 4 + 2 * M * Nn * 2)
        flops = 2.0 * M * Nn * Kd
        units = M * Nn
        kernel = "mlp_outproj_kernel<7>"
        config = {"workload": "mlp_outproj bf16 8192x1024x8192 + 7 fp32 partials + bias + dropout(0.1) + residual",
                  "M": M, "N": Nn, "K": Kd}
    elif wl in ("matmul_bf16", "matmul_bf16_c16"):
        # the MatMul step of the unfused schedules alone (the reference: cublasGemmEx, src/codegen.cpp:1058-1136), with C in
        # fp32 (what the unfused lowering here keeps) or in the operands' 16-bit type (what the reference's call writes)
        M = Nn = 8192
        Kd = 1024
        c16 = wl == "matmul_bf16_c16"
        X = torch.randn(M, Kd, device="cuda", generator=gen).to(torch.bfloat16)
        Wm = (torch.randn(Kd, Nn, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
        Cm = torch.empty(M, Nn, device="cuda", dtype=torch.bfloat16 if c16 else torch.float32)
        step = (lambda t: capi.matmul_16(X, Wm, Cm, M, Nn, Kd, stream)) if c16 else (lambda t: capi.matmul_bf16_f32(X, Wm, Cm, M, Nn, Kd, stream))
        alg_bytes = float(M * Kd * 2 + Kd * Nn * 2 + M * Nn * (2 if c16 else 4))
        flops = 2.0 * M * Nn * Kd
        units = M * Nn
        kernel = "matmul_tile256_kernel<false, true>" if c16 else "matmul_tile256_kernel<false, false>"
        config = {"workload": f"matmul bf16 8192x1024x8192 -> {'bf16' if c16 else 'fp32'} (the unfused schedule's MatMul step)",
                  "M": M, "N": Nn, "K": Kd}
    elif wl == "copy_stream":
        # a 1R:1W stream through the library's own streaming kernel (ccn_reduce_f32 over one rank buffer is a copy): the
        # ceiling of this box for the launch shape the fused kernels use
        N = 1 << (a.log2n or 30)
        bufs = Buffers(capi, torch, allocator == "torch")
        src = bufs.from_tensor(torch.empty(N, dtype=torch.float32, device="cuda").normal_(generator=gen))
        dst = bufs.from_tensor(torch.empty(N, dtype=torch.float32, device="cuda"))
        step = lambda t: capi.reduce_f32([src], dst, N, stream)
        alg_bytes = 8.0 * N
        units = N
        kernel = "fused_stream_kernel<ReduceMath, 1, 4, 1, 256>"
        config = {"workload": f"copy of 2^{int(np.log2(N))} fp32 through the library's streaming kernel (ccn_reduce_f32, P=1)"}
        keep = [bufs]
    else:   # plain device copy, the practical HBM ceiling of this box
        N = 1 << (a.log2n or 30)
        src = torch.empty(N, dtype=torch.float32, device="cuda").normal_(generator=gen)
        dst = torch.empty_like(src)
        step = lambda t: dst.copy_(src)
        alg_bytes = 8.0 * N
        units = N
        kernel = "torch copy"
        config = {"workload": f"device copy of 2^{int(np.log2(N))} fp32"}
    return step, alg_bytes, units, kernel, config, flops, P, keep


def release(keep, capi, torch):
    """Gives a workload's device memory back before the next one is allocated."""
    for k in keep:
        if isinstance(k, Buffers):
            for x in k.keep:
                if isinstance(x, int):
                    capi.free(x)
            k.keep = []
        elif hasattr(k, "close"):
            k.close()
    keep.clear()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def timed_steps(step, K, W, capi, torch, stream):
    """W untimed steps, then K steps bracketed by a device synchronisation on both sides.  Returns the wall-clock and the
    HIP-event time per step (events recorded on the launch stream)."""
    for t in range(1, W + 1):
        step(t)
    torch.cuda.synchronize()
    e0, e1 = capi.Event(), capi.Event()
    t0 = time.perf_counter()
    e0.record(stream)
    for t in range(W + 1, W + K + 1):
        step(t)
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / K, e0.elapsed_ms(e1) / K


def other_workloads(a, capi, torch, stream):
    """Short runs of the other benchmark configurations, and of the headline kernel on plain (unstaggered) allocations,
    so that every configuration's figure comes from the same command as the headline.  Few steps each: these are HBM-bound
    kernels of a few milliseconds whose launch times spread by about a percent."""
    rows = []
    # The headline kernel on plain allocations, in a process of its own: same-sized blocks straight from a fresh
    # allocator are the case a caller that does not use ccn_malloc starts from (what an allocator hands out after other
    # buffers have come and gone in the same process is placed differently and measures differently).
    import subprocess
    child = subprocess.run([sys.executable, os.path.abspath(__file__), "--allocator", "torch", "--steps", "30", "--warmup", "10",
                            "--no-cpu-baseline", "--no-others"], capture_output=True, text=True, timeout=300)
    try:
        c = json.loads(child.stdout.strip().splitlines()[-1])
        rows.append({"workload": c["config"]["workload"], "allocator": "torch (fresh process)", "steps": c["steps"],
                     "warmup": c["warmup"], "ms_per_step": c["ms_per_step"], "avg_launch_ms": c["roofline"]["avg_launch_ms"],
                     "algorithmic_GBps": c["roofline"]["achieved"], "frac_of_hbm_peak": c["roofline"]["frac"],
                     "kernel": c["roofline"]["kernel"],
                     "algorithmic_bytes_per_launch": c["roofline"]["algorithmic_bytes_per_launch"], "traffic": None})
    except (ValueError, KeyError, IndexError):
        rows.append({"workload": "adam_f32 on plain allocations", "error": (child.stderr or child.stdout)[-300:]})
    for wl, allocator in (("adam_f32", "torch"), ("sgd_f32", "ccn"), ("sgd_f32_graph", "ccn"), ("sgd_f32_large", "ccn"),
                          ("adam_f16g", "ccn"), ("lamb_f32", "ccn"), ("mlp_outproj", "ccn"), ("matmul_bf16", "ccn"), ("matmul_bf16_c16", "ccn"),
                          ("copy", "torch"), ("copy_stream", "ccn")):
        replay = 64 if wl == "sgd_f32_graph" else 0      # configuration 1 again, 64 recorded steps per graph launch
        own = capi.Stream() if replay else None          # the null stream cannot be recorded
        st = own.h if own else stream
        step, alg_bytes, units, kernel, config, flops, P, keep = build_workload(a, "sgd_f32" if replay else wl, capi, torch, st,
                                                                                allocator)
        steps, warm = (200, 20) if alg_bytes < 1e9 else (30, 10)
        if replay:
            step(1)
            torch.cuda.synchronize()
            with capi.Graph(own) as graph:
                for t in range(replay):
                    step(2 + t)
            wall_ms, ev_ms = timed_steps(lambda t: graph.launch(), steps, warm, capi, torch, st)
            wall_ms, ev_ms, steps = wall_ms / replay, ev_ms / replay, steps * replay
            config["workload"] += f", {replay} recorded steps per ccn_graph_launch"
        else:
            wall_ms, ev_ms = timed_steps(step, steps, warm, capi, torch, st)
        ach = alg_bytes / (ev_ms * 1e-3) / 1e9
        row = {"workload": config["workload"], "allocator": allocator, "steps": steps, "warmup": warm,
               "ms_per_step": round(wall_ms, 5), "avg_launch_ms": round(ev_ms, 5), "algorithmic_GBps": round(ach, 2),
               "frac_of_hbm_peak": round(ach / HBM_PEAK_GBPS, 4), "kernel": kernel,
               "algorithmic_bytes_per_launch": alg_bytes,
               "traffic": traffic_from_profiles(f"{'sgd_f32' if wl == 'sgd_f32_large' else wl}.pmc.txt") if allocator == "ccn" else None}
        if alg_bytes < 1e9 and not wl.startswith("matmul_bf16"):
            row["note"] = "fits the caches and is bound by launches: not a roofline figure"
        if wl == "copy":
            row["note"] = "torch's device-to-device copy_ on this box"
        if wl == "copy_stream":
            row["note"] = ("the measured ceiling of a 1R:1W stream on this box in the launch shape of the fused kernels: read the "
                           "fractions of the 8 TB/s nominal peak against it")
        if replay:
            graph.close()
            own.close()
        if flops:
            row["mfma_TFLOPs"] = round(flops / (ev_ms * 1e-3) / 1e12, 2)
            row["frac_of_mfma_peak"] = round(flops / (ev_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)
        rows.append(row)
        del step
        release(keep, capi, torch)
    return rows


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the reduce over P rank buffers is local); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from coconet_amd import capi
    capi.load()
    capi.init(0)
    torch.cuda.set_device(0)
    info = capi.device_info()
    K, W = a.steps, a.warmup
    wl = a.workload
    own_stream = capi.Stream() if a.graph_steps > 0 else None      # the null stream cannot be recorded
    stream = own_stream.h if own_stream else torch.cuda.current_stream().cuda_stream

    step, alg_bytes, units, kernel, config, flops, P, keep = build_workload(a, wl, capi, torch, stream, a.allocator)

    if a.graph_steps > 0:
        if wl in ("copy",):
            sys.exit("--graph-steps records library calls only")
        step(1)                                  # first call outside the recording (LAMB plans query occupancy once)
        torch.cuda.synchronize()
        with capi.Graph(own_stream) as graph:
            for t in range(a.graph_steps):
                step(2 + t)
        eager_step, K = step, max(1, K // a.graph_steps)
        step = lambda t: graph.launch()
        config["graph_steps"] = a.graph_steps
    wall_ms, ev_ms = timed_steps(step, K, W, capi, torch, stream)
    if a.graph_steps > 0:
        wall_ms, ev_ms = wall_ms / a.graph_steps, ev_ms / a.graph_steps
        K *= a.graph_steps                       # steps actually run

    # the spread of single launches, each bracketed by its own pair of events (outside the timed region)
    n_single = 0 if a.graph_steps > 0 else min(K, 50)
    pairs = [(capi.Event(), capi.Event()) for _ in range(n_single)]
    for i, (s0, s1) in enumerate(pairs):
        s0.record(stream)
        step(W + K + 1 + i)
        s1.record(stream)
    torch.cuda.synchronize()
    singles = sorted(s0.elapsed_ms(s1) for s0, s1 in pairs)

    gbps = alg_bytes / (wall_ms * 1e-3) / 1e9
    ach = alg_bytes / (ev_ms * 1e-3) / 1e9
    line = {
        "metric": METRIC if wl == "adam_f32" else f"{wl} algorithmic GB/s",
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"adam_f16g": "f16 gradients, f32 state", "adam_bf16g": "bf16 gradients, f32 state",
                  "lamb_nccl_f16g": "f16 gradients (f16 sum), f32 state",
                  "mlp_outproj": "bf16 x bf16 -> f32", "matmul_bf16": "bf16 x bf16 -> f32",
                  "matmul_bf16_c16": "bf16 x bf16 -> f32 -> bf16"}.get(wl, "f32"),
        "data": "synthetic", "config": config,
        "params_per_s": round(units / (wall_ms * 1e-3), 1),
        "device": info,
        "roofline": {"bound": "hbm", "achieved": round(ach, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": traffic_from_profiles(f"{wl}.pmc.txt"),
                     "kernel": kernel, "avg_launch_ms": round(ev_ms, 5), "algorithmic_bytes_per_launch": alg_bytes,
                     "median_launch_ms": round(singles[len(singles) // 2], 5) if singles else None,
                     "min_launch_ms": round(singles[0], 5) if singles else None},
    }
    if flops:
        line["mfma"] = {"achieved": round(flops / (ev_ms * 1e-3) / 1e12, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(flops / (ev_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
    if wl.startswith("matmul_bf16"):     # the one compute-bound kernel of the path: its roofline is the matrix cores'
        line["roofline"].update({"bound": "mfma", "achieved": line["mfma"]["achieved"], "peak": MFMA_BF16_PEAK_TFLOPS,
                                 "unit": "TFLOP/s", "frac": line["mfma"]["frac"], "algorithmic_flops_per_launch": flops})
    default_run = (wl == "adam_f32" and a.allocator == "ccn" and a.graph_steps == 0 and a.log2n is None and a.ranks is None)
    if default_run and not a.no_others:
        del step
        release(keep, capi, torch)
        line["other_workloads"] = other_workloads(a, capi, torch, stream)
    if wl not in ("copy", "copy_stream") and not a.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(wl, P if wl not in ("mlp_outproj", "matmul_bf16", "matmul_bf16_c16") else 8)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
