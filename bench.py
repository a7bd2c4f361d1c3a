#!/usr/bin/env python3
"""Benchmark of the native-layout hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--case TEXT] [--no-cpu] [--case-steps S]
                    [--no-eager] [--no-blas] [--counters]

Prints ONE JSON line.  The headline workload is the fp16 narrow GeMM of the
second benchmark configuration (`gemm_layoutA`, weights 11008 x 4096 in
layout-A, 16 tokens); one step is one call.  Inputs are synthetic, seeded and
resident in HBM before the timed region.  Every call of a timed region reads a
different weight copy (enough copies to exceed the 256 MiB Infinity Cache), so
the bandwidth is HBM bandwidth.

Timing protocol: the K calls are recorded into one HIP graph.  After the W
warm-up calls and un-timed replays of the graph for at least 100 ms, the graph
is replayed five times, each replay (exactly K calls) bracketed by HIP events
on the stream that runs it and queued behind at least half a millisecond of
un-timed replays.  A graph takes some 7 us from its launch to its first kernel
even then, and a short graph bills that to its few calls (+0.4 us per call at
K = 20, +1.5 us at K = 5): below K = 200 the timed GeMV / GeMM calls are
therefore launched one by one between the events, behind 5 ms of queued
replays that give the host its head start (16.0 us per call at any K, against
15.9 us from a graph of 1000).  The headline value is the median of the five timed runs (as for the yardsticks);
the first and the minimum of the five are reported beside it, and for every
other configuration.  `ms_per_step` is the host clock around one more replay
between two synchronizations, launch latency included.  Why 100 ms and why long replays: the capture
leaves the GPU idle and the first replays after an idle period run several
percent below the steady state; the kernels that stream the largest matrices
(the 235 MB soft-FP8 GeMV / GeMM) only reach their steady state after some
50 to 100 ms of continuous load (38.4 us per call in 4 ms replays after 40 ms,
36.3 us in 38 ms replays after 100 ms).  The GeMV / GeMM configurations
therefore time 1000 calls per replay (--case-steps), as the reference's own
benchmark scripts time long back-to-back runs.

`per_config` holds the other configurations (bf16 / soft-FP8 GeMV, the M sweep,
the native-layout chain, the relayout kernels and the fused MoE layer) with
microseconds per call, achieved GB/s of algorithmic bytes, the fraction of the
8 TB/s HBM peak, a pure-read launch of the same weight bytes as a yardstick
where the weights are small, HBM traffic from hardware counters where a
profile under profiles/ holds it, and the CPU baseline of that configuration:
the reference's CPU-runnable torch path (a library linear on the un-packed
weights, or its dense MoE loop) timed on the host cores on a bounded sample.
The prefill lines ("next: prefill ...") report TFLOP/s and the fraction of the 2.5 PFLOP/s MFMA peak, the vendor BLAS
on un-packed weights of the same shape (`blas_us`) and `mfma_only_tflops`: what a loop of nothing but the MFMA instruction
sustains in the same run on operand values drawn like the benchmark's (the power limit, not the issue rate, sets it).

`eager_calls` holds the public Python API timed the way the reference's own
scripts time it: the wall clock around 1000 eager calls (300 for the fused MoE),
synchronized at both ends, host work included, next to the device time per
call of the same configuration.

`--counters` is for runs under `rocprofv3 --pmc`: every call is launched
directly, a handful per case, and no HIP graph is built (counter collection
over graph replays with thousands of dispatches crashed the profiler).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16 / bf16 (soft-FP8 weights are widened to bf16 before the product)
MALL_BYTES = 256 << 20
TIMED_REPLAYS = 5


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--quick", action="store_true", help="headline workload only")
    ap.add_argument("--moe-steps", type=int, default=20, help="fused_moe calls per timed replay")
    ap.add_argument("--no-blas", action="store_true", help="skip the vendor BLAS yardsticks (counter runs)")
    ap.add_argument("--case-steps", type=int, default=1000,
                    help="calls per timed replay of the per-configuration cases (never more than --steps)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--case", default=None,
                    help="besides the headline, run only the per-configuration cases whose name contains this text "
                         "(several texts separated by commas; for profiling single kernels)")
    ap.add_argument("--counters", action="store_true",
                    help="for runs under a hardware-counter profiler: every call is launched directly (no HIP graph is "
                         "built or replayed: counter collection over graph replays with thousands of dispatches has "
                         "crashed the profiler), no settle replays, --steps calls per case after --warmup calls, no "
                         "yardsticks, no vendor BLAS, no CPU legs, no eager-call lines; the headline runs only if "
                         "--case names it; timings of such a run are not benchmark numbers")
    ap.add_argument("--no-eager", action="store_true", help="skip the eager-call lines (public Python API, wall clock)")
    ap.add_argument("--tunable", action="append", default=[], metavar="ID=VALUE",
                    help="set an experiment switch of the library (mlk_set_tunable) before anything runs; repeatable")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain copy kernel of known size (256 MiB in, 256 MiB out) so that "
                         "hardware byte counters can be scaled against it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.counters:
        args.no_cpu = args.no_blas = args.no_eager = True

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    import muxi_native_layout_kernels_amd as mlk
    from muxi_native_layout_kernels_amd import _lib, arg_selector
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    lib = _lib.load()
    for item in args.tunable:
        ident, value = item.split("=")
        lib.mlk_set_tunable(int(ident), int(value))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(2025)
    DT = {0: torch.float16, 1: torch.bfloat16}
    cores = torch.get_num_threads()
    host_cpus = os.cpu_count() or 0

    traffic_table = {}
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        try:
            traffic_table = json.load(open(tpath))
        except (OSError, ValueError):
            traffic_table = {}

    def copies_for(nbytes):
        return int(max(2, min(24, (3 * MALL_BYTES + nbytes - 1) // nbytes)))

    def weights(n, k, kind, count):
        """`count` independent weight tensors, already in layout-A (values are i.i.d., so drawing
        them directly in packed order is the same distribution as packing a drawn matrix)."""
        out = []
        for _ in range(count):
            if kind == 2:
                w = (torch.randn((n // 16, k // 8, 16, 8), generator=gen, device=dev) * 16).clamp_(-448, 448)
                out.append(w.to(torch.float8_e4m3fn).view(torch.uint8))
            else:
                out.append((torch.randn((n // 16, k // 8, 16, 8), generator=gen, device=dev) * 0.02).to(DT[kind]))
        return out

    def block_scales(shape):
        """fp32 block scales of soft-FP8 weights: arbitrary values, as in the reference's scripts (a scale matrix drawn
        at random, benchmark_and_test/gemv_benchmark_soft_fp8.py:30), so the kernels take their general widening
        path; scales that are all exact powers of two take a cheaper one and are timed on one extra line."""
        return torch.rand(shape, generator=gen, device=dev) * 0.02 + 0.001

    bench_stream = torch.cuda.Stream()      # every timed region runs on this one stream

    def settle_replays(steps):
        return 1 + max(1, int(0.1 / (steps * 20e-6)))       # >= 100 ms at 20 us per call

    def run_graph(calls, steps, warmup, reps=TIMED_REPLAYS, direct_if_short=False):
        """Time `steps` calls (cycling through `calls`) `reps` times, each time between HIP events on the launching
        stream and queued behind un-timed work, so that the first timed call starts on a busy GPU.  The timed calls
        are one replay of a HIP graph that holds them.  A graph takes some 7 us from its launch to its first kernel
        even when it is queued behind other work, which a short graph bills to its few calls; so with
        `direct_if_short` (plain library calls, cheap on the host) fewer than 200 steps are launched one by one
        instead, behind 5 ms of queued replays that give the host its head start.  Returns microseconds per call of
        the median over the runs (`us`), the first run and the minimum, and the host-clock seconds of one more replay
        of the graph between two synchronizations."""
        stream = bench_stream
        if args.counters:
            with torch.cuda.stream(stream):
                for i in range(min(warmup, 3)):
                    calls[i % len(calls)]()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                n = min(steps, 8)
                t0 = time.perf_counter()
                e0.record()
                for i in range(n):
                    calls[i % len(calls)]()
                e1.record()
                torch.cuda.synchronize()
                wall = time.perf_counter() - t0
            us = e0.elapsed_time(e1) * 1e3 / n
            return dict(us=us, us_first=us, us_median=us, us_min=us, wall=wall * steps / n,
                        how="counter run: %d direct launches, no graph" % n)
        with torch.cuda.stream(stream):
            for i in range(max(warmup, 3)):
                calls[i % len(calls)]()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(steps):
                    calls[i % len(calls)]()
            for _ in range(settle_replays(steps)):
                graph.replay()
            torch.cuda.synchronize()

            def timed(lead, direct):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                for _ in range(lead):
                    graph.replay()
                e0.record()
                if direct:
                    for i in range(steps):
                        calls[i % len(calls)]()
                else:
                    graph.replay()
                e1.record()
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) * 1e3 / steps

            direct = direct_if_short and steps < 200
            lead = max(1, -(-500 // (steps * 15)))           # >= 0.5 ms of un-timed replays ahead of a timed one
            if direct:
                lead = max(1, int(5000.0 / (steps * timed(lead, False))) + 1)
            us = [timed(lead, direct) for _ in range(reps)]
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        return dict(us=statistics.median(us), us_first=us[0], us_median=statistics.median(us), us_min=min(us), wall=wall,
                    how="launched one by one behind queued graph replays" if direct else "one graph replay")

    def finish(name, t, algo, **extra):
        row = dict(name=name, us=t["us"], us_first=t["us_first"], us_median=t["us_median"], us_min=t["us_min"], bytes=algo,
                   gbps=algo / t["us"] / 1e3, frac=algo / t["us"] / 1e3 / HBM_PEAK_GBPS, wall=t["wall"], how=t["how"])
        row.update(extra)
        got = traffic_table.get(name)
        if isinstance(got, dict):
            # counted for one routing / one set of launch parameters: valid only for a run that has the same
            ok = got.get("active_experts") == extra.get("active_experts") if "active_experts" in got else True
            if "params" in got and list(got["params"]) != list(extra.get("params") or []):
                ok = False
            got = got["bytes"] if ok else None
        if got is not None:
            row["traffic"] = got
            row["traffic_over_algorithmic"] = got / algo
        return row

    def read_only_us(nbytes, steps, shapes=((512, 1024), (1024, 512), (256, 2048), (512, 512), (1024, 256))):
        """One launch that only reads `nbytes` (rotating copies, GeMV access pattern): best us per launch."""
        nbytes -= nbytes % 4096
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(copies_for(nbytes))]
        best = None
        for block, wgs in shapes:
            if (nbytes // 1024) % wgs:
                continue

            def mk(b):
                def call():
                    _lib.check(lib.mlk_stream_read(b.data_ptr(), nbytes, block, wgs, 0,
                                                   torch.cuda.current_stream().cuda_stream), "stream_read")
                return call
            t = run_graph([mk(b) for b in bufs], steps, 5, reps=3, direct_if_short=True)
            best = t["us_median"] if best is None else min(best, t["us_median"])
        return best

    # ------------------------------------------------------------------ CPU baselines
    def cpu_time(fn, budget_s=0.8, min_reps=3, max_reps=50):
        for _ in range(2):
            fn()
        reps, t0 = 0, time.perf_counter()
        while reps < min_reps or (time.perf_counter() - t0 < budget_s and reps < max_reps):
            fn()
            reps += 1
        return (time.perf_counter() - t0) / reps, reps

    def cpu_linear(n, k, m, kind, rows, native=False):
        """The reference's CPU-runnable path for one GeMV / GeMM configuration on the first `rows` weight rows:
        a library linear on the un-packed weights in the configuration's dtype; soft-FP8 weights are first
        widened and scaled per block in bf16 (done once, outside the timing, as the reference's scripts do);
        the native chain adds the view/permute pack and un-pack of the output."""
        if args.no_cpu:
            return None
        from oracle import gemm as ogemm
        rows = min(rows, n)
        g = torch.Generator().manual_seed(2025)
        dt = torch.bfloat16 if kind == 2 else DT[kind]
        if kind == 2:
            codes = (torch.randn((rows, k), generator=g) * 16).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
            w = ogemm.torch_path_softfp8_weight(codes, torch.ones(((rows + 127) // 128, (k + 127) // 128)))
        else:
            w = (torch.randn((rows, k), generator=g) * 0.02).to(dt)
        b = torch.randn((m, k), generator=g).to(dt)

        def fn():
            c = ogemm.torch_path_linear(w, b)
            if native:
                c_nat = ogemm.layout_c_of(c)
                c = c_nat.view(rows // 32, m // 16, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(m, rows)
            return c
        dt_s, reps = cpu_time(fn)
        sample_bytes = rows * k * (1 if kind == 2 else 2) + m * k * 2 + m * rows * 2
        return dict(value=round(sample_bytes / dt_s / 1e9, 3), unit="GB/s", us_scaled_to_full=round(dt_s * 1e6 * n / rows, 1),
                    cores=cores, kind="port",
                    sample="torch linear in %s on the first %d of %d un-packed weight rows, M=%d, %d reps, %.3f ms each; "
                           "host has %d logical CPUs" % (str(dt).replace("torch.", ""), rows, n, m, reps, dt_s * 1e3,
                                                          host_cpus))

    cpu_moe_w = {}

    def cpu_moe(T, slab=8):
        """The reference's dense torch MoE (all 8 experts on every token) on 1/slab of the intermediate size."""
        if args.no_cpu:
            return None
        from oracle import moe as omoe
        E, K, H, I = 8, 2, 4096, 14336 // slab
        g = torch.Generator().manual_seed(2025)
        if "w" not in cpu_moe_w:
            cpu_moe_w["w"] = ((torch.randn((E, 2 * I, H), generator=g) * 0.02).to(torch.bfloat16),
                              (torch.randn((E, H, I), generator=g) * 0.02).to(torch.bfloat16))
        w1, w2 = cpu_moe_w["w"]
        x = torch.randn((T, H), generator=g).to(torch.bfloat16)
        logits = torch.randn((T, E), generator=g).to(torch.bfloat16)
        dt_s, reps = cpu_time(lambda: omoe.torch_path_fused_moe(x, w1, w2, logits, K, renormalize=True),
                              budget_s=1.0, min_reps=2, max_reps=20)
        sample_bytes = E * 3 * I * H * 2 + 2 * T * H * 2 + T * E * 2
        return dict(value=round(sample_bytes / dt_s / 1e9, 3), unit="GB/s", us_scaled_to_full=round(dt_s * 1e6 * slab, 1),
                    cores=cores, kind="port",
                    sample="dense torch MoE in bf16 (softmax, top-2, renormalised, all 8 experts on every token) with "
                           "H=4096 and 1/%d of the intermediate size (I=%d), T=%d, %d reps, %.1f ms each; host has %d "
                           "logical CPUs" % (slab, I, T, reps, dt_s * 1e3, host_cpus))

    # ------------------------------------------------------------------ GPU cases
    def gemv_case(name, n, k, kind, steps, warmup, yardstick=False, cpu_rows=2048, unit_scales=False):
        xk = 1 if kind == 2 else kind
        wbytes = n * k * (1 if kind == 2 else 2)
        A = weights(n, k, kind, copies_for(wbytes))
        x = torch.randn((1, k), generator=gen, device=dev).to(DT[xk])
        y = torch.empty((1, n), dtype=DT[xk], device=dev)
        scale = None
        if kind == 2:
            scale = torch.ones(((n + 127) // 128, (k + 127) // 128), dtype=torch.float32, device=dev) if unit_scales \
                else block_scales(((n + 127) // 128, (k + 127) // 128))
        sel = {0: "gemv_fp16", 1: "gemv_bf16", 2: "gemv_soft_fp8"}[kind]
        block, kid, p1, p2 = arg_selector.gemv_guard(arg_selector.selector(sel).get_args((n, k)), n, k)

        def mk(a):
            def call():
                st = torch.cuda.current_stream().cuda_stream
                _lib.check(lib.mlk_gemv_layout_a(a.data_ptr(), x.data_ptr(), y.data_ptr(), 1, n, k, kind, xk, 1.0, 0,
                                                 0 if scale is None else scale.data_ptr(), block, kid, p1, p2, st),
                           "gemv")
            return call
        t = run_graph([mk(a) for a in A], steps, warmup, direct_if_short=True)
        algo = wbytes + (scale.numel() * 4 if scale is not None else 0) + k * 2 + n * 2
        extra = dict(params=[block, kid, p1, p2], copies=len(A))
        del A
        if yardstick and not args.counters:
            extra["read_only_us"] = read_only_us(wbytes, steps)
        if cpu_rows:
            extra["cpu_baseline"] = cpu_linear(n, k, 1, kind, cpu_rows)
        return finish(name, t, algo, **extra)

    def blas_yardstick(row, n, k, dt, m, steps, count):
        """torch.matmul (vendor BLAS) on `count` rotating un-packed copies of a weight matrix of the same shape."""
        W = [(torch.randn((n, k), generator=gen, device=dev) * 0.02).to(dt) for _ in range(count)]
        b = torch.randn((m, k), generator=gen, device=dev).to(dt)
        out = torch.empty((m, n), dtype=dt, device=dev)
        t = run_graph([(lambda w=w: torch.matmul(b, w.t(), out=out)) for w in W], steps, 3, reps=3, direct_if_short=True)
        row["blas_us"] = t["us_median"]
        row["blas_note"] = ("torch.matmul (vendor BLAS) on %d rotating un-packed %s weight matrices of the same shape"
                            % (count, str(dt).replace("torch.", "")))
        del W

    def gemm_case(name, n, k, kind, m, steps, warmup, native=False, copies=None, cpu_rows=2048, cpu=True, blas=False,
                  relayout=True):
        xk = 1 if kind == 2 else kind
        A = weights(n, k, kind, copies or copies_for(n * k * (1 if kind == 2 else 2)))
        b = torch.randn((m, k), generator=gen, device=dev).to(DT[xk])
        scale = block_scales((n // 128, k // 128)) if kind == 2 else None
        table = "layoutA_soft_fp8_gemm" if kind == 2 else ("layout_gemm" if native else "layoutA_gemm")
        kid, p1, p2, p3 = mlk.ops._gemm_guard(arg_selector.selector(table).get_args((n, m, k)), n)
        if native:
            b_in = mlk.layoutB(b)
            c = torch.empty((n // 32, m // 16, 4, 16, 8), dtype=DT[xk], device=dev)
            c_rm = torch.empty((m, n), dtype=DT[xk], device=dev)
        else:
            b_in = b
            c = torch.empty((m, n), dtype=DT[xk], device=dev)

        def mk(a):
            def call():
                st = torch.cuda.current_stream().cuda_stream
                ws_ptr, ws_len = 0, 0
                if p3 > 1:      # per-stream scratch of the K split (allocated by the warm-up calls, before the capture)
                    ws = mlk.ops._workspace(dev, lib.mlk_gemm_workspace_bytes(m, n, p1, p3), lib.mlk_gemm_counter_bytes(), st)
                    ws_ptr, ws_len = ws.data_ptr(), ws.numel()
                _lib.check(lib.mlk_gemm_layout_a(a.data_ptr(), b_in.data_ptr(), c.data_ptr(), m, n, k, kind, xk,
                                                 1 if native else 0, 1 if native else 0, 1.0, 0,
                                                 0 if scale is None else scale.data_ptr(), kid, p1, p2, p3, ws_ptr, ws_len,
                                                 st),
                           "gemm")
                if native and relayout:
                    _lib.check(lib.mlk_re_layout_c(c.data_ptr(), c_rm.data_ptr(), m, n, st), "reLayoutC")
            return call
        t = run_graph([mk(a) for a in A], steps, warmup, direct_if_short=True)
        algo = n * k * (1 if kind == 2 else 2) + (scale.numel() * 4 if scale is not None else 0) + m * k * 2 + m * n * 2
        if native and relayout:
            algo += 2 * m * n * 2
        row = finish(name, t, algo, params=[kid, p1, p2, p3], copies=len(A))
        if cpu:
            row["cpu_baseline"] = cpu_linear(n, k, m, kind, cpu_rows, native=native)
        if blas and kind != 2 and not args.no_blas:
            count = len(A)
            del A
            blas_yardstick(row, n, k, DT[kind], m, steps, count)
        return row

    mfma_only = {}

    def mfma_only_tflops(dt):
        """Matrix-core yardstick: a loop of nothing but v_mfma_f32_32x32x16 on operand values drawn like the
        benchmark's (weights 0.02 * N(0, 1), activations N(0, 1)), one workgroup of eight waves per CU, replayed
        like the cases.  The power limit, not the instruction rate, sets what the chip sustains on such values."""
        if dt not in mfma_only:
            a = (torch.randn((64 * 1024,), generator=gen, device=dev) * 0.02).to(dt)
            b = torch.randn((64 * 1024,), generator=gen, device=dev).to(dt)
            cus = torch.cuda.get_device_properties(dev).multi_processor_count
            iters = 4000

            def call():
                _lib.check(lib.mlk_mfma_probe(a.data_ptr(), b.data_ptr(), iters, cus, 0,
                                              torch.cuda.current_stream().cuda_stream), "mfma_probe")
            t = run_graph([call], 10, 3, reps=3, direct_if_short=True)
            mfma_only[dt] = cus * 8 * iters * 16 * 32768.0 / t["us_median"] / 1e6
        return mfma_only[dt]

    def panel_case(name, n, k, kind, m, steps):
        """Prefill-sized token counts: bound by the matrix cores (or by the weight stream up to ~300 tokens).
        The vendor BLAS on an un-packed 16-bit copy of the same shape is timed beside it, and the rate of a loop
        that only issues the same MFMA instruction on like-valued operands (`mfma_only_tflops`)."""
        row = gemm_case(name, n, k, kind, m, steps, 3, copies=2, cpu=False)
        flops = 2.0 * m * n * k
        row["tflops"] = flops / row["us"] / 1e6
        row["mfma_frac"] = row["tflops"] / MFMA_PEAK_TFLOPS
        if not args.counters:
            row["mfma_only_tflops"] = mfma_only_tflops(torch.bfloat16)
            row["frac_of_mfma_only"] = row["tflops"] / row["mfma_only_tflops"]
        row["bound"] = "mfma" if flops / (MFMA_PEAK_TFLOPS * 1e6) > row["bytes"] / (HBM_PEAK_GBPS * 1e3) else "hbm"
        dt = torch.bfloat16 if kind == 2 else DT[kind]
        W = [(torch.randn((n, k), generator=gen, device=dev) * 0.02).to(dt) for _ in range(2)]
        b = torch.randn((m, k), generator=gen, device=dev).to(dt)
        out = torch.empty((m, n), dtype=dt, device=dev)
        t = run_graph([(lambda w=w: torch.matmul(b, w.t(), out=out)) for w in W], steps, 3, reps=3, direct_if_short=True)
        row["blas_us"] = t["us_median"]
        row["blas_tflops"] = flops / t["us_median"] / 1e6
        row["blas_note"] = "torch.matmul (vendor BLAS) on un-packed %s weights of the same shape" % str(dt).replace("torch.", "")
        return row

    moe_w = {}

    def moe_case(name, T, fp8, steps, warmup):
        E, K, H, I = 8, 2, 4096, 14336
        key = "fp8" if fp8 else "bf16"
        if key not in moe_w:
            moe_w.clear()
            torch.cuda.empty_cache()
            if fp8:
                w1 = (torch.randn((E, 2 * I, H), generator=gen, device=dev) * 16).clamp_(-448, 448)
                w1 = w1.to(torch.float8_e4m3fn).view(torch.uint8)
                w2 = (torch.randn((E, H, I), generator=gen, device=dev) * 16).clamp_(-448, 448)
                w2 = w2.to(torch.float8_e4m3fn).view(torch.uint8)
                s1 = block_scales((E, 2 * I // 128, H // 128))
                s2 = block_scales((E, H // 128, I // 128))
                moe_w[key] = (w1, w2, s1, s2)
            else:
                w1 = (torch.randn((E, 2 * I, H), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
                w2 = (torch.randn((E, H, I), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
                moe_w[key] = (w1, w2, None, None)
        w1, w2, s1, s2 = moe_w[key]
        x = torch.randn((T, H), generator=gen, device=dev).to(torch.bfloat16)
        logits = torch.randn((T, E), generator=gen, device=dev).to(torch.bfloat16)
        kw = dict(w1_scale=s1, w2_scale=s2, block_shape=[128, 128], soft_fp8=True) if fp8 else {}

        def call():
            return fused_moe(x, w1, w2, logits, K, True, **kw)
        y = call()
        ids = torch.topk(torch.softmax(logits.float(), dim=-1), K, dim=-1).indices
        e_act = int(torch.unique(ids).numel())
        t = run_graph([call], steps, warmup)
        wbytes = 1 if fp8 else 2
        algo = e_act * 3 * I * H * wbytes + 2 * T * H * 2 + T * E * 2
        if fp8:
            algo += e_act * 3 * (I // 128) * (H // 128) * 4
        del y
        roof = algo / HBM_PEAK_GBPS / 1e3
        row = finish(name, t, algo, active_experts=e_act, roofline_us=roof, ratio_to_roofline=t["us"] / roof)
        base = cpu_moe(T)
        if base is not None and fp8:
            base = dict(base, sample=base["sample"] + "; the reference's CPU path for soft-FP8 weights is the same loop "
                                                      "on weights widened to bf16 beforehand")
        row["cpu_baseline"] = base
        return row

    def moe_next_case(name, T, steps, warmup):
        """The routing configuration the reference's own router is written for (256 experts in 8 groups, 4 groups
        kept, top-8, sigmoid scores with a selection bias) on expert matrices of H = 7168, I = 2048."""
        E, K, H, I = 256, 8, 7168, 2048
        if "next" not in moe_w:
            moe_w.clear()
            torch.cuda.empty_cache()
            w1 = torch.empty((E, 2 * I, H), dtype=torch.bfloat16, device=dev)
            w2 = torch.empty((E, H, I), dtype=torch.bfloat16, device=dev)
            for e0 in range(0, E, 16):
                w1[e0:e0 + 16] = (torch.randn((16, 2 * I, H), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
                w2[e0:e0 + 16] = (torch.randn((16, H, I), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
            moe_w["next"] = (w1, w2, None, None)
        w1, w2, _, _ = moe_w["next"]
        x = torch.randn((T, H), generator=gen, device=dev).to(torch.bfloat16)
        logits = torch.randn((T, E), generator=gen, device=dev).to(torch.bfloat16)
        bias = (torch.randn((E,), generator=gen, device=dev) * 0.05).abs().to(torch.bfloat16)

        def call():
            return fused_moe(x, w1, w2, logits, K, True, use_grouped_topk=True, num_expert_group=8, topk_group=4,
                             gating_bias=bias, score_func="sigmoid")
        y = call()
        ids = torch.empty((T, K), dtype=torch.int32, device=dev)
        wts = torch.empty((T, K), dtype=torch.bfloat16, device=dev)
        mlk.fused_routing_gate(logits, 1, T, H, 8, 4, ids, wts, K, bias)
        e_act = int(torch.unique(ids).numel())
        t = run_graph([call], steps, warmup)
        algo = e_act * 3 * I * H * 2 + 2 * T * H * 2 + T * E * 2
        del y
        roof = algo / HBM_PEAK_GBPS / 1e3
        return finish(name, t, algo, active_experts=e_act, roofline_us=roof, ratio_to_roofline=t["us"] / roof)

    def relayout_case(name, which, steps):
        """The relayout / repack kernels: read + write of the tensor."""
        st_of = lambda: torch.cuda.current_stream().cuda_stream     # noqa: E731
        if which == "fp8_weight_repack":
            n, k = 28672, 8192
            src = [torch.randint(0, 255, (n, k), dtype=torch.uint8, device=dev) for _ in range(2)]
            dst = torch.empty_like(src[0])
            calls = [(lambda a=a: _lib.check(lib.mlk_fp8_weight_repack(a.data_ptr(), dst.data_ptr(), a.numel(), st_of()),
                                             "repack")) for a in src]
            algo = 2 * n * k
        elif which == "layoutB":
            m, k = 32, 8192
            src = [torch.randn((m, k), generator=gen, device=dev).to(torch.bfloat16) for _ in range(4)]
            dst = torch.empty((k // 32, m // 16, 4, 16, 8), dtype=torch.bfloat16, device=dev)
            calls = [(lambda a=a: _lib.check(lib.mlk_layout_b(a.data_ptr(), dst.data_ptr(), m, k, st_of()), "layoutB"))
                     for a in src]
            algo = 2 * m * k * 2
        else:
            m, n = 32, 8192
            src = [torch.randn((n // 32, m // 16, 4, 16, 8), generator=gen, device=dev).to(torch.bfloat16) for _ in range(4)]
            dst = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            calls = [(lambda a=a: _lib.check(lib.mlk_re_layout_c(a.data_ptr(), dst.data_ptr(), m, n, st_of()), "reLayoutC"))
                     for a in src]
            algo = 2 * m * n * 2
        t = run_graph(calls, steps, 3)
        return finish(name, t, algo)

    def pack_case(name, e, n, k, steps):
        """The device step of the checkpoint converter: row-major expert matrices -> layout-A (read + write)."""
        src = [(torch.randn((e, n, k), generator=gen, device=dev) * 0.02).to(torch.bfloat16) for _ in range(2)]
        dst = torch.empty((e, n // 16, k // 8, 16, 8), dtype=torch.bfloat16, device=dev)

        def mk(a):
            def call():
                _lib.check(lib.mlk_pack_layout_a(a.data_ptr(), dst.data_ptr(), e, n, k, 2,
                                                 torch.cuda.current_stream().cuda_stream), "pack_layout_a")
            return call
        t = run_graph([mk(a) for a in src], steps, 3)
        return finish(name, t, 2 * e * n * k * 2)

    def eager_case(name, make, calls=1000, warm=1000):
        """The public Python API called eagerly, the way the reference's scripts time it
        (benchmark_and_test/gemv_benchmark.py:62-73, benchmark_muxi_moe.py:40-49): `warm` calls, a synchronization,
        then the wall clock around `calls` back-to-back calls with one synchronization at the end.  Host work per call
        (argument checks, table lookup, output allocation, the ctypes call, the launch) is part of it; `graph_us`
        beside it is the same configuration's device time per call from the graph-replay timing.  `make` returns
        (call, name of the per_config line that holds the device time, or None for the headline)."""
        call, ref = make()
        with torch.cuda.stream(bench_stream):
            for _ in range(warm):
                call()
            torch.cuda.synchronize()
            runs = []
            for _ in range(3):
                t0 = time.perf_counter()
                for _ in range(calls):
                    call()
                torch.cuda.synchronize()
                runs.append((time.perf_counter() - t0) * 1e6 / calls)
            # host cost alone: the same calls with nothing waiting on the device (queue drained first, clock stopped
            # before the synchronization)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(200):
                call()
            host = (time.perf_counter() - t0) * 1e6 / 200
            torch.cuda.synchronize()
        row = dict(name=name, eager_us=round(statistics.median(runs), 3), eager_us_min=round(min(runs), 3),
                   host_us_per_call=round(host, 3), calls=calls,
                   how="wall clock around %d eager calls of the public Python API, synchronized at both ends; median of 3" % calls)
        dev = head["us"] if ref is None else next((r["us"] for r in per_config if r["name"] == ref), None)
        if dev is not None:
            row["graph_us"] = round(dev, 3)
            row["eager_over_graph"] = round(row["eager_us"] / dev, 3)
        return row

    def eager_gemv(n, k, kind, ref):
        def make():
            xk = 1 if kind == 2 else kind
            a = weights(n, k, kind, copies_for(n * k * (1 if kind == 2 else 2)))
            x = torch.randn((1, k), generator=gen, device=dev).to(DT[xk])
            scale = block_scales(((n + 127) // 128, (k + 127) // 128)) if kind == 2 else None
            state = {"i": 0}

            def call():
                state["i"] = (state["i"] + 1) % len(a)
                return mlk.gemv_layoutA(a[state["i"]], x, scale_matrix=scale)
            return call, ref
        return make

    def eager_gemm(n, k, kind, m, ref):
        def make():
            a = weights(n, k, kind, copies_for(n * k * 2))
            b = torch.randn((m, k), generator=gen, device=dev).to(DT[kind])
            state = {"i": 0}

            def call():
                state["i"] = (state["i"] + 1) % len(a)
                return mlk.gemm_layoutA(a[state["i"]], b)
            return call, ref
        return make

    def eager_moe(T, fp8, ref):
        def make():
            E, K, H, I = 8, 2, 4096, 14336
            key = "fp8" if fp8 else "bf16"
            if key not in moe_w:
                moe_case("(weights for the eager line)", T, fp8, 2, 1)     # draws and caches the expert weights
            w1, w2, s1, s2 = moe_w[key]
            x = torch.randn((T, H), generator=gen, device=dev).to(torch.bfloat16)
            logits = torch.randn((T, E), generator=gen, device=dev).to(torch.bfloat16)
            kw = dict(w1_scale=s1, w2_scale=s2, block_shape=[128, 128], soft_fp8=True) if fp8 else {}
            return (lambda: fused_moe(x, w1, w2, logits, K, True, **kw)), ref
        return make

    if args.calibrate_copy:
        src = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):   # the repack kernel as a plain copy of known size: 16 bytes in and 16 bytes out per thread
            _lib.check(lib.mlk_fp8_weight_repack(src.data_ptr(), dst.data_ptr(), src.numel(),
                                                 torch.cuda.current_stream().cuda_stream), "copy")
        torch.cuda.synchronize()
        del src, dst

    def read_ceiling(steps, nbytes=256 << 20, copies=4, shapes=((512, 2048), (1024, 1024), (256, 4096))):
        """Pure streaming read of `copies` rotating buffers of `nbytes` with the GeMV access pattern: best GB/s."""
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(copies)]
        best = 0.0
        for block, wgs in shapes:
            def mk(b):
                def call():
                    _lib.check(lib.mlk_stream_read(b.data_ptr(), nbytes, block, wgs, 0,
                                                   torch.cuda.current_stream().cuda_stream), "stream_read")
                return call
            t = run_graph([mk(b) for b in bufs], steps, 5, reps=3, direct_if_short=True)
            best = max(best, nbytes / t["us_median"] / 1e3)
        return best

    # ------------------------------------------------------------ headline
    N, K_, M = 11008, 4096, 16
    HEAD = "C2 fp16 gemm_layoutA 11008x4096 M=16"
    head_wanted = not args.counters or (args.case is not None and any(part and part in HEAD for part in args.case.split(",")))
    if head_wanted:
        head = gemm_case(HEAD, N, K_, 0, M, args.steps, args.warmup, blas=not args.quick, cpu=not args.counters)
    else:       # a counter run on other cases: no headline launches among the profiled dispatches
        head = dict(name=HEAD, us=0.0, us_first=0.0, us_median=0.0, us_min=0.0,
                    gbps=0.0, frac=0.0, wall=0.0, how="not run (--counters without the headline in --case)",
                    bytes=N * K_ * 2 + M * K_ * 2 + M * N * 2, copies=0, params=None)
    per_config = []
    eager = []

    def add(case, name, *a, **kw):
        """Run one per-configuration case unless --case asks for others only."""
        if args.case is None or any(part and part in name for part in args.case.split(",")):
            per_config.append(case(name, *a, **kw))
    ceiling = None
    resident = None
    same_size = None
    def add_eager(name, make, **kw):
        if not args.no_eager and (args.case is None or any(part and part in name for part in args.case.split(","))):
            eager.append(eager_case(name, make, **kw))
    if not args.quick:
        if not args.counters:
            one = gemm_case("headline workload, one weight copy (stays in the 256 MiB Infinity Cache)", N, K_, 0, M,
                            args.steps, args.warmup, copies=1, cpu=False)
            resident = {"us_per_call": round(one["us"], 3), "gbps": round(one["gbps"], 1),
                        "what": "same kernel and launch parameters on a single 86 MiB weight copy: the stream comes from "
                                "the Infinity Cache, not HBM; reported for information, never the headline"}
            ceiling = round(read_ceiling(40), 1)
            # the same yardstick at the headline's size: one launch that only reads as many bytes as the weights hold
            same_size = read_only_us(N * K_ * 2, args.steps)
        short = max(20, min(args.steps, args.case_steps)) if not args.counters else args.steps
        add(gemv_case, "C1 bf16 gemv 4096x4096", 4096, 4096, 1, short, 10, yardstick=True, cpu_rows=4096)
        # the same GeMV on larger squares (the target speaks of N = K >= 4096), each with its own read-only yardstick
        add(gemv_case, "C1+ bf16 gemv 8192x8192", 8192, 8192, 1, short, 10, yardstick=True, cpu_rows=0)
        add(gemv_case, "C1+ bf16 gemv 16384x16384", 16384, 16384, 1, max(20, short // 4), 10, yardstick=True, cpu_rows=0)
        add_eager("eager: gemv_layoutA bf16 4096x4096", eager_gemv(4096, 4096, 1, "C1 bf16 gemv 4096x4096"))
        add_eager("eager: gemm_layoutA fp16 11008x4096 M=16", eager_gemm(N, K_, 0, M, None))
        for m in (1, 8, 32, 64):
            add(gemm_case, "C2 fp16 gemm_layoutA 11008x4096 M=%d" % m, N, K_, 0, m, short, 10, blas=True)
        add(gemv_case, "C2 fp16 gemv 11008x4096", N, K_, 0, short, 10)
        add(gemv_case, "C3 soft-fp8 gemv 28672x8192", 28672, 8192, 2, short, 10, yardstick=True, cpu_rows=1024)
        add(gemv_case, "C3 soft-fp8 gemv 28672x8192, power-of-two block scales", 28672, 8192, 2, short, 10, cpu_rows=0,
            unit_scales=True)
        for m in (4, 16):
            add(gemm_case, "C3 soft-fp8 gemm_layoutA 28672x8192 M=%d" % m, 28672, 8192, 2, m, short, 10, cpu_rows=1024)
        add_eager("eager: gemv_layoutA soft-fp8 28672x8192", eager_gemv(28672, 8192, 2, "C3 soft-fp8 gemv 28672x8192"))
        add(gemm_case, "C4 bf16 gemm_layoutABC+reLayoutC 8192x8192 M=32", 8192, 8192, 1, 32, short, 10, native=True,
            cpu_rows=1024, blas=True)
        # the product alone, output left in layout-C as a following native-layout product would take it
        add(gemm_case, "C4 bf16 gemm_layoutABC 8192x8192 M=32, output kept in layout-C", 8192, 8192, 1, 32, short, 10,
            native=True, cpu=False, relayout=False)
        add(relayout_case, "C4 layoutB bf16 [32, 8192]", "layoutB", short)
        add(relayout_case, "C4 reLayoutC bf16 [32, 8192]", "reLayoutC", short)
        add(relayout_case, "C3 fp8_weight_repack 28672x8192", "fp8_weight_repack", 10)
        for T in (1, 16, 64, 256):
            add(moe_case, "C5 bf16 fused_moe T=%d" % T, T, False, args.moe_steps, 5)
        for T in (1, 16):
            add_eager("eager: fused_moe bf16 T=%d" % T, eager_moe(T, False, "C5 bf16 fused_moe T=%d" % T), calls=300, warm=100)
        for T in (1, 16, 64, 256):
            add(moe_case, "C5 soft-fp8 fused_moe T=%d" % T, T, True, args.moe_steps, 5)
        for T in (1, 16):
            add_eager("eager: fused_moe soft-fp8 T=%d" % T, eager_moe(T, True, "C5 soft-fp8 fused_moe T=%d" % T), calls=300,
                      warm=100)
        for T in (1, 16):
            add(moe_next_case, "next: grouped-routing MoE E=256 top-8 H=7168 I=2048 bf16 T=%d" % T, T, args.moe_steps, 5)
        moe_w.clear()
        torch.cuda.empty_cache()
        for m in (128, 256, 1024, 4096):
            add(panel_case, "next: prefill gemm_layoutA fp16 11008x4096 M=%d" % m, N, K_, 0, m, 20)
        add(panel_case, "next: prefill gemm_layoutA bf16 8192x8192 M=4096", 8192, 8192, 1, 4096, 10)
        add(panel_case, "next: prefill gemm_layoutA soft-fp8 28672x8192 M=1024", 28672, 8192, 2, 1024, 10)
        torch.cuda.empty_cache()
        add(pack_case, "next: checkpoint conversion, pack_layout_a bf16 [8, 28672, 4096]", 8, 28672, 4096, 10)
        torch.cuda.empty_cache()
        for row in per_config:
            row.pop("wall", None)
            row.pop("how", None)
            for key in ("us", "us_first", "us_median", "us_min", "gbps", "frac", "roofline_us", "ratio_to_roofline", "tflops",
                        "mfma_frac", "read_only_us", "blas_us", "blas_tflops", "traffic_over_algorithmic",
                        "mfma_only_tflops", "frac_of_mfma_only"):
                if row.get(key) is not None:
                    row[key] = round(row[key], 4)

    line = {
        "metric": "achieved GB/s of algorithmic bytes per call (us/call and % of HBM peak alongside)",
        "value": round(head["gbps"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["wall"] * 1e3 / args.steps, 6),
        "us_per_call": round(head["us"], 3),
        "us_per_call_first_of_%d_replays" % TIMED_REPLAYS: round(head["us_first"], 3),
        "us_per_call_median_of_%d_replays" % TIMED_REPLAYS: round(head["us_median"], 3),
        "us_per_call_min_of_%d_replays" % TIMED_REPLAYS: round(head["us_min"], 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": head["name"], "weights": "fp16 N(0,0.02) in layout-A, %d rotating copies" % head["copies"],
                   "activations": "fp16 N(0,1) row-major [16, 4096]",
                   "untimed_graph_replays_before_timing": settle_replays(args.steps),
                   "timed_calls": head["how"],
                   "launch_params": head["params"],
                   "algorithmic_bytes": head["bytes"]},
        "roofline": {"bound": "hbm", "achieved": round(head["gbps"], 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(head["frac"], 4), "traffic": head.get("traffic")},
        "hbm_read_ceiling": None if ceiling is None else {
            "value": ceiling, "unit": "GB/s",
            "what": "pure streaming read (mlk_stream_read, 256 MiB x 4 rotating buffers) measured in this run",
            "us_for_one_launch_reading_the_headline_weights": round(same_size, 3)},
        "infinity_cache_resident": resident,
        "vendor_blas": None if head.get("blas_us") is None else {
            "us_per_call": round(head["blas_us"], 3), "what": head["blas_note"] + ", same token count, same graph-replay timing"},
        "cpu_baseline": head.get("cpu_baseline"),
        "eager_calls": eager,
        "per_config": per_config,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
