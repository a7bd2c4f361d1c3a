"""Offline launch-parameter scan for gfx950: brute-forces the `_wapper` entry points over the
parameter grid of each kernel, keeps the fastest configuration that passes a correctness gate and
writes csv rows the selectors can parse.

Counterpart of the reference's eight scan scripts (kernel_args_scan/gemv_kernel_args_scan.py:135-165,
gemv_kernel_args_scan_sf8.py, gemm_kernel_args_scan_kernel_all*.py): same idea (time every
configuration through the wapper, gate on the difference to an expected product, keep the best, emit
`m,k,...` / `m,n,k,...` rows), with the gfx950 kernels' own parameter grids.

    python -m muxi_native_layout_kernels_amd.kernel_args_scan.scan gemv_bf16 --shapes 4096x4096,28672x8192
    python -m muxi_native_layout_kernels_amd.kernel_args_scan.scan layoutA_gemm --shapes 11008x4096 --tokens 1,8,16,32,64
    python -m muxi_native_layout_kernels_amd.kernel_args_scan.scan all --update

Tables: gemv_fp16, gemv_bf16, gemv_soft_fp8, layoutA_gemm, layoutA_soft_fp8_gemm, continuous_gemm, layout_gemm.
`--update` appends the rows to the packaged csv (later rows win on lookup); without it they go to
`<table>_scan_best_args.csv` in the current directory.

Timing: each configuration is captured `--iters` times into one HIP graph over rotating weight
copies that together exceed the Infinity Cache, and timed with HIP events.
"""
import argparse
import os
import sys

import torch

from .. import ops, arg_selector

GEMV_TABLES = {"gemv_fp16": torch.float16, "gemv_bf16": torch.bfloat16, "gemv_soft_fp8": None}
GEMM_TABLES = {"layoutA_gemm": ("rowmajor", torch.float16), "layoutA_soft_fp8_gemm": ("fp8", torch.bfloat16),
               "continuous_gemm": ("continuous", torch.bfloat16), "layout_gemm": ("native", torch.bfloat16)}
# weight shapes (rows x K): the benchmark configurations, then the model lists the reference's scripts scan
# (benchmark_and_test/gemv_benchmark.py:122-137): Llama2-7B, Qwen2-7B, DeepSeek-R1
BENCH_16BIT = [(4096, 4096), (11008, 4096), (8192, 8192), (28672, 4096), (4096, 14336)]
BENCH_FP8 = [(28672, 8192), (4096, 4096), (8192, 8192)]
LLAMA2_7B = [(32000, 4096), (12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]
QWEN2_7B = [(37888, 3584), (4608, 3584), (3584, 3584), (3584, 18944)]
DEEPSEEK_R1 = [(2112, 7168), (3072, 1536), (7168, 2048), (7168, 256), (512, 7168), (4608, 7168), (7168, 2304)]
MODEL_SHAPES = LLAMA2_7B + QWEN2_7B + DEEPSEEK_R1


def _unique(shapes):
    return list(dict.fromkeys(shapes))


DEFAULT_SHAPES = {
    "gemv_fp16": _unique([(11008, 4096), (4096, 4096), (4096, 11008)] + MODEL_SHAPES),
    "gemv_bf16": _unique(BENCH_16BIT + [(28672, 8192)] + MODEL_SHAPES),
    "gemv_soft_fp8": _unique(BENCH_FP8 + MODEL_SHAPES),
    "layoutA_gemm": _unique([(11008, 4096), (4096, 4096), (4096, 11008)] + MODEL_SHAPES),
    "layoutA_soft_fp8_gemm": _unique(BENCH_FP8[:2] + MODEL_SHAPES),
    "continuous_gemm": _unique([(8192, 8192), (11008, 4096)] + MODEL_SHAPES),
    "layout_gemm": _unique([(8192, 8192), (11008, 4096)] + MODEL_SHAPES),
}
# Weight shapes (rows, K) that the reference's packaged tables hold rows for (the keys of
# /root/reference/muxi_layout_kernels/layout_gemv_dispatch_arg.csv and layout_gemv_bf16_dispatch_arg.csv (the same
# 90 shapes), layout_gemv_soft_fp8_dispatch_arg.csv, layoutA_gemm_dispatch_arg.csv,
# layoutA_Soft_Fp8_gemm_dispatch_arg.csv, continuous_gemm_dispatch_arg.csv and layout_gemm_dispatch_arg.csv):
# `--shape-set tables` scans these, so that a model served from the reference's tables finds a scanned row here too.
_TABLE_GEMV_16BIT = [
    (16, 4096), (16, 6144), (128, 5120), (512, 7168), (512, 8192), (896, 5120), (1024, 5120), (1024, 6144),
    (1280, 5120), (1280, 8192), (1536, 4096), (2112, 7168), (2560, 8192), (2752, 8192), (3072, 1536), (3072,
    8192), (3200, 5120), (3584, 3584), (3584, 18944), (4000, 6144), (4000, 8192), (4096, 1024), (4096, 4096),
    (4096, 6144), (4096, 8192), (4096, 11008), (4096, 13696), (4608, 3584), (4608, 4096), (4608, 7168), (4992,
    6656), (5120, 640), (5120, 1024), (5120, 3200), (5120, 3424), (5120, 3456), (5120, 5120), (5120, 8192),
    (5120, 13824), (5120, 25600), (5504, 8192), (6144, 768), (6144, 2048), (6144, 8192), (6400, 5120), (6656,
    1664), (6656, 4480), (6848, 5120), (6912, 5120), (7168, 256), (7168, 2048), (7168, 2304), (7168, 8192),
    (8000, 6656), (8000, 8192), (8192, 1024), (8192, 2048), (8192, 2752), (8192, 3584), (8192, 4096), (8192,
    5120), (8192, 5504), (8192, 7168), (8192, 7392), (8192, 14336), (8960, 6656), (10240, 5120), (11008, 4096),
    (11008, 8192), (12288, 4096), (13696, 4096), (13824, 5120), (14336, 8192), (14784, 8192), (15360, 5120),
    (16032, 8192), (19008, 5120), (22016, 4096), (25600, 5120), (27392, 4096), (27648, 5120), (28672, 8192),
    (32000, 4096), (32000, 5120), (32064, 8192), (37888, 3584), (38016, 8192), (51200, 5120), (65024, 4096),
    (125696, 4096)]
_TABLE_GEMV_FP8 = [
    (128, 5120), (512, 7168), (512, 8192), (1024, 5120), (1280, 5120), (2112, 7168), (3072, 1536), (3200, 5120),
    (4096, 8192), (4608, 7168), (5120, 1024), (5120, 3200), (5120, 5120), (5120, 8192), (5120, 25600), (5120,
    27648), (6400, 5120), (7168, 256), (7168, 2048), (7168, 2304), (7168, 5120), (8192, 4096), (8192, 5120),
    (8192, 14336), (10240, 5120), (14336, 8192), (25600, 5120), (28672, 8192), (51200, 5120), (55296, 5120)]
_TABLE_LAYOUTA_GEMM = [
    (128, 5120), (512, 7168), (512, 8192), (896, 5120), (1024, 5120), (1280, 5120), (2112, 7168), (3072, 1536),
    (3200, 5120), (4096, 8192), (4608, 7168), (5120, 640), (5120, 1024), (5120, 3200), (5120, 3456), (5120,
    8192), (5120, 25600), (6400, 5120), (6912, 5120), (7168, 256), (7168, 2048), (7168, 2304), (8192, 4096),
    (8192, 5120), (8192, 14336), (10240, 5120), (14336, 8192), (25600, 5120), (28672, 8192), (51200, 5120)]
_TABLE_LAYOUTA_FP8_GEMM = [
    (128, 5120), (512, 7168), (512, 8192), (1024, 5120), (1280, 5120), (3072, 1536), (3200, 5120), (4096, 8192),
    (4608, 7168), (5120, 1024), (5120, 3200), (5120, 5120), (5120, 8192), (5120, 25600), (5120, 27648), (6400,
    5120), (7168, 256), (7168, 2048), (7168, 2304), (7168, 5120), (8192, 4096), (8192, 5120), (8192, 14336),
    (10240, 5120), (14336, 8192), (25600, 5120), (28672, 8192), (51200, 5120), (55296, 5120)]
_TABLE_CONTINUOUS_GEMM = [
    (128, 5120), (512, 8192), (896, 5120), (1024, 5120), (1280, 5120), (3072, 1536), (3200, 5120), (3584, 3584),
    (3584, 18944), (4096, 8192), (4608, 3584), (4608, 7168), (5120, 640), (5120, 1024), (5120, 3200), (5120,
    3456), (5120, 8192), (5120, 25600), (6400, 5120), (6912, 5120), (7168, 256), (7168, 2048), (7168, 2304),
    (8192, 4096), (8192, 5120), (8192, 14336), (10240, 5120), (14336, 8192), (25600, 5120), (28672, 8192),
    (37888, 3584), (51200, 5120)]
_TABLE_LAYOUT_GEMM = [
    (128, 4096), (128, 5120), (128, 6144), (512, 7168), (512, 8192), (896, 5120), (1024, 5120), (1024, 6144),
    (1280, 5120), (1280, 8192), (1536, 4096), (2560, 8192), (2816, 8192), (3072, 1536), (3072, 8192), (3200,
    5120), (3584, 3584), (3584, 18944), (4096, 1024), (4096, 4096), (4096, 6144), (4096, 8192), (4096, 11008),
    (4096, 13696), (4608, 3584), (4608, 4096), (4608, 7168), (4992, 6656), (5120, 640), (5120, 1024), (5120,
    3200), (5120, 3456), (5120, 5120), (5120, 8192), (5120, 13824), (5120, 25600), (5504, 8192), (6144, 768),
    (6144, 8192), (6400, 5120), (6656, 1664), (6656, 4480), (6912, 5120), (7168, 256), (7168, 2048), (7168,
    2304), (7168, 8192), (8064, 6656), (8064, 8192), (8192, 1024), (8192, 2048), (8192, 2816), (8192, 3584),
    (8192, 4096), (8192, 5120), (8192, 5504), (8192, 7168), (8192, 7424), (8192, 14336), (8960, 6656), (10240,
    5120), (11008, 4096), (11008, 8192), (12288, 4096), (13696, 4096), (13824, 5120), (14336, 8192), (14848,
    8192), (15360, 5120), (16128, 8192), (19072, 5120), (22016, 4096), (25600, 5120), (27392, 4096), (27648,
    5120), (28672, 8192), (32000, 4096), (32000, 5120), (32128, 8192), (37888, 3584), (38016, 8192), (51200,
    5120), (65024, 4096), (125696, 4096)]
TABLE_SHAPES = {
    "gemv_fp16": _TABLE_GEMV_16BIT, "gemv_bf16": _TABLE_GEMV_16BIT, "gemv_soft_fp8": _TABLE_GEMV_FP8,
    "layoutA_gemm": _TABLE_LAYOUTA_GEMM, "layoutA_soft_fp8_gemm": _TABLE_LAYOUTA_FP8_GEMM,
    "continuous_gemm": _TABLE_CONTINUOUS_GEMM, "layout_gemm": _TABLE_LAYOUT_GEMM,
}
DEFAULT_TOKENS = {"layoutA_gemm": [1, 8, 16, 32, 48, 64], "layoutA_soft_fp8_gemm": [1, 4, 16, 32, 64],
                  "continuous_gemm": [16, 32, 64], "layout_gemm": [16, 32, 64]}
MALL_BYTES = 256 << 20


def _time_graph(calls, iters):
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for c in calls[:2]:
            c()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(iters):
                calls[i % len(calls)]()
        # The capture leaves the GPU idle and the first replays after an idle period run several percent
        # below the steady state, so replay un-timed for about 10 ms first, then time back-to-back replays.
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        for _ in range(max(1, int(10.0 / max(e0.elapsed_time(e1), 0.05)))):
            graph.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (3 * iters)


def _weights(n, k, dtype, fp8, count, gen):
    out = []
    for _ in range(count):
        w = torch.randn((n, k), generator=gen, device="cuda")
        if fp8:
            out.append((w * 16).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8))
        else:
            out.append((w * 0.02).to(dtype))
    return out


def _block_scales(rows, cols, gen):
    """fp32 block scales of soft-FP8 weights with arbitrary values (the general widening path; scales that are all
    powers of two would take a cheaper one and tune the tables for a special case)."""
    return torch.rand((rows, cols), generator=gen, device="cuda") * 0.02 + 0.001


def _scaled(codes, scale):
    """Value of soft-FP8 weights as the kernels widen them: e4m3 code times the fp32 scale of its 128 x 128 block,
    low 16 bits dropped (a bf16 by truncation)."""
    n, k = codes.shape
    full = scale.repeat_interleave(128, 0)[:n].repeat_interleave(128, 1)[:, :k]
    wide = codes.view(torch.float8_e4m3fn).float() * full
    return (wide.view(torch.int32) & -65536).view(torch.float32)


def _copies(nbytes):
    return int(max(2, min(16, (3 * MALL_BYTES + nbytes - 1) // nbytes)))


GATE_FAILURES = []      # configurations that ran and gave a wrong result: a bug to report, not a slow candidate


def _gate(got, want, what=None):
    """True when `got` matches the fp32 product within rtol = atol = 1e-2.  A configuration that ran but fails is
    named on stderr and remembered: main() exits non-zero if there was any, so a kernel path that computes wrong
    results for some shape shows up instead of silently dropping out of the tables."""
    err = (got.float() - want).abs()
    ok = bool((err <= 1e-2 + 1e-2 * want.abs()).all())
    if not ok and what is not None:
        GATE_FAILURES.append(what)
        print("WRONG RESULT (max error %g): %s" % (float(err.max()), what), file=sys.stderr, flush=True)
    return ok


def scan_gemv(table, shapes, iters, progress=None):
    dtype = GEMV_TABLES[table]
    fp8 = dtype is None
    xdt = torch.bfloat16 if fp8 else dtype
    gen = torch.Generator(device="cuda").manual_seed(2025)
    rows = []
    for n, k in shapes:
        plain = _weights(n, k, xdt, fp8, _copies(n * k * (1 if fp8 else 2)), gen)
        packed = [ops.pack_layout_a(w) for w in plain]
        x = torch.randn((1, k), generator=gen, device="cuda").to(xdt)
        scale = _block_scales((n + 127) // 128, (k + 127) // 128, gen) if fp8 else None
        w0 = _scaled(plain[0], scale) if fp8 else plain[0].float()
        want = x.float() @ w0.t()
        best = None
        # kernel 1: (threads, row groups per workgroup, loads in flight); kernels 2 and 3 (soft-FP8 only):
        # (threads, workgroups per CU, loads in flight)
        grid = [(block, 1, p1, p2) for block in (256, 512, 1024) for p1 in (1, 2, 4) for p2 in (2, 4, 6, 8)
                if (block // 64) % p1 == 0 and (n // 16) % p1 == 0]
        grid += [(block, kid, per_cu, p2) for kid in ((2, 3) if fp8 else (2,)) for block in (256, 512, 1024)
                 for per_cu in (1, 2, 4) for p2 in (2, 4) if block * per_cu <= 2048 and block * per_cu >= 512]
        for block, kid, p1, p2 in grid:
            def call(a):
                return lambda: ops.gemv_layoutA_wapper(a, x, n, k, 1, 0, block, kid, p1, p2, scale, None)
            try:
                if not _gate(call(packed[0])(), want, "%s %dx%d BLOCK_DIM_X=%d kernelId=%d p1=%d p2=%d" % (table, n, k, block, kid, p1, p2)):
                    continue
            except RuntimeError:                             # a configuration the library rejects for this shape
                continue
            us = _time_graph([call(a) for a in packed], iters)
            if best is None or us < best[0]:
                best = (us, block, kid, p1, p2)
        print("%s %dx%d -> %s" % (table, n, k, best), file=sys.stderr, flush=True)
        if best is None:
            continue
        rows.append("%d,%d,%d,%d,%d,%d" % (n, k, best[1], best[2], best[3], best[4]))
        if progress is not None:
            progress(rows[-1])
        del plain, packed
    return rows


def scan_gemm(table, shapes, tokens, iters, progress=None, known=(), kernel_ids=None):
    mode, dtype = GEMM_TABLES[table]
    fp8 = mode == "fp8"
    gen = torch.Generator(device="cuda").manual_seed(2025)
    rows = []
    for n, k in shapes:
        if n % 128 or k % 128:
            print("%s %dx%d skipped: the GEMM entry points need rows and K in multiples of 128" % (table, n, k),
                  file=sys.stderr)
            continue
        todo = [m for m in tokens if (n, m, k) not in known and not (mode in ("continuous", "native") and m % 16)]
        if not todo:
            continue
        plain = _weights(n, k, dtype, fp8, _copies(n * k * (1 if fp8 else 2)), gen)
        packed = [ops.pack_layout_a(w) for w in plain]
        scale = _block_scales(n // 128, k // 128, gen) if fp8 else None
        w0 = _scaled(plain[0], scale) if fp8 else plain[0].float()
        for m in todo:
            b = torch.randn((m, k), generator=gen, device="cuda").to(dtype)
            want = b.float() @ w0.t()
            b_in = ops.layoutB(b) if mode in ("continuous", "native") else b
            best = None
            # eight row groups per wave exist for one token block, or with row-major activations and output
            grid = [(1, r, w, sk) for r in ((1, 2, 4, 8) if m <= 16 or mode in ("rowmajor", "fp8") else (1, 2, 4))
                    for w in (1, 2, 4, 8, 16)
                    for sk in ((1, 2, 4) if n <= 8192 else (1,))]
            # kernel 2 (row-shared tiles): 4 waves x p1 row groups per workgroup, K split only across workgroups
            grid += [(2, r, 1, sk) for r in (1, 2, 4) for sk in (1, 2, 4, 8)
                     if (n // 16) % (4 * r) == 0 and (k // 32) % (4 * sk) == 0 and m > 16]
            # kernels 12..18: the wave kernel with 2, 4, 6 or 8 k tiles in flight per wave (one token block,
            # row-major activations and output)
            if m <= 16 and mode in ("rowmajor", "fp8"):
                grid += [(10 + u, r, w, sk) for (_, r, w, sk) in list(grid) if _ == 1 for u in (2, 4, 6, 8)]
            # kernel 4: one workgroup per CU, row groups dealt out evenly (16-bit weights, up to 64 tokens; from three
            # token blocks on, and at two token blocks with eight waves, the activations are shared through LDS)
            if mode == "rowmajor" and m <= 64:
                grid += [(4, 1, w, 1) for w in ((1, 2, 4, 8) if m <= 32 else (2, 4, 8))]
            # the same with soft-FP8 weights or layout-B activations, from two token blocks on (staged windows only)
            if mode in ("fp8", "continuous", "native") and 16 < m <= 64:
                grid += [(4, 1, w, 1) for w in (4, 8)]
            # kernel 3: panels of 128 / 256 rows x 128 / 256 tokens (row-major operands, K % 128 == 0); above 64 tokens the
            # wave kernel is out of the race
            if mode in ("rowmajor", "fp8") and m > 64 and k % 128 == 0:
                grid = [g for g in grid if g[0] != 1]
                grid += [(3, rg, w, sk) for rg, w in ((2, 1), (4, 1), (4, 2)) for sk in (1, 2, 4) if (k // 128) // sk >= 2]
                # kernel 5: the same with only the panels of the last, partial round sliced
                grid += [(5, rg, w, sk) for rg, w in ((2, 1), (4, 1), (4, 2)) for sk in (2, 3, 4) if (k // 128) // sk >= 2]
            for kid, p1, p2, p3 in grid:
                if (n // 16) % p1 or (kernel_ids is not None and kid not in kernel_ids):
                    continue
                if True:
                    def call(a):
                        if mode == "rowmajor":
                            return lambda: ops.gemm_layoutA_wapper(a, b_in, n, m, k, 1, 0, p1, p2, p3, kid, None)
                        if mode == "fp8":
                            return lambda: ops.gemm_layoutA_soft_fp8_wapper(a, scale, b_in, n, m, k, 1, 0, p1, p2, p3, kid,
                                                                            None)
                        if mode == "continuous":
                            return lambda: ops.gemm_layoutAB_ContinuousC_wapper(a, b_in, n, m, k, 1, 0, p1, p2, p3, kid, None)
                        return lambda: ops.gemm_layoutABC_wapper(a, b_in, n, m, k, 1, 0, p1, p2, p3, kid, None)
                    try:
                        got = call(packed[0])()
                    except RuntimeError:                     # a configuration the library rejects for this shape
                        continue
                    if mode == "native":
                        got = ops.reLayoutC(got)
                    if not _gate(got, want, "%s %dx%d M=%d kernelId=%d p1=%d p2=%d p3=%d" % (table, n, k, m, kid, p1, p2, p3)):
                        continue
                    us = _time_graph([call(a) for a in packed], iters)
                    if best is None or us < best[0]:
                        best = (us, kid, p1, p2, p3)
            print("%s %dx%d M=%d -> %s" % (table, n, k, m, best), file=sys.stderr, flush=True)
            if best is None:
                continue
            rows.append("%d,%d,%d,%d,%d,%d,%d" % (n, m, k, best[1], best[2], best[3], best[4]))
            if progress is not None:
                progress(rows[-1])
        del plain, packed
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("table", choices=list(GEMV_TABLES) + list(GEMM_TABLES) + ["all"])
    ap.add_argument("--shapes", default=None, help="comma separated MxK weight shapes, e.g. 4096x4096,11008x4096")
    ap.add_argument("--shape-set", choices=["default", "tables"], default="default",
                    help="without --shapes: the benchmark and model shapes, or the shapes of the reference's tables")
    ap.add_argument("--skip-known", action="store_true", help="leave out keys the packaged table already holds")
    ap.add_argument("--out-dir", default=".", help="where <table>_scan_best_args.csv goes without --update")
    ap.add_argument("--kernel-ids", default=None, help="GEMM tables: only these kernel ids, e.g. 3,5")
    ap.add_argument("--tokens", default=None, help="comma separated token counts for the GEMM tables")
    ap.add_argument("--iters", type=int, default=100)
    ap.add_argument("--update", action="store_true", help="append the rows to the packaged csv")
    args = ap.parse_args()
    tables = (list(GEMV_TABLES) + list(GEMM_TABLES)) if args.table == "all" else [args.table]
    for table in tables:
        shapes = (TABLE_SHAPES if args.shape_set == "tables" else DEFAULT_SHAPES)[table] if args.shapes is None else \
            [tuple(int(v) for v in s.split("x")) for s in args.shapes.split(",")]
        known = set(arg_selector.selector(table).table()) if args.skip_known else set()
        gemv = table in GEMV_TABLES
        header = "m,k,BLOCK_DIM_X,KernelId,KernelParam1,KernelParam2" if gemv else \
            "m,n,k,kernelId,kernelParam1,kernelParam2,kernelParam3"
        if args.update:
            path = arg_selector.selector(table).path()
            out = open(path, "a")
        else:
            path = os.path.join(args.out_dir, "%s_scan_best_args.csv" % table)
            out = open(path, "w")
            out.write(header + "\n")

        def progress(row):               # rows reach the file as they are found
            out.write(row + "\n")
            out.flush()
        if gemv:
            rows = scan_gemv(table, [s for s in shapes if s not in known], args.iters, progress)
        else:
            tokens = DEFAULT_TOKENS[table] if args.tokens is None else [int(v) for v in args.tokens.split(",")]
            ids = None if args.kernel_ids is None else {int(v) for v in args.kernel_ids.split(",")}
            rows = scan_gemm(table, shapes, tokens, args.iters, progress, known, ids)
        out.close()
        print("wrote %d rows to %s" % (len(rows), path), file=sys.stderr)
    if GATE_FAILURES:
        print("%d configurations ran but gave wrong results (listed above)" % len(GATE_FAILURES), file=sys.stderr)
        sys.exit(2)


if __name__ == "__main__":
    main()
