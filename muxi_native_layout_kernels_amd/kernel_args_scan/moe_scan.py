"""Offline scan of the fused-MoE launch switches on gfx950.

Counterpart of the reference's kernel_args_scan/muxi_moe_args_scan.py:92-110, which times its `fused_moe` over
`APerWarp x splitK x tile_m_2` for every token count and keeps the fastest.  Here the switches are the library's
`mlk_set_tunable` ids (include/mlk.h):

    one token          ids 2, 3 (row groups per workgroup and waves splitting K in the gate/up GeMV kernel),
                       4 (waves of the down kernel), 5 (16-byte loads in flight per wave)
    2 .. 16 tokens     id 7 (row groups per wave = K slices of the decode down kernel)
    above 16 tokens    id 8 (upper limit of the 16-token blocks that share one pass over an expert's weights),
                       the row-shared kernels on / off (`mlk_moe_set_tile_path`) and, with soft-FP8 weights, id 10
                       (panel kernels: K slices of the down projection + 16 x two workgroups per CU; ignored
                       where the panel kernels do not run)

Every setting is gated on the output of the default setting (rtol = atol = 1e-2, which the parity tests pin
against the oracle), timed as HIP-graph replays of the whole `fused_moe` call, and the fastest one is written
with the default's time beside it:

    python -m muxi_native_layout_kernels_amd.kernel_args_scan.moe_scan --preset mixtral --tokens 1,16,64,256
    python -m muxi_native_layout_kernels_amd.kernel_args_scan.moe_scan --experts 128 --topk 8 --hidden 2048 --inter 768 --grouped --fp8

As in the reference, the result file is a report: the library's defaults (csrc/mlk_moe.hip) are set from it by
hand; nothing reads the csv at run time.
"""
import argparse
import itertools
import sys

import torch

from .. import _lib
from ..moe_planC import fused_moe

PRESETS = {
    "mixtral": dict(experts=8, topk=2, hidden=4096, inter=14336, grouped=False),
    "deepseek": dict(experts=256, topk=8, hidden=7168, inter=2048, grouped=True),
    "deepseek_tp8": dict(experts=256, topk=8, hidden=7168, inter=256, grouped=True),
    "qwen3_30b": dict(experts=128, topk=8, hidden=2048, inter=768, grouped=True),
}
DEFAULTS = {2: 1, 3: 8, 4: 16, 5: 0, 7: 0, 8: 0, 10: 0}


def _time_graph(call, iters):
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(iters):
                call()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / iters
            best = us if best is None else min(best, us)
    return best


def settings_for(tokens, topk, fp8=False):
    """The grid of (tunable id -> value, tile path) settings that can matter at this token count."""
    if tokens == 1:
        out = []
        for g, wk in ((1, 8), (1, 4), (2, 4), (2, 2), (1, 2)):
            for dw in sorted({16, max(8, topk)}):
                for depth in (2, 3, 4, 6, 8):
                    out.append(({2: g, 3: wk, 4: dw, 5: depth}, 1))
        return out
    if tokens <= 16:
        return [({7: r}, 1) for r in (1, 2, 4)]
    out = [({8: cap}, tile) for cap, tile in itertools.product((0, 1, 2, 3, 4, 6, 8), (1, 0)) if tile or cap <= 4]
    if fp8:
        out += [({10: v}, 1) for v in (1, 2, 4, 8, 17, 18, 20, 24)]
    return out


def apply(lib, setting):
    values, tile = setting
    for tid, default in DEFAULTS.items():
        lib.mlk_set_tunable(tid, values.get(tid, default))
    lib.mlk_moe_set_tile_path(1 if tile else 0)


def scan(experts, topk, hidden, inter, grouped, fp8, tokens, iters, out):
    lib = _lib.load()
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev).manual_seed(2025)
    dtype = torch.bfloat16
    if fp8:
        w1 = (torch.randn((experts, 2 * inter, hidden), generator=gen, device=dev) * 16).clamp_(-448, 448)
        w1 = w1.to(torch.float8_e4m3fn).view(torch.uint8)
        w2 = (torch.randn((experts, hidden, inter), generator=gen, device=dev) * 16).clamp_(-448, 448)
        w2 = w2.to(torch.float8_e4m3fn).view(torch.uint8)
        # arbitrary block scales: the general widening path (powers of two would take a cheaper one)
        kw = dict(w1_scale=torch.rand((experts, 2 * inter // 128, hidden // 128), generator=gen, device=dev) * 2e-3 + 1e-4,
                  w2_scale=torch.rand((experts, hidden // 128, inter // 128), generator=gen, device=dev) * 2e-3 + 1e-4,
                  block_shape=[128, 128], soft_fp8=True)
    else:
        w1 = (torch.randn((experts, 2 * inter, hidden), generator=gen, device=dev) * 0.02).to(dtype)
        w2 = (torch.randn((experts, hidden, inter), generator=gen, device=dev) * 0.02).to(dtype)
        kw = {}
    if grouped:
        kw.update(use_grouped_topk=True, num_expert_group=8, topk_group=4, score_func="sigmoid")
    for t in tokens:
        x = torch.randn((t, hidden), generator=gen, device=dev).to(dtype)
        logits = torch.randn((t, experts), generator=gen, device=dev).to(dtype)

        def call():
            return fused_moe(x, w1, w2, logits, topk, True, **kw)
        apply(lib, ({}, 1))
        want = call().float()
        us_default = _time_graph(call, iters)
        best = (us_default, ({}, 1))
        for setting in settings_for(t, topk, fp8):
            apply(lib, setting)
            try:
                got = call().float()
            except RuntimeError:
                continue
            if not bool(((got - want).abs() <= 1e-2 + 1e-2 * want.abs()).all()):
                print("  T=%d %s: output differs from the default setting, skipped" % (t, setting), file=sys.stderr)
                continue
            us = _time_graph(call, iters)
            if us < best[0]:
                best = (us, setting)
        apply(lib, ({}, 1))
        # the default was timed first, on a GPU that had been idle: time it again and keep the better of the two
        us_default = min(us_default, _time_graph(call, iters))
        if us_default < best[0]:
            best = (us_default, ({}, 1))
        values, tile = best[1]
        row = [t, experts, topk, hidden, inter, int(fp8), "%.2f" % best[0], "%.2f" % us_default] + \
              [values.get(tid, DEFAULTS[tid]) for tid in sorted(DEFAULTS)] + [tile]
        print("moe T=%d -> %s" % (t, row), file=sys.stderr, flush=True)
        out.write(",".join(str(v) for v in row) + "\n")
        out.flush()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--preset", choices=sorted(PRESETS), default=None)
    ap.add_argument("--experts", type=int, default=8)
    ap.add_argument("--topk", type=int, default=2)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--inter", type=int, default=14336)
    ap.add_argument("--grouped", action="store_true", help="8 expert groups, 4 kept, sigmoid scores")
    ap.add_argument("--fp8", action="store_true", help="soft-FP8 weights")
    ap.add_argument("--tokens", default="1,16,64,256")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--out", default="moe_scan_best_args.csv")
    args = ap.parse_args()
    cfg = dict(experts=args.experts, topk=args.topk, hidden=args.hidden, inter=args.inter, grouped=args.grouped)
    if args.preset:
        cfg = dict(PRESETS[args.preset])
    tokens = [int(v) for v in args.tokens.split(",")]
    with open(args.out, "a") as out:
        if out.tell() == 0:
            out.write("tokens,experts,topk,hidden,inter,fp8,us_best,us_default," +
                      ",".join("tunable%d" % tid for tid in sorted(DEFAULTS)) + ",tile_path\n")
        scan(cfg["experts"], cfg["topk"], cfg["hidden"], cfg["inter"], cfg["grouped"], args.fp8, tokens, args.iters, out)


if __name__ == "__main__":
    main()
