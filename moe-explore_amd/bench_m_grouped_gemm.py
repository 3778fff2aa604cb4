"""Grouped-GEMM sweep in the shape of the reference's bench/bench_m_grouped_gemm.py
(:10-41 configurations, :164-223 providers, :264 CSV output): time of one M-grouped GEMM
against the number of tokens for grouped-only / +gather / +scatter, next to a batched GEMM
(torch.bmm) of the same FLOPs, with balanced, skewed, OLMoE-measured or perfect routing.
Prints a table (median of event timings) and, with --csv, writes the reference's CSV layout
(one row a token count, one TFLOP/s column a provider).

    python moe-explore_amd/bench_m_grouped_gemm.py [--shape qwen3|mixtral|olmoe]
        [--routing balanced|skewed|olmoe|perfect] [--tokens 256,1024,...] [--csv DIR]
"""
import argparse
import csv
import math
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import torch

from moe_explore.expert_permute import get_token_indices
from moe_explore.testing import (perfect_routing, random_olmoe_routing, random_routing,
                                 random_skewed_routing)
from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams, m_grouped_gemm

SHAPES = {  # experts, N, K, topk  (bench_m_grouped_gemm.py:43-60 and the Mixtral / OLMoE gate-up shapes)
    "qwen3": (128, 2048, 768, 8),
    "olmoe": (64, 2048, 2048, 8),
    "mixtral": (8, 28672, 4096, 2),
}
PROVIDERS = ("gemm-reference", "grouped-only", "grouped-gather", "grouped-scatter")
ROUTINGS = ("balanced", "skewed", "olmoe", "perfect")


def median_ms(fn, warmup=5, reps=20):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        times.append(s.elapsed_time(e))
    return sorted(times)[len(times) // 2]


def route(routing, T, E, topk, dev, dt):
    if routing == "balanced":
        return random_routing(T, E, topk, dev, dt)[1]
    if routing == "skewed":
        return random_skewed_routing(T, E, topk, 8, 16, dev, dt)[1]
    if routing == "olmoe":
        return random_olmoe_routing(T, E, topk, dev, dt)[1]
    return perfect_routing(T, E, topk, dev, dt)[1]


def run_sweep(shape, routing, tokens, warmup=5, reps=20, seed=0):
    """Rows of ``{"num_tokens", provider: TFLOP/s ..., provider + "_ms": ms ...}`` for the token
    counts in ``tokens``; the batched-GEMM column is NaN where the rows do not divide evenly."""
    E, N, K, topk = SHAPES[shape]
    dev, dt = torch.device("cuda"), torch.bfloat16
    torch.manual_seed(seed)   # random routers: seeded as in bench_m_grouped_gemm.py:243
    weight = torch.randn((E, K, N), device=dev, dtype=dt) / math.sqrt(N)
    rows = []
    for T in tokens:
        idx = route(routing, T, E, topk, dev, dt)
        p = get_token_indices(idx, topk, E, zero_prefix=True)
        R = T * topk
        flops = 2.0 * R * N * K
        x = torch.randn((T, K), device=dev, dtype=dt)
        xr = torch.randn((R, K), device=dev, dtype=dt)
        ms = {}
        if R % E == 0:
            xb = xr.view(E, R // E, K)
            ms["gemm-reference"] = median_ms(lambda: torch.bmm(xb, weight), warmup, reps)
        else:
            ms["gemm-reference"] = float("nan")
        only = MGroupedGEMMParams(weight, p.group_indices, None, False, False, R, topk)
        ms["grouped-only"] = median_ms(lambda: m_grouped_gemm(xr, only), warmup, reps)
        gat = MGroupedGEMMParams(weight, p.group_indices, p.indices, True, False, T, topk)
        ms["grouped-gather"] = median_ms(lambda: m_grouped_gemm(x, gat), warmup, reps)
        sca = MGroupedGEMMParams(weight, p.group_indices, p.indices, False, True, T, topk)
        ms["grouped-scatter"] = median_ms(lambda: m_grouped_gemm(xr, sca), warmup, reps)
        row = {"num_tokens": T}
        for name in PROVIDERS:
            row[name] = flops / ms[name] / 1e9
            row[name + "_ms"] = ms[name]
        rows.append(row)
    return rows


def write_csv(rows, path):
    """The layout of the reference's perf_report CSV: num_tokens, then TFLOP/s per provider."""
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["num_tokens", *PROVIDERS])
        for r in rows:
            w.writerow([r["num_tokens"], *("%.3f" % r[name] for name in PROVIDERS)])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", default="qwen3", choices=sorted(SHAPES))
    ap.add_argument("--routing", default="balanced", choices=ROUTINGS)
    ap.add_argument("--tokens", default="256,1024,2048,4096,8192")
    ap.add_argument("--csv", default=None, metavar="DIR",
                    help="also write DIR/m_grouped_gemm_<shape>_<routing>.csv")
    a = ap.parse_args()
    E, N, K, topk = SHAPES[a.shape]
    if a.routing == "olmoe" and E != 64:
        ap.error("the OLMoE load table has 64 experts: use --shape olmoe")
    print(f"{a.shape}: E={E} K={K} N={N} top-{topk}, {a.routing} routing, bf16; ms (TFLOP/s)")
    print(f"{'tokens':>7} " + " ".join(f"{name:>18}" for name in PROVIDERS))
    rows = []
    for T in [int(t) for t in a.tokens.split(",")]:
        row = run_sweep(a.shape, a.routing, [T])[0]
        rows.append(row)
        print(f"{T:7d} " + " ".join(f"{row[n + '_ms']:8.3f} ({row[n]:7.1f})" for n in PROVIDERS), flush=True)
    if a.csv:
        os.makedirs(a.csv, exist_ok=True)
        path = os.path.join(a.csv, f"m_grouped_gemm_{a.shape}_{a.routing}.csv")
        write_csv(rows, path)
        print("wrote", path)


if __name__ == "__main__":
    main()
