"""Headline benchmark: the MoE layer at the Mixtral shape (BASELINE config 1) on one
MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mode fwdbwd|fwd] [--no-cpu]

(Stage-by-stage profiling aids for runs under rocprofv3 live in moe-explore_amd/bench_stages.py.)

A step is one pass of the hot path over one batch of synthetic, already resident
inputs, through the layer's entry point `topk_moe_forward`: router (logits, softmax,
top-k), routing preprocessing, gate/up grouped GEMM with fused gather + SwiGLU, down
grouped GEMM with row scatter, top-k combine and (mode fwdbwd) the whole backward
pass, router included.  Prints ONE JSON line: whole-job TFLOP/s over the timed steps, the
roofline of the dominant kernel (measured with events on the launch stream) and
the CPU oracle timed on a bounded sample of the same workload.

Timing: W untimed warm-up steps, then exactly K steps between two device synchronisations on
the host clock (`ms_per_step`, `value`: what an outside clock around the run sees), and next to
it the median of per-step event pairs on the launch stream over max(K, 50) further steps
(`median_ms`), which is free of the host's launch jitter.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "moe-explore_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

# published dense peaks of MI355X
PEAK_BF16_TFLOPS = 2500.0

CONFIG1 = dict(name="mixtral-moe-layer T=4096 d=4096 ff=14336 E=8 top2 swiglu bf16",
               T=4096, d=4096, ff=14336, E=8, k=2)


def make_inputs(cfg, device, seed=0):
    import torch
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    T, d, ff, E, k = cfg["T"], cfg["d"], cfg["ff"], cfg["E"], cfg["k"]
    dt = torch.bfloat16
    x = torch.randn((T, d), generator=g).to(dt).to(device)
    gd = torch.Generator(device=device)
    gd.manual_seed(seed)
    w1 = torch.empty((E, d, 2 * ff), device=device, dtype=dt).normal_(0.0, 0.02, generator=gd)
    w2 = torch.empty((E, ff, d), device=device, dtype=dt).normal_(0.0, 0.02, generator=gd)
    wr = (torch.randn((d, E), generator=g) * d ** -0.5).to(dt).to(device)  # logits ~ N(0, 1)
    dout = torch.randn((T, d), generator=g).to(dt).to(device)
    return x, w1, w2, wr, dout


PROFILE_OF_DOMINANT_KERNEL = os.path.join(ROOT, "profiles", "m_grouped_dma_kernel_mixtral_config1.txt")
KERNEL_SOURCES = [os.path.join(ROOT, "moe-explore_amd", "csrc", f) for f in ("gemm_mfma_dma.hip", "gemm_mfma.h")]


def kernel_source_digest():
    """sha256 (first 16 hex digits) over the sources of the dominant kernel."""
    import hashlib
    h = hashlib.sha256()
    for path in KERNEL_SOURCES:
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic_bytes():
    """HBM bytes a launch of the dominant kernel from the tracked rocprofv3 summary (its line
    `TRAFFIC_BYTES_PER_LAUNCH=... KERNEL_SOURCE_SHA256_16=...`), or None when the summary is
    missing or was made from other kernel sources than the ones in the tree."""
    import re
    try:
        text = open(PROFILE_OF_DOMINANT_KERNEL).read()
    except OSError:
        return None
    m = re.search(r"TRAFFIC_BYTES_PER_LAUNCH=([0-9.eE+]+)\s+KERNEL_SOURCE_SHA256_16=([0-9a-f]{16})", text)
    if not m or m.group(2) != kernel_source_digest():
        return None
    return float(m.group(1))


def device_clock_mhz():
    """Maximum shader clock of the first GPU agent that rocminfo lists (0.0 if it cannot be
    read); run as a child process."""
    import re
    import subprocess
    try:
        text = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=30).stdout
    except (OSError, subprocess.SubprocessError):
        return 0.0
    for agent in text.split("*******")[1:]:
        if "Device Type:             GPU" in agent or re.search(r"Device Type:\s+GPU", agent):
            m = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent)
            if m:
                return float(m.group(1))
    return 0.0


def cpu_baseline(cfg, x, w1, w2, scores, idx, dout, mode, sample_tokens=4096):
    """The oracle's per-expert fp32 loop (and autograd backward) on the host cores, on
    the first `sample_tokens` tokens of the same batch with the same weights."""
    import torch
    from oracle import moe_ref
    E, k, d, ff = cfg["E"], cfg["k"], cfg["d"], cfg["ff"]
    xs, ss, ii, do = (t[:sample_tokens].cpu() for t in (x, scores, idx, dout))
    w1c, w2c = w1.cpu().float(), w2.cpu().float()
    R = sample_tokens * k
    t0 = time.perf_counter()
    if mode == "fwd":
        moe_ref.experts_forward(xs, w1c, w2c, ss, ii, E, k, "swiglu")
        flops = 6.0 * R * d * ff
    else:
        moe_ref.experts_backward(xs, w1c, w2c, ss, ii, E, k, "swiglu", do)
        flops = 18.0 * R * d * ff
    dt = time.perf_counter() - t0
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {sample_tokens} of {cfg['T']} tokens, full d/ff/E, fp32 oracle {mode}, "
                  f"{dt:.2f} s on {os.cpu_count()} visible cpus",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--mode", choices=["fwdbwd", "fwd"], default="fwdbwd")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from moe_explore import _C
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.functional.topk_moe import topk_moe_forward
    from moe_explore.params import GLUInterleavedParams, MOEParams, TopkRouterParams
    from moe_explore.router import topk_router
    from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams, m_grouped_gemm

    _C.load()
    dev = torch.device("cuda:0")
    cfg = CONFIG1
    T, d, ff, E, k = cfg["T"], cfg["d"], cfg["ff"], cfg["E"], cfg["k"]
    R = T * k
    x, w1, w2, wr, dout = make_inputs(cfg, dev)
    router_params = TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True)
    params = MOEParams(router_params, GLUInterleavedParams(w1, w2, "swiglu"), E, k)
    with torch.no_grad():
        scores, idx = topk_router(x, router_params)
    train = args.mode == "fwdbwd"
    if train:
        x.requires_grad_(True)
        w1.requires_grad_(True)
        w2.requires_grad_(True)
        wr.requires_grad_(True)

    def step():
        out = topk_moe_forward(x, params)
        if train:
            x.grad = w1.grad = w2.grad = wr.grad = None
            out.backward(dout)
        return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    flops_step = (18.0 if train else 6.0) * R * d * ff
    value = flops_step / (ms_per_step * 1e-3) / 1e12

    def median_of_event_pairs(fn, n):
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for s, e in evs:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return sorted(s.elapsed_time(e) for s, e in evs)[n // 2]

    median_ms = median_of_event_pairs(step, max(args.steps, 50))

    # forward alone, same protocol, for the fwd half of the metric
    with torch.no_grad():
        for _ in range(args.warmup):
            topk_moe_forward(x, params)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            topk_moe_forward(x, params)
        torch.cuda.synchronize()
        fwd_ms = (time.perf_counter() - t0) / args.steps * 1e3
        fwd_median_ms = median_of_event_pairs(lambda: topk_moe_forward(x, params), max(args.steps, 50))
    fwd_tflops = 6.0 * R * d * ff / (fwd_ms * 1e-3) / 1e12

    # dominant kernel: gate/up grouped GEMM (fused gather + SwiGLU), 4*R*d*ff flops a launch
    with torch.no_grad():
        p = get_token_indices(idx, k, E, zero_prefix=True)
        gp = MGroupedGEMMParams(w1, p.group_indices, p.indices, True, False, T, k, activation="swiglu")
        a_out = torch.empty((R, ff), device=dev, dtype=torch.bfloat16)
        for _ in range(3):
            m_grouped_gemm(x, gp, out=a_out)
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
               for _ in range(args.steps)]
        for s, e in evs:
            s.record()
            m_grouped_gemm(x, gp, out=a_out)
            e.record()
        torch.cuda.synchronize()
        k_ms = sum(s.elapsed_time(e) for s, e in evs) / len(evs)
    k_flops = 4.0 * R * d * ff
    achieved = k_flops / (k_ms * 1e-3) / 1e12

    props = torch.cuda.get_device_properties(0)
    clock_mhz = device_clock_mhz()
    # 4096 dense bf16 FLOP per clock and CU (1024 per SIMD and clock)
    device_peak = props.multi_processor_count * 4096 * clock_mhz * 1e6 / 1e12
    line = {
        "metric": "MoE-layer TFLOP/s (%s) at Mixtral shape" % ("fwd+bwd" if train else "fwd"),
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "median_ms": round(median_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": cfg["name"], "mode": args.mode, "routed_rows": R,
                   "flops_per_step": flops_step},
        "pct_of_bf16_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "fwd": {"ms": round(fwd_ms, 4), "median_ms": round(fwd_median_ms, 4), "tflops": round(fwd_tflops, 2),
                "pct_of_bf16_peak": round(100.0 * fwd_tflops / PEAK_BF16_TFLOPS, 2)},
        "roofline": {"kernel": "m_grouped_dma_kernel (gate/up grouped GEMM, fused gather + swiglu)",
                     "bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "launch_ms": round(k_ms, 4), "flops_per_launch": k_flops,
                     # HBM bytes a launch from rocprofv3 FETCH_SIZE / WRITE_SIZE, calibrated
                     # with a 1 GiB copy, read from the tracked summary of that profile; null
                     # when the kernel's sources have changed since it was made
                     "traffic": profiled_traffic_bytes()},
        # peak recomputed from what the device reports; the sustained clock under this load
        # is lower (about 1.65-1.8 GHz with random operands)
        "device": {"name": props.name, "cus": props.multi_processor_count, "clock_mhz": clock_mhz,
                   "bf16_peak_from_device_tflops": round(device_peak, 1)},
    }
    if not args.no_cpu:
        x.requires_grad_(False)
        line["cpu_baseline"] = cpu_baseline(cfg, x.detach(), w1.detach(), w2.detach(), scores, idx,
                                            dout, args.mode)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
