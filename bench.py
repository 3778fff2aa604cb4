"""Headline benchmark: the MoE layer at the Mixtral shape (BASELINE config 1) on one
MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mode fwdbwd|fwd] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic, already resident
inputs, through the layer's entry point `topk_moe_forward`: router (logits, softmax,
top-k), routing preprocessing, gate/up grouped GEMM with fused gather + SwiGLU, down
grouped GEMM with row scatter, top-k combine and (mode fwdbwd) the whole backward
pass, router included.  Prints ONE JSON line: whole-job TFLOP/s over the timed steps, the
roofline of the dominant kernel (measured with events on the launch stream) and
the CPU oracle timed on a bounded sample of the same workload.
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
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mode", choices=["fwdbwd", "fwd"], default="fwdbwd")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only", choices=["all", "kernel", "copy", "router", "passes", "configs23", "models", "fp32", "fp8", "digest", "ablation"],
                    default="all",
                    help="profiling aids: 'kernel' launches only the dominant GEMM --steps times, "
                         "'copy' only a 1 GiB device copy (the known-size kernel that calibrates "
                         "the FETCH_SIZE / WRITE_SIZE counters), 'router' the fused router and "
                         "then its ATen formulation at the shapes of configs 1-3, 'passes' the "
                         "HBM-bound passes (routing preprocessing, row gather, row scatter, top-k "
                         "combine) at the shapes of configs 1-3 with their algorithmic bytes and "
                         "event-timed GB/s, 'configs23' the routed experts (forward, then forward + "
                         "backward) at the shapes of configs 2 and 3, config 3 with Zipf(1.2) expert "
                         "loads, 'models' the whole layer (router included; forward, then forward + backward) "
                         "at the Qwen3-30B-A3B, OLMoE-1B-7B and Ernie-4.5 layer shapes with 32000 tokens "
                         "(the shapes and the token count of the reference's bench_glu.py / profile_proton.py), "
                         "'fp32' the layer in fp32 (exact products on 32x32x2 fp32 MFMAs; forward, then "
                         "forward + backward) with T = 8192, d = 2048, ff = 4096, E = 8, top-2, "
                         "'fp8' the fp8 inference layer (config 4: T = 128, 1024, 8192, GeGLU) "
                         "with its weight-streaming rate and TFLOP/s, 'digest' prints the digest of "
                         "the dominant kernel's sources that a profile summary records, 'ablation' times "
                         "the four GEMM shapes of config 1 (gate/up, dX, G without its fused epilogue, "
                         "dW1 and dW2) with evenly loaded experts on N(0,1) and on all-zero operands, "
                         "for runs with MOE_HIP_LIB pointing at a `build.py --ablate N` library; none "
                         "of them prints the JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    if args.only == "digest":
        print("KERNEL_SOURCE_SHA256_16=" + kernel_source_digest())
        return
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
    if args.only == "copy":
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(args.steps):
            dst.copy_(src)
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end) / args.steps
        # (what a plain device copy reaches is the practical roof of the HBM-bound passes)
        print("copied 1 GiB x %d: %.3f ms a copy = %.0f GB/s read + written (%.2f of 8 TB/s)"
              % (args.steps, ms, 2 * (1 << 30) / ms / 1e6, 2 * (1 << 30) / ms / 1e6 / 8000))
        return
    if args.only == "ablation":
        from moe_explore.hip_kernels.row_gather_scatter import row_gather_kmajor
        from moe_explore.testing import perfect_routing
        from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
        T, d, ff, E, k = cfg["T"], cfg["d"], cfg["ff"], cfg["E"], cfg["k"]
        R = T * k
        tag = os.path.basename(_C.lib_path())

        def timed(fn, flops, what, kind):
            for _ in range(args.warmup):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / args.steps * 1e3
            print("%-28s %-5s %-46s %7.3f ms %7.1f TFLOP/s" % (tag, kind, what, ms, flops / ms / 1e9), flush=True)

        for kind in ("rand", "zero"):
            torch.manual_seed(0)
            mk = (lambda *s: torch.randn(*s, device=dev, dtype=torch.bfloat16)) if kind == "rand" else \
                (lambda *s: torch.zeros(*s, device=dev, dtype=torch.bfloat16))
            w1, w2 = mk(E, d, 2 * ff) * 0.02, mk(E, ff, d) * 0.02
            x, dout, dh, a = mk(T, d), mk(T, d), mk(R, 2 * ff), mk(R, ff)
            _, idx = perfect_routing(T, E, k, dev, torch.bfloat16)
            p = get_token_indices(idx.view(T, k), k, E, zero_prefix=True)
            out = torch.empty((R, ff), device=dev, dtype=torch.bfloat16)
            gu = MGroupedGEMMParams(w1, p.group_indices, p.indices, True, False, T, k, activation="swiglu")
            px = MGroupedGEMMParams(w1, p.group_indices, p.indices, False, True, T, k)
            pg = MGroupedGEMMParams(w2, p.group_indices, p.indices, True, False, T, k)
            xt = row_gather_kmajor(x, p.indices, k, p.group_indices)
            dt = row_gather_kmajor(dout, p.indices, k, p.group_indices)
            with torch.no_grad():
                timed(lambda: m_grouped_gemm(x, gu, out=out), 4.0 * R * d * ff, "gate/up (N-contiguous W, gather, swiglu)", kind)
                timed(lambda: m_grouped_gemm(dh, px, transpose_weight=True), 4.0 * R * d * ff,
                      "dX (K-contiguous W, K = 2 ff, scatter)", kind)
                timed(lambda: m_grouped_gemm(dout, pg, transpose_weight=True), 2.0 * R * d * ff,
                      "G (K-contiguous W, K = d, gather, no epilogue)", kind)
                timed(lambda: k_grouped_gemm(xt, dh, p.group_indices, a_kmajor=True), 4.0 * R * d * ff,
                      "dW1 (K-grouped, a K-major)", kind)
                timed(lambda: k_grouped_gemm(a, dt, p.group_indices, b_kmajor=True), 2.0 * R * d * ff,
                      "dW2 (K-grouped, b K-major)", kind)
            del w1, w2, x, dout, dh, a, out, xt, dt
        return
    if args.only == "fp32":
        # (157.3 TFLOP/s is the device's fp32 matrix-core peak)
        T, d, ff, E, k = 8192, 2048, 4096, 8, 2
        torch.manual_seed(0)
        x = torch.randn(T, d, device=dev).requires_grad_(True)
        w1 = (torch.randn(E, d, 2 * ff, device=dev) * 0.02).requires_grad_(True)
        w2 = (torch.randn(E, ff, d, device=dev) * 0.02).requires_grad_(True)
        wr = (torch.randn(d, E, device=dev) * d ** -0.5).requires_grad_(True)
        mp = MOEParams(TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True),
                       GLUInterleavedParams(w1, w2, "swiglu"), E, k)
        dout = torch.randn(T, d, device=dev)

        def fwd():
            with torch.no_grad():
                topk_moe_forward(x, mp)

        def fwdbwd():
            x.grad = w1.grad = w2.grad = wr.grad = None
            topk_moe_forward(x, mp).backward(dout)

        for fn, units, label in ((fwd, 6, "fwd"), (fwdbwd, 18, "fwd+bwd")):
            for _ in range(args.warmup):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                fn()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / args.steps * 1e3
            tf = units * T * k * d * ff / ms / 1e9
            print("fp32 layer T=%d d=%d ff=%d E=%d top-%d  %-8s %8.3f ms %7.1f TFLOP/s (%.2f of 157.3)" % (
                T, d, ff, E, k, label, ms, tf, tf / 157.3), flush=True)
        return
    if args.only == "fp8":
        from moe_explore.fp8 import Fp8MLPParams, quantize_expert_weights, routed_experts_fp8
        from moe_explore.router import route_from_logits
        d, ff, E, k = cfg["d"], cfg["ff"], cfg["E"], cfg["k"]
        gd = torch.Generator(device=dev).manual_seed(0)
        w1 = torch.empty((E, d, 2 * ff), device=dev, dtype=torch.bfloat16).normal_(0.0, 0.02, generator=gd)
        w2 = torch.empty((E, ff, d), device=dev, dtype=torch.bfloat16).normal_(0.0, 0.02, generator=gd)
        params = Fp8MLPParams(quantize_expert_weights(w1), quantize_expert_weights(w2), "geglu")
        del w1, w2
        weight_bytes = 3.0 * E * d * ff      # e4m3: one byte a weight
        for T in (128, 1024, 8192):
            x = torch.randn((T, d), device=dev, generator=gd).to(torch.bfloat16)
            scores, idx = route_from_logits(torch.randn((T, E), device=dev, generator=gd), k, True, True,
                                            torch.bfloat16)
            with torch.no_grad():
                for _ in range(args.warmup):
                    routed_experts_fp8(x, params, scores, idx, E, k)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    routed_experts_fp8(x, params, scores, idx, E, k)
                torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / args.steps * 1e3
            print("fp8 layer fwd (geglu) T=%5d: %7.3f ms  %7.1f TFLOP/s  weights streamed at %6.0f GB/s" % (
                T, ms, 6.0 * T * k * d * ff / ms / 1e9, weight_bytes / ms / 1e6), flush=True)
        return
    if args.only == "router":
        from moe_explore.router import route_from_logits
        for (T, d, E, k) in [(4096, 4096, 8, 2), (8192, 2048, 64, 8), (16384, 2048, 64, 6)]:
            x = torch.randn((T, d), device=dev, dtype=torch.bfloat16)
            wr = (torch.randn((d, E), device=dev) * d ** -0.5).to(torch.bfloat16)
            rp = TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True)
            with torch.no_grad():
                for _ in range(args.steps):
                    topk_router(x, rp)
                torch.cuda.synchronize()
                for _ in range(args.steps):
                    route_from_logits(x @ wr, k, True, True, x.dtype)
                torch.cuda.synchronize()
            print("router T=%d d=%d E=%d top-%d: fused x %d, ATen x %d" % (T, d, E, k, args.steps, args.steps))
        return
    if args.only == "passes":
        from moe_explore.expert_permute import get_token_indices as route
        from moe_explore.functional.scale_and_reduce import scale_and_reduce
        from moe_explore.triton_kernels.row_gather_scatter import row_gather, row_scatter

        def timed(fn):
            for _ in range(3):
                fn()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in range(args.steps)]
            for s, e in evs:
                s.record()
                fn()
                e.record()
            torch.cuda.synchronize()
            return sorted(s.elapsed_time(e) for s, e in evs)[len(evs) // 2] * 1e-3

        for (T, d, E, k) in [(4096, 4096, 8, 2), (8192, 2048, 64, 8), (16384, 2048, 64, 6)]:
            R = T * k
            g = torch.Generator(device=dev).manual_seed(0)
            x = torch.randn((T, d), device=dev, dtype=torch.bfloat16, generator=g)
            y = torch.randn((R, d), device=dev, dtype=torch.bfloat16, generator=g)
            logits = torch.randn((T, E), device=dev, generator=g)
            sc, idx = torch.topk(torch.softmax(logits, -1), k, dim=-1)
            sc = (sc / sc.sum(-1, keepdim=True)).to(torch.bfloat16)
            perm = route(idx, k, E, zero_prefix=True)
            # algorithmic bytes: expert ids read + slot ids written + offsets; rows read + written
            # + one index a row; k rows and k scores read + one row written
            passes = [
                ("route_preprocess (count, scan, place)", 8 * R + 8 * R + 4 * (E + 1),
                 lambda: route(idx, k, E, zero_prefix=True)),
                ("row_gather   x[idx // k] -> [R, d]", 2 * R * d * 2 + 8 * R,
                 lambda: row_gather(x, perm.indices, index_div=k)),
                ("row_scatter  y -> out[idx]", 2 * R * d * 2 + 8 * R,
                 lambda: row_scatter(y, perm.indices)),
                ("scale_and_reduce [R, d] -> [T, d]", (R + T) * d * 2 + R * 2,
                 lambda: scale_and_reduce(y, sc, T, k, d)),
            ]
            with torch.no_grad():
                for name, nbytes, fn in passes:
                    sec = timed(fn)
                    print("T=%d d=%d E=%d top-%d  %-40s %10.3f MB  %7.1f us  %7.1f GB/s" % (
                        T, d, E, k, name, nbytes / 1e6, sec * 1e6, nbytes / sec / 1e9))
        return
    if args.only == "configs23":
        from moe_explore.functional.topk_moe import routed_experts
        from moe_explore.router import route_from_logits
        for name, T, d, ff, E, k, zipf in (("config 2", 8192, 2048, 1024, 64, 8, None),
                                          ("config 3", 16384, 2048, 1408, 64, 6, 1.2)):
            torch.manual_seed(0)
            dt = torch.bfloat16
            x = torch.randn(T, d, device=dev, dtype=dt)
            w1 = torch.randn(E, d, 2 * ff, device=dev, dtype=dt) * 0.02
            w2 = torch.randn(E, ff, d, device=dev, dtype=dt) * 0.02
            logits = torch.randn(T, E, device=dev)
            if zipf:  # per-expert bias: expert i is chosen with probability ~ (i + 1) ** -zipf
                pz = torch.tensor([(i + 1.0) ** -zipf for i in range(E)])
                logits = logits + torch.log(pz / pz.sum() * E).to(dev)
            scores, idx = route_from_logits(logits, k, True, True, dt)
            cnt = torch.bincount(idx.flatten(), minlength=E)
            dout = torch.randn(T, d, device=dev, dtype=dt)
            R = T * k
            for t in (x, w1, w2):
                t.requires_grad_(True)

            def fwd():
                with torch.no_grad():
                    routed_experts(x, w1, w2, scores, idx, E, k, "swiglu")

            def fwdbwd():
                x.grad = w1.grad = w2.grad = None
                routed_experts(x, w1, w2, scores, idx, E, k, "swiglu").backward(dout)

            for fn, units, label in ((fwd, 6, "fwd"), (fwdbwd, 18, "fwd+bwd")):
                for _ in range(args.warmup):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    fn()
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t0) / args.steps * 1e3
                print("%s T=%d d=%d ff=%d E=%d top-%d rows/expert %d..%d  %-8s %8.3f ms %7.1f TFLOP/s" % (
                    name, T, d, ff, E, k, cnt.min().item(), cnt.max().item(), label, ms,
                    units * R * d * ff / ms / 1e9), flush=True)
        return
    if args.only == "models":
        # (bench/bench_glu.py:74-103 for the shapes, bench/profile_proton.py:16-21 for the tokens;
        # under `rocprofv3 --kernel-trace --stats` the kernels are the stages of the reference's
        # profile: router, get_token_indices, fused grouped GLU, down grouped GEMM, scale_and_reduce)
        from moe_explore.params import ErnieRouterParams
        for name, d, ff, E, k, ernie in (("Qwen3-30B-A3B", 2048, 768, 128, 8, False),
                                         ("OLMoE-1B-7B", 2048, 1024, 64, 8, False),
                                         ("Ernie-4.5-21B-A3B", 2560, 1536, 64, 6, True)):
            torch.manual_seed(0)
            T, dt = 32000, torch.bfloat16
            R = T * k
            x = torch.randn(T, d, device=dev, dtype=dt).requires_grad_(True)
            w1 = (torch.randn(E, d, 2 * ff, device=dev, dtype=dt) * 0.02).requires_grad_(True)
            w2 = (torch.randn(E, ff, d, device=dev, dtype=dt) * 0.02).requires_grad_(True)
            if ernie:
                wr = (torch.randn(d, E, device=dev) * d ** -0.5).requires_grad_(True)
                rp = ErnieRouterParams(wr, torch.rand(E, device=dev) * (2.0 / E), k)
            else:
                wr = (torch.randn(d, E, device=dev, dtype=dt) * d ** -0.5).requires_grad_(True)
                rp = TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True)
            mp = MOEParams(rp, GLUInterleavedParams(w1, w2, "swiglu"), E, k)
            dout = torch.randn(T, d, device=dev, dtype=dt)

            def fwd():
                with torch.no_grad():
                    topk_moe_forward(x, mp)

            def fwdbwd():
                x.grad = w1.grad = w2.grad = wr.grad = None
                topk_moe_forward(x, mp).backward(dout)

            for fn, units, label in ((fwd, 6, "fwd"), (fwdbwd, 18, "fwd+bwd")):
                for _ in range(args.warmup):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    fn()
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t0) / args.steps * 1e3
                print("%-18s T=%d d=%d ff=%d E=%d top-%d  %-8s %8.3f ms %7.1f TFLOP/s" % (
                    name, T, d, ff, E, k, label, ms, units * R * d * ff / ms / 1e9), flush=True)
            del x, w1, w2, wr, dout, mp
        return
    T, d, ff, E, k = cfg["T"], cfg["d"], cfg["ff"], cfg["E"], cfg["k"]
    R = T * k
    x, w1, w2, wr, dout = make_inputs(cfg, dev)
    router_params = TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True)
    params = MOEParams(router_params, GLUInterleavedParams(w1, w2, "swiglu"), E, k)
    with torch.no_grad():
        scores, idx = topk_router(x, router_params)
    train = args.mode == "fwdbwd"
    if args.only == "kernel":
        with torch.no_grad():
            p = get_token_indices(idx, k, E, zero_prefix=True)
            gp = MGroupedGEMMParams(w1, p.group_indices, p.indices, True, False, T, k, activation="swiglu")
            a_out = torch.empty((R, ff), device=dev, dtype=torch.bfloat16)
            for _ in range(args.steps):
                m_grouped_gemm(x, gp, out=a_out)
        torch.cuda.synchronize()
        print("launched the gate/up grouped GEMM x %d" % args.steps)
        return
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
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": cfg["name"], "mode": args.mode, "routed_rows": R,
                   "flops_per_step": flops_step},
        "pct_of_bf16_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "fwd": {"ms": round(fwd_ms, 4), "tflops": round(fwd_tflops, 2),
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
