"""Profiling aids: one stage of the MoE layer at a time, for runs under rocprofv3.

    python moe-explore_amd/bench_stages.py STAGE [--steps K] [--warmup W]

None of them prints the JSON line of bench.py (the headline benchmark at the repository root);
each prints its own short table, and the kernel trace / counters of the profiler are the result.

  kernel     the dominant GEMM alone (gate/up grouped GEMM of the Mixtral-shape layer, fused
             gather + SwiGLU, the bench's routing), --steps times
  copy       a 1 GiB device copy: the known-size kernel that calibrates FETCH_SIZE / WRITE_SIZE
  router     the fused router, then its ATen formulation, at the shapes of configs 1-3
  passes     the HBM-bound passes (routing preprocessing, row gather, row scatter, top-k combine)
             at the shapes of configs 1-3 with their algorithmic bytes and event-timed GB/s
  configs23  the routed experts (forward, then forward + backward) at the shapes of configs 2 and
             3, config 3 with Zipf(1.2) expert loads
  models     the whole layer (router included) at the Qwen3-30B-A3B, OLMoE-1B-7B and Ernie-4.5
             layer shapes with 32000 tokens (the shapes of the reference's bench/bench_glu.py:74-103,
             the token count of bench/profile_proton.py:16-21)
  fp32       the layer in fp32 (exact products on 32x32x2 fp32 MFMAs) with T = 8192, d = 2048,
             ff = 4096, E = 8, top-2
  fp8        the fp8 inference layer (config 4: T = 128, 1024, 8192, GeGLU) with its
             weight-streaming rate and TFLOP/s
  gemms      the six grouped GEMMs of a Mixtral-shape training step one by one (median of event
             pairs), with the bench's routing and with evenly loaded experts
  routings   the four M-grouped GEMMs of a Mixtral-shape training step with other routings: five
             more seeds of router logits at 4096 tokens, then 3000, 6144, 8192 and 2048 tokens
  combine    the down projection of the Mixtral-shape layer with its top-k combine, two ways: rows
             stored in slot order (split K) + scale_and_reduce, as the layer runs it, and the
             weighted scatter-add fused into the GEMM's store (fp32 atomics, m_grouped_gemm(combine=True))
  digest     the digest of the dominant kernel's sources that a profile summary records
"""
import argparse
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for p in (ROOT, HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import bench  # noqa: E402  (the headline benchmark: config, inputs, digest)

STAGES = ["kernel", "copy", "router", "passes", "configs23", "models", "fp32", "fp8", "gemms", "routings", "combine", "digest"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("stage", choices=STAGES)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    args = ap.parse_args()
    if args.stage == "digest":
        print("KERNEL_SOURCE_SHA256_16=" + bench.kernel_source_digest())
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
    cfg = bench.CONFIG1
    if args.stage == "copy":
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
    if args.stage == "fp32":
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
    if args.stage == "fp8":
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
    if args.stage == "router":
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
    if args.stage == "passes":
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
    if args.stage == "configs23":
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
    if args.stage == "models":
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
    x, w1, w2, wr, dout = bench.make_inputs(cfg, dev)
    router_params = TopkRouterParams(wr, k, softmax_before_topk=True, normalize_routing=True)
    with torch.no_grad():
        scores, idx = topk_router(x, router_params)
    if args.stage == "kernel":
        with torch.no_grad():
            p = get_token_indices(idx, k, E, zero_prefix=True)
            gp = MGroupedGEMMParams(w1, p.group_indices, p.indices, True, False, T, k, activation="swiglu")
            a_out = torch.empty((R, ff), device=dev, dtype=torch.bfloat16)
            for _ in range(args.steps):
                m_grouped_gemm(x, gp, out=a_out)
        torch.cuda.synchronize()
        print("launched the gate/up grouped GEMM x %d" % args.steps)
        return
    if args.stage == "combine":
        from moe_explore.functional.scale_and_reduce import scale_and_reduce
        from moe_explore.functional.topk_moe import _ksplit_for

        def median_ms(fn):
            for _ in range(args.warmup):
                fn()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in range(args.steps)]
            for s, e in evs:
                s.record()
                fn()
                e.record()
            torch.cuda.synchronize()
            return sorted(s.elapsed_time(e) for s, e in evs)[len(evs) // 2]

        with torch.no_grad():
            p = get_token_indices(idx, k, E, zero_prefix=True)
            a = torch.randn((R, ff), device=dev, dtype=torch.bfloat16)
            dn = MGroupedGEMMParams(w2, p.group_indices, p.indices, False, True, T, k, scales=scores)
            ks = _ksplit_for(R, E, d, ff)

            def two_passes():
                y = m_grouped_gemm(a, dn, ksplit=ks)
                return scale_and_reduce(y, scores, T, k, d, nsplit=y.size(0) // R)

            t_gemm = median_ms(lambda: m_grouped_gemm(a, dn, ksplit=ks))
            t_two = median_ms(two_passes)
            t_fused = median_ms(lambda: m_grouped_gemm(a, dn, combine=True))
            ref, got = two_passes().float(), m_grouped_gemm(a, dn, combine=True).float()
            err = ((got - ref).norm() / ref.norm()).item()
        print("down projection + top-%d combine, T=%d d=%d ff=%d E=%d (%.0f M output elements scattered):" % (k, T, d, ff, E, R * d / 1e6))
        print("  GEMM storing rows in slot order (split K = %d)        %7.3f ms" % (ks, t_gemm))
        print("  ... + scale_and_reduce (the layer's path)            %7.3f ms" % t_two)
        print("  GEMM with the weighted scatter-add fused (fp32 atomics) %7.3f ms   (rel. difference of the results %.1e)" % (t_fused, err))
        return
    if args.stage == "routings":
        from moe_explore.functional.topk_moe import _ksplit_for
        from moe_explore.hip_kernels.m_grouped_gemm import m_grouped_gemm_glu_bwd
        from moe_explore.router import route_from_logits

        def timed(fn):
            for _ in range(args.warmup):
                fn()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in range(args.steps)]
            for s, e in evs:
                s.record()
                fn()
                e.record()
            torch.cuda.synchronize()
            return sorted(s.elapsed_time(e) for s, e in evs)[len(evs) // 2]

        del x, dout
        total = 0.0
        for tokens, seed in ((T, 1), (T, 2), (T, 3), (T, 4), (T, 5), (3000, 6), (6144, 7), (8192, 8), (2048, 9)):
            g = torch.Generator(device=dev).manual_seed(seed)
            xs = torch.randn(tokens, d, device=dev, generator=g).to(torch.bfloat16)
            ds = torch.randn(tokens, d, device=dev, generator=g).to(torch.bfloat16)
            sc, ii = route_from_logits(torch.randn(tokens, E, device=dev, generator=g), k, True, True,
                                       torch.bfloat16)
            with torch.no_grad():
                p = get_token_indices(ii, k, E, zero_prefix=True)
                gi, ind = p.group_indices, p.indices
                gu = MGroupedGEMMParams(w1, gi, ind, True, False, tokens, k, activation="swiglu")
                a, h = m_grouped_gemm(xs, gu, save_preact=True)
                dn = MGroupedGEMMParams(w2, gi, ind, False, True, tokens, k, scales=sc)
                pf = MGroupedGEMMParams(w2, gi, ind, True, False, tokens, k, scales=sc)
                dh, _, _ = m_grouped_gemm_glu_bwd(ds, pf, h, "swiglu", transpose_weight=True, want_dscale=True)
                px = MGroupedGEMMParams(w1, gi, ind, False, True, tokens, k)
                ks, ksx = _ksplit_for(tokens * k, E, d, ff), _ksplit_for(tokens * k, E, d, 2 * ff)
                ms = [timed(lambda: m_grouped_gemm(xs, gu, save_preact=True)),
                      timed(lambda: m_grouped_gemm(a, dn, ksplit=ks)),
                      timed(lambda: m_grouped_gemm_glu_bwd(ds, pf, h, "swiglu", transpose_weight=True,
                                                           want_dscale=True)),
                      timed(lambda: m_grouped_gemm(dh, px, transpose_weight=True, ksplit=ksx))]
            total += sum(ms)
            print("T=%d seed %d rows %s split K %d/%d: gate/up %.3f  down %.3f  G fused %.3f  dX %.3f  sum %.3f ms" % (
                tokens, seed, (gi[1:] - gi[:-1]).tolist(), ks, ksx, *ms, sum(ms)), flush=True)
            del xs, ds, a, h, dh
        print("total %.3f ms" % total)
        return
    if args.stage == "gemms":
        from moe_explore.functional.topk_moe import _ksplit_for
        from moe_explore.hip_kernels.m_grouped_gemm import k_grouped_gemm, m_grouped_gemm_glu_bwd
        from moe_explore.hip_kernels.row_gather_scatter import row_gather_kmajor
        from moe_explore.testing import perfect_routing

        def timed(fn):
            for _ in range(args.warmup):
                fn()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in range(args.steps)]
            for s, e in evs:
                s.record()
                fn()
                e.record()
            torch.cuda.synchronize()
            return sorted(s.elapsed_time(e) for s, e in evs)[len(evs) // 2]

        ps, pidx = perfect_routing(T, E, k, dev, torch.bfloat16)
        with torch.no_grad():
            for tag, sc, ii in (("bench routing", scores, idx), ("even loads", ps.view(T, k), pidx.view(T, k))):
                p = get_token_indices(ii, k, E, zero_prefix=True)
                gi, ind = p.group_indices, p.indices
                print("%s: rows per expert %s" % (tag, (gi[1:] - gi[:-1]).tolist()), flush=True)
                gu = MGroupedGEMMParams(w1, gi, ind, True, False, T, k, activation="swiglu")
                a, h = m_grouped_gemm(x, gu, save_preact=True)
                dn = MGroupedGEMMParams(w2, gi, ind, False, True, T, k, scales=sc)
                pf = MGroupedGEMMParams(w2, gi, ind, True, False, T, k, scales=sc)
                dh, a_s, _ = m_grouped_gemm_glu_bwd(dout, pf, h, "swiglu", transpose_weight=True, want_dscale=True)
                px = MGroupedGEMMParams(w1, gi, ind, False, True, T, k)
                ks, ksx = _ksplit_for(R, E, d, ff), _ksplit_for(R, E, d, 2 * ff)
                xt = row_gather_kmajor(x, ind, k, gi)
                dt = row_gather_kmajor(dout, ind, k, gi)
                total = 0.0
                for name, units, fn in (
                        ("gate/up (gather, swiglu, saves H)", 4, lambda: m_grouped_gemm(x, gu, save_preact=True)),
                        ("down (scatter, split K = %d)" % ks, 2, lambda: m_grouped_gemm(a, dn, ksplit=ks)),
                        ("G = dOut W2^T, fused GLU backward", 2,
                         lambda: m_grouped_gemm_glu_bwd(dout, pf, h, "swiglu", transpose_weight=True, want_dscale=True)),
                        ("dX = dH W1^T (scatter, split K = %d)" % ksx, 4,
                         lambda: m_grouped_gemm(dh, px, transpose_weight=True, ksplit=ksx)),
                        ("dW1 (K-grouped, a K-major)", 4, lambda: k_grouped_gemm(xt, dh, gi, a_kmajor=True)),
                        ("dW2 (K-grouped, b K-major)", 2, lambda: k_grouped_gemm(a_s, dt, gi, b_kmajor=True))):
                    ms = timed(fn)
                    total += ms
                    print("  %-40s %7.3f ms %7.1f TFLOP/s" % (name, ms, units * R * d * ff / ms / 1e9), flush=True)
                print("  sum %.3f ms" % total, flush=True)
        return


if __name__ == "__main__":
    main()
