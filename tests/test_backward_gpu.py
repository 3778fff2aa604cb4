"""Backward pass on the GPU (dX via transposed M-grouped GEMM, dW via K-grouped
GEMM, activation gradient, routing-weight gradient) against torch.autograd through
the oracle's fp32 expert loop.  The reference is forward-only; autograd through the
restated forward is the definition being checked."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity, randn, random_group_indices, seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,E,Ka,Nb,dtype", [
    (500, 4, 128, 256, torch.bfloat16), (1000, 8, 264, 136, torch.float16),
    (300, 3, 50, 70, torch.float32), (4096, 8, 512, 512, torch.bfloat16),
])
def test_k_grouped_gemm_plain(rows, E, Ka, Nb, dtype):
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    g = seeded(rows + Ka)
    a, b = randn((rows, Ka), g, dtype), randn((rows, Nb), g, dtype)
    gi = random_group_indices(rows, E, g)
    out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda())
    ref = moe_ref.k_grouped_matmul(a, b, gi)
    assert out.shape == (E, Ka, Nb)
    assert_parity(out, ref, dtype, "k_grouped_gemm")
    # experts without rows get exact zeros
    lens = (gi[1:] - gi[:-1])
    for e in torch.nonzero(lens == 0).flatten().tolist():
        assert (out[e] == 0).all()


@pytest.mark.parametrize("sizes", [
    [0, 1, 64, 65, 0, 130, 7, 0],              # empty experts between short segments
    [1] * 12,                                  # every tile is a single K step
    [0, 0, 0, 300, 0, 0],                      # one expert owns everything
    [64, 128, 192, 256, 63, 129],              # segment ends on and next to step boundaries
    [5, 0, 700, 0, 3, 64, 0, 0, 1, 250, 17, 0, 0, 90, 2, 66],
    # 64 experts with Zipf-like loads and a few empty ones: chunks dealt by load, not round-robin
    [max(0, int(2500 / (i + 1) ** 1.2) - 12) for i in range(64)],
])
@pytest.mark.parametrize("gather", [None, "a", "b"])
def test_k_grouped_gemm_tile_pipeline(sizes, gather):
    """More tiles than workgroups, so that a workgroup runs several tiles (and tiles
    of different experts) through one copy pipeline, with ragged and empty segments."""
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    g = seeded(sum(sizes) + len(sizes))
    E, rows, Ka, Nb, topk = len(sizes), sum(sizes), 776, 2568, 2   # 4 x 11 tiles an expert, ragged edges
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    perm = torch.randperm(rows, generator=g)          # slot ids in sorted order
    tokens = (rows + topk - 1) // topk
    a = randn((tokens if gather == "a" else rows, Ka), g, torch.bfloat16)
    b = randn((tokens if gather == "b" else rows, Nb), g, torch.bfloat16)
    if gather is None:
        out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda())
        ref = moe_ref.k_grouped_matmul(a, b, gi)
    else:
        out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda(), perm.cuda(), topk,
                             gather_a=gather == "a", gather_b=gather == "b")
        ref = moe_ref.k_grouped_matmul(a, b, gi, perm, topk, gather == "a", gather == "b")
    assert_parity(out, ref, torch.bfloat16, "k_grouped_gemm pipeline")
    for e, n in enumerate(sizes):
        if n == 0:
            assert (out[e] == 0).all()


@pytest.mark.parametrize("sizes", [
    [0, 1, 64, 65, 0, 130, 7, 0],
    [1] * 12,
    [32, 31, 33, 0, 300],                      # segment ends on and next to K-step boundaries
    [5, 0, 700, 0, 3, 64, 0, 0, 1, 250, 17, 0, 0, 90, 2, 66],
])
@pytest.mark.parametrize("Ka,Nb", [(776, 2568), (132, 36)])
@pytest.mark.parametrize("gather", [None, "a", "b"])
def test_k_grouped_gemm_fp32_matrix_core_kernel(sizes, Ka, Nb, gather):
    """fp32 with widths that are multiples of 4 runs on 32x32x2 fp32 MFMAs: 256- and 128-row
    output tiles (by tile count), ragged tile edges, ragged and empty segments, fetched rows."""
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    g = seeded(sum(sizes) + len(sizes) + Ka)
    E, rows, topk = len(sizes), sum(sizes), 2
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    perm = torch.randperm(rows, generator=g)
    tokens = (rows + topk - 1) // topk
    a = randn((tokens if gather == "a" else rows, Ka), g, torch.float32)
    b = randn((tokens if gather == "b" else rows, Nb), g, torch.float32)
    if gather is None:
        out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda())
        ref = moe_ref.k_grouped_matmul(a, b, gi)
    else:
        out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda(), perm.cuda(), topk,
                             gather_a=gather == "a", gather_b=gather == "b")
        ref = moe_ref.k_grouped_matmul(a, b, gi, perm, topk, gather == "a", gather == "b")
    assert_parity(out, ref, torch.float32, "fp32 k_grouped_gemm")
    for e, n in enumerate(sizes):
        if n == 0:
            assert (out[e] == 0).all()
        else:
            assert_parity(out[e], ref[e], torch.float32, f"expert {e}")


def test_k_grouped_gemm_many_uneven_experts():
    """100 experts with Zipf-like loads: the kernel numbers its tiles by expert rank and deals
    the chunks by load; ranks 64 and up come from the second half of the ranking."""
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    sizes = [max(0, int(2000 / (i + 1) ** 1.1) - 9) for i in range(100)]
    sizes = [sizes[(37 * i) % 100] for i in range(100)]      # loads not in expert order
    g = seeded(100)
    E, rows, Ka, Nb = len(sizes), sum(sizes), 264, 520         # 2 x 3 tiles an expert
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    a, b = randn((rows, Ka), g, torch.bfloat16), randn((rows, Nb), g, torch.bfloat16)
    out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda())
    ref = moe_ref.k_grouped_matmul(a, b, gi)
    assert_parity(out, ref, torch.bfloat16, "k_grouped_gemm, 100 uneven experts")
    for e, n in enumerate(sizes):
        if n == 0:
            assert (out[e] == 0).all()
    # every expert on its own: a misplaced tile shows in one expert, not in the norm of all
    for e in (0, 36, 63, 64, 99):
        if sizes[e]:
            assert_parity(out[e], ref[e], torch.bfloat16, f"expert {e}")


@pytest.mark.parametrize("E,Ka,Nb", [(160, 264, 520), (200, 520, 776)])
def test_k_grouped_gemm_more_experts_than_the_balanced_deal_takes(E, Ka, Nb):
    """More than 128 uneven experts (and, second case, more than 512 chunks of tiles): the
    kernel keeps its round-robin deal of tile chunks instead of the one balanced by load."""
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    sizes = [max(0, int(1500 / (i + 1) ** 1.1) - 5) for i in range(E)]
    sizes = [sizes[(53 * i) % E] for i in range(E)]
    g = seeded(E)
    rows = sum(sizes)
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    a, b = randn((rows, Ka), g, torch.bfloat16), randn((rows, Nb), g, torch.bfloat16)
    out = k_grouped_gemm(a.cuda(), b.cuda(), gi.cuda())
    ref = moe_ref.k_grouped_matmul(a, b, gi)
    assert_parity(out, ref, torch.bfloat16, f"k_grouped_gemm, {E} uneven experts")
    for e in range(E):
        if sizes[e] == 0:
            assert (out[e] == 0).all()
        elif e % 7 == 0 or sizes[e] < 4:
            assert_parity(out[e], ref[e], torch.bfloat16, f"expert {e} ({sizes[e]} rows)")


@pytest.mark.parametrize("sizes,T,d,dtype", [
    ([130, 0, 64, 1, 63, 65, 300, 0], 400, 72, torch.bfloat16),
    ([1000, 1030, 990, 1076], 2048, 256, torch.bfloat16),
    ([5] * 20, 77, 136, torch.float16),
    ([0, 0, 700], 350, 64, torch.bfloat16),
    ([130, 0, 64, 1, 63, 65, 300, 0], 400, 328, torch.bfloat16),   # one feature group and a partial one
    ([900, 1100], 1000, 1024, torch.float16),
])
def test_row_gather_kmajor_layout(sizes, T, d, dtype):
    """moe_row_gather_kmajor: expert e's rows, transposed, start at column 64 * (lo // 64 + e)
    and are followed by zeros up to the next multiple of 64 (exact: a copy)."""
    from moe_explore.hip_kernels.row_gather_scatter import row_gather_kmajor
    g = seeded(sum(sizes) + d)
    E, R, k = len(sizes), sum(sizes), 2
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    slots = torch.randint(0, T * k, (R,), generator=g)
    x = randn((T, d), g, dtype)
    out = row_gather_kmajor(x.cuda(), slots.cuda(), k, gi.cuda())
    assert out is not None and out.shape == (d, 64 * (R // 64 + E + 1))
    out = out.cpu()
    for e, n in enumerate(sizes):
        lo = int(gi[e])
        qs = 64 * (lo // 64 + e)
        want = x[slots[lo:lo + n] // k].t()
        assert torch.equal(out[:, qs:qs + n], want), f"expert {e}"
        pad = (-n) % 64
        if n:
            assert (out[:, qs + n:qs + n + pad] == 0).all(), f"zero fill of expert {e}"


@pytest.mark.parametrize("which", ["a", "b"])
@pytest.mark.parametrize("sizes,Ka,Nb", [
    ([700, 0, 515, 1300, 5, 600], 264, 520),
    ([0, 1, 64, 65, 0, 130, 7, 0], 776, 2568),
    ([1024, 1000, 1050, 1022], 512, 768),
    ([max(0, int(2500 / (i + 1) ** 1.2) - 12) for i in range(64)], 256, 520),
])
def test_k_grouped_gemm_kmajor_operand(which, sizes, Ka, Nb):
    """The weight-gradient GEMM with its gathered operand given feature-major
    (row_gather_kmajor), against the oracle's gathered product."""
    from moe_explore.hip_kernels.row_gather_scatter import row_gather_kmajor
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    g = seeded(sum(sizes) + Ka)
    E, R, topk = len(sizes), sum(sizes), 2
    T = (R + topk - 1) // topk
    gi = torch.zeros(E + 1, dtype=torch.int32)
    gi[1:] = torch.cumsum(torch.tensor(sizes), 0)
    perm = torch.randperm(R, generator=g)
    if which == "a":
        a, b = randn((T, Ka), g, torch.bfloat16), randn((R, Nb), g, torch.bfloat16)
        at = row_gather_kmajor(a.cuda(), perm.cuda(), topk, gi.cuda())
        out = k_grouped_gemm(at, b.cuda(), gi.cuda(), a_kmajor=True)
    else:
        a, b = randn((R, Ka), g, torch.bfloat16), randn((T, Nb), g, torch.bfloat16)
        bt = row_gather_kmajor(b.cuda(), perm.cuda(), topk, gi.cuda())
        out = k_grouped_gemm(a.cuda(), bt, gi.cuda(), b_kmajor=True)
    ref = moe_ref.k_grouped_matmul(a, b, gi, perm, topk, which == "a", which == "b")
    assert out.shape == (E, Ka, Nb)
    assert_parity(out, ref, torch.bfloat16, f"k_grouped_gemm, K-major {which}")
    for e, n in enumerate(sizes):
        if n == 0:
            assert (out[e] == 0).all()
        elif e % 9 == 0 or n < 8:
            assert_parity(out[e], ref[e], torch.bfloat16, f"expert {e} ({n} rows)")


def test_k_grouped_gemm_kmajor_is_refused_outside_the_mfma_kernel():
    from moe_explore import _C
    from moe_explore.hip_kernels.row_gather_scatter import row_gather_kmajor
    g = seeded(3)
    x = randn((40, 36), g, torch.float32)
    gi = torch.tensor([0, 30, 64], dtype=torch.int32)
    assert row_gather_kmajor(x.cuda(), torch.arange(64).cuda(), 2, gi.cuda()) is None   # fp32
    xb = randn((40, 36), g, torch.bfloat16)                                              # 36 % 8 != 0
    assert row_gather_kmajor(xb.cuda(), torch.arange(64).cuda(), 2, gi.cuda()) is None


@pytest.mark.parametrize("which", ["a", "b"])
def test_k_grouped_gemm_gather(which):
    from moe_explore.expert_permute import get_token_indices
    from moe_explore.triton_kernels.m_grouped_gemm import k_grouped_gemm
    g = seeded(21)
    T, E, k, Ka, Nb = 400, 8, 2, 128, 192
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    p = get_token_indices(idx.cuda(), k, E, zero_prefix=True)
    if which == "a":
        a, b = randn((T, Ka), g, torch.bfloat16), randn((T * k, Nb), g, torch.bfloat16)
    else:
        a, b = randn((T * k, Ka), g, torch.bfloat16), randn((T, Nb), g, torch.bfloat16)
    out = k_grouped_gemm(a.cuda(), b.cuda(), p.group_indices, p.indices, k,
                         gather_a=which == "a", gather_b=which == "b")
    ref = moe_ref.k_grouped_matmul(a, b, p.group_indices, p.indices, k, which == "a", which == "b")
    assert_parity(out, ref, torch.bfloat16, "k_grouped_gemm gather " + which)


@pytest.mark.parametrize("act", ["silu", "gelu", "approx_gelu", "swiglu", "geglu"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N", [96, 100, 1048])   # 100: rows that only take the one-column path
def test_act_bwd(act, dtype, N):
    from moe_explore.hip_kernels.m_grouped_gemm import act_bwd
    g = seeded(len(act) + N)
    R = 300
    No = N // 2 if "glu" in act else N
    h, dy = randn((R, N), g, dtype), randn((R, No), g, dtype)
    scale = torch.rand((R,), generator=g).to(dtype)
    perm = torch.randperm(R, generator=g)
    dh, ys, ds = act_bwd(h.cuda(), dy.cuda(), act, row_scale=scale.cuda(), permute_indices=perm.cuda(),
                         want_y_scaled=True, want_dscale=True)
    hf = h.float().requires_grad_(True)
    y = moe_ref.activation(hf, act)
    w = scale.float()[perm].unsqueeze(1)
    (y * w * dy.float()).sum().backward()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert dh.dtype == dtype and ys.dtype == dtype
    assert_parity(dh, hf.grad, dtype, "dh", tol=tol)
    assert_parity(ys, (y * w).detach(), dtype, "y_scaled", tol=tol)
    ds_ref = torch.zeros(R)
    ds_ref[perm] = (y.detach() * dy.float()).sum(1)
    assert_parity(ds, ds_ref, torch.float32, "dscale", tol=1e-4 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("act", ["swiglu", "geglu"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sizes", [[700, 0, 515, 1300, 5, 600], [40, 130, 0, 78]])
def test_fused_glu_backward_matches_the_two_steps_and_the_oracle(act, dtype, sizes):
    """moe_m_grouped_gemm_glu_bwd (G = dOut @ W2^T never stored; dH, s*A and dscore from the
    GEMM's epilogue) against m_grouped_gemm + act_bwd and against autograd through the oracle's
    activation; large ragged groups (256-row tiles) and small ones (128-row tiles)."""
    from moe_explore.hip_kernels.m_grouped_gemm import (MGroupedGEMMParams, act_bwd, m_grouped_gemm,
                                                        m_grouped_gemm_glu_bwd)
    g = seeded(sum(sizes) + len(act))
    E, topk, d, ff = len(sizes), 2, 192, 264
    R = sum(sizes)
    T = R // topk
    assert R % topk == 0
    gi = torch.tensor([0] + list(torch.tensor(sizes).cumsum(0)), dtype=torch.int32)
    perm = torch.randperm(R, generator=g)            # slot id of every sorted position
    dout = randn((T, d), g, dtype)
    w2 = randn((E, ff, d), g, dtype, 0.1)
    h = randn((R, 2 * ff), g, dtype)
    scores = torch.rand((T, topk), generator=g).to(dtype)
    pf = MGroupedGEMMParams(w2.cuda(), gi.cuda(), perm.cuda(), True, False, T, topk, scales=scores.cuda())
    fused = m_grouped_gemm_glu_bwd(dout.cuda(), pf, h.cuda(), act, transpose_weight=True, want_dscale=True)
    assert fused is not None
    dh, ys, ds = fused
    pg = MGroupedGEMMParams(w2.cuda(), gi.cuda(), perm.cuda(), True, False, T, topk)
    G = m_grouped_gemm(dout.cuda(), pg, transpose_weight=True)
    dh2, ys2, ds2 = act_bwd(h.cuda(), G, act, row_scale=scores.cuda(), permute_indices=perm.cuda(),
                            want_y_scaled=True, want_dscale=True)
    # same rounded G and the same formulas; the compiler may contract the fp32 products
    # differently in the two kernels, which shows in the last bit of an fp16 result
    assert_parity(dh, dh2.float().cpu(), dtype, "dh vs two steps", tol=2e-3)
    assert_parity(ys, ys2.float().cpu(), dtype, "y_scaled vs two steps", tol=2e-3)
    torch.testing.assert_close(ds, ds2, rtol=1e-4, atol=1e-4)
    # oracle: fp32 products and autograd through the activation
    Gref = moe_ref.grouped_matmul_gather_scatter(dout, w2.transpose(1, 2), gi, perm, gather=True,
                                                 num_tokens=T, topk=topk)
    hf = h.float().requires_grad_(True)
    y = moe_ref.activation(hf, act)
    s_pos = scores.float().view(-1)[perm].unsqueeze(1)
    (y * s_pos * Gref).sum().backward()
    assert_parity(dh, hf.grad, dtype, "dh")
    assert_parity(ys, (y * s_pos).detach(), dtype, "y_scaled")
    ds_ref = torch.zeros(R)
    ds_ref[perm] = (y.detach() * Gref).sum(1)
    assert_parity(ds, ds_ref, torch.float32, "dscale", tol=2e-2)


def test_fused_glu_backward_declines_what_it_cannot_run():
    from moe_explore.hip_kernels.m_grouped_gemm import MGroupedGEMMParams, m_grouped_gemm_glu_bwd
    g = seeded(3)
    E, R, d, ff = 2, 64, 72, 40     # K = 72 is not a multiple of 64
    gi = torch.tensor([0, 30, 64], dtype=torch.int32)
    p = MGroupedGEMMParams(randn((E, ff, d), g, torch.bfloat16).cuda(), gi.cuda(), None, False, False, R, 1)
    out = m_grouped_gemm_glu_bwd(randn((R, d), g, torch.bfloat16).cuda(), p,
                                 randn((R, 2 * ff), g, torch.bfloat16).cuda(), "swiglu",
                                 transpose_weight=True)
    assert out is None


@pytest.mark.parametrize("T,d,ff,E,k,act,dtype", [
    (64, 32, 48, 4, 2, "swiglu", torch.float32),
    (300, 128, 96, 8, 2, "geglu", torch.float32),
    (257, 64, 80, 8, 3, "silu", torch.float32),
    # fp32 on the matrix cores with 256-row tiles (512 rows an expert) and every K-step path
    (2048, 512, 768, 8, 2, "swiglu", torch.float32),
    (1500, 260, 132, 4, 2, "geglu", torch.float32),
    (512, 256, 512, 8, 2, "swiglu", torch.bfloat16),
    (999, 256, 128, 64, 8, "swiglu", torch.bfloat16),
    (640, 128, 256, 8, 2, "gelu", torch.float16),
    # 16-bit widths that are not multiples of 8: the feature-major operand of the weight-gradient
    # kernel is refused and the backward gathers row-major instead
    (300, 128, 100, 8, 2, "silu", torch.bfloat16),
    (300, 128, 50, 8, 2, "swiglu", torch.bfloat16),
    (200, 64, 36, 4, 2, "geglu", torch.float16),
])
def test_layer_backward(T, d, ff, E, k, act, dtype):
    from moe_explore.functional.topk_moe import routed_experts
    g = seeded(T + ff)
    n1 = 2 * ff if "glu" in act else ff
    x = randn((T, d), g, dtype)
    w1 = randn((E, d, n1), g, dtype, 0.1)
    w2 = randn((E, ff, d), g, dtype, 0.1)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, dtype)
    dout = randn((T, d), g, dtype)
    xc = x.cuda().requires_grad_(True)
    w1c = w1.cuda().requires_grad_(True)
    w2c = w2.cuda().requires_grad_(True)
    sc = scores.cuda().requires_grad_(True)
    out = routed_experts(xc, w1c, w2c, sc, idx.cuda(), E, k, act)
    out.backward(dout.cuda())
    # (fp32 results are held to 1e-5 against the oracle computed in fp64, whose own summation
    # noise is then far below the bar)
    ref_out, dx, dw1, dw2, ds = moe_ref.experts_backward(
        x, w1, w2, scores, idx, E, k, act, dout,
        compute_dtype=torch.float64 if dtype == torch.float32 else torch.float32)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert_parity(out, ref_out, dtype, "out", tol=tol)
    assert_parity(xc.grad, dx, dtype, "dx", tol=tol)
    assert_parity(w1c.grad, dw1, dtype, "dw1", tol=tol)
    assert_parity(w2c.grad, dw2, dtype, "dw2", tol=tol)
    assert_parity(sc.grad, ds, dtype, "dscores", tol=tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_layer_backward_of_an_empty_batch(dtype):
    """T = 0: every launch is skipped or runs over no positions; the weight gradients are
    zero and dX is empty."""
    from moe_explore.functional.topk_moe import routed_experts
    d, ff, E, k = 64, 96, 4, 2
    x = torch.zeros((0, d), dtype=dtype).cuda().requires_grad_(True)
    w1 = randn((E, d, 2 * ff), seeded(1), dtype, 0.1).cuda().requires_grad_(True)
    w2 = randn((E, ff, d), seeded(2), dtype, 0.1).cuda().requires_grad_(True)
    scores = torch.zeros((0, k), dtype=dtype).cuda().requires_grad_(True)
    idx = torch.zeros((0, k), dtype=torch.int64).cuda()
    out = routed_experts(x, w1, w2, scores, idx, E, k, "swiglu")
    assert out.shape == (0, d)
    out.backward(torch.zeros((0, d), dtype=dtype).cuda())
    assert x.grad.shape == (0, d) and scores.grad.shape == (0, k)
    assert w1.grad.shape == w1.shape and not w1.grad.any()
    assert w2.grad.shape == w2.shape and not w2.grad.any()


def test_backward_config1_properties():
    """BASELINE config 1 with d_ff reduced 8x and T=1024, so that autograd through the
    oracle covers every element of every gradient in seconds (the full size is checked on
    token and column subsets in test_backward_configs_gpu.py)."""
    from moe_explore.functional.topk_moe import routed_experts
    g = seeded(8)
    T, d, ff, E, k = 1024, 1024, 1792, 8, 2
    x = randn((T, d), g, torch.bfloat16)
    w1 = randn((E, d, 2 * ff), g, torch.bfloat16, 0.02)
    w2 = randn((E, ff, d), g, torch.bfloat16, 0.02)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, torch.bfloat16)
    dout = randn((T, d), g, torch.bfloat16)
    xc, w1c, w2c = (t.cuda().requires_grad_(True) for t in (x, w1, w2))
    out = routed_experts(xc, w1c, w2c, scores.cuda(), idx.cuda(), E, k, "swiglu")
    out.backward(dout.cuda())
    _, dx, dw1, dw2, _ = moe_ref.experts_backward(x, w1, w2, scores, idx, E, k, "swiglu", dout)
    assert_parity(xc.grad, dx, torch.bfloat16, "dx")
    assert_parity(w1c.grad, dw1, torch.bfloat16, "dw1")
    assert_parity(w2c.grad, dw2, torch.bfloat16, "dw2")
