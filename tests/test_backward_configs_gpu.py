"""Backward pass at the FULL sizes of BASELINE configs 1, 2 and 3 against autograd through the
oracle's fp32 expert loop (`moe_ref.experts_backward`), which is too slow for the whole problem
but exact on two restrictions of it:

* tokens: out[t], dX[t] and dscores[t] depend on token t alone, so the oracle runs on a subset
  of the tokens with the full weights;
* GLU columns: with J a set of hidden columns, dW1[e][:, (2j, 2j+1) for j in J] and
  dW2[e][J, :] depend on W1[e][:, those columns], W2[e][J, :] and all tokens only
  (H[:, 2j:2j+2] = X_e W1[e][:, 2j:2j+2], G[:, j] = dOut_e W2[e][j, :]^T), so the oracle runs
  the layer restricted to those columns over ALL tokens and returns exactly those slices of
  the weight gradients, for every expert.

Between those restrictions the whole tensors are covered by a second reference: the same
per-expert loop and autograd in plain PyTorch fp32 ON THE GPU (library GEMMs, none of this
package's kernels), which is first held to the CPU oracle on the restrictions above (1e-4) and
then compared with the HIP results over every element: whole tensors, every expert on its own,
and every 256 x 256 tile of every expert's weight gradients on its own (a wrong or dropped
tile is under 1 % of an expert's gradient and would pass a whole-tensor norm).

These are the shapes the benchmark times: split-K dX over K = 2*ff = 28672 with transposed
weights (config 1), 64 experts with 88 tiles each (configs 2 and 3), Zipf(1.2) loads with
near-empty experts next to one of ~16000 rows (config 3: the weight-gradient kernel's
load-balanced chunk deal)."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2   # bf16 against the fp32-accumulated oracle


def _inputs(T, d, ff, E, k, zipf, seed):
    dev = torch.device("cuda")
    gd = torch.Generator(device=dev).manual_seed(seed)
    gc = torch.Generator().manual_seed(seed)
    dt = torch.bfloat16
    x = torch.randn((T, d), generator=gc).to(dt)
    dout = torch.randn((T, d), generator=gc).to(dt)
    w1 = torch.empty((E, d, 2 * ff), device=dev, dtype=dt).normal_(0.0, 0.02, generator=gd)
    w2 = torch.empty((E, ff, d), device=dev, dtype=dt).normal_(0.0, 0.02, generator=gd)
    logits = torch.randn((T, E), generator=gc)
    if zipf is not None:
        # expert loads ~ rank^-zipf over a seeded permutation of the experts
        rank = torch.randperm(E, generator=gc).float() + 1.0
        p = rank.pow(-zipf)
        logits = logits + torch.log(p / p.sum())
    scores, idx = moe_ref.route_from_logits(logits, k, True, True, dt)
    return x, dout, w1, w2, scores, idx


def _token_subset(idx, E, n_random, gen):
    """A few tokens of every expert that has any (so that near-empty experts are checked),
    plus random ones."""
    T = idx.size(0)
    picked = set(torch.randperm(T, generator=gen)[:n_random].tolist())
    for e in range(E):
        rows = torch.nonzero((idx == e).any(-1)).flatten()
        if rows.numel():
            picked.add(int(rows[0]))
            picked.add(int(rows[-1]))
    return torch.tensor(sorted(picked))


def _torch_fp32_on_gpu(x, w1, w2, scores, idx, dout, E, k):
    """The per-expert loop of topk_moe.py:67-102 (SwiGLU on the interleaved layout of
    functional/activation.py:19-20) and its autograd backward, plain PyTorch fp32 on the GPU.
    Returns out, dx, dw1, dw2, dscores."""
    xs, w1s, w2s, ss = (t.detach().float().requires_grad_(True) for t in (x, w1, w2, scores))
    flat = idx.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    ends = torch.bincount(flat, minlength=E).cumsum(0).tolist()
    out = torch.zeros((x.size(0), w2.size(2)), device=x.device)
    start = 0
    for e, end in enumerate(ends):
        if end > start:
            sl = order[start:end]
            tok = sl // k
            h = xs[tok] @ w1s[e]
            a = torch.nn.functional.silu(h[:, 0::2]) * h[:, 1::2]
            out = out.index_add(0, tok, (a @ w2s[e]) * ss.reshape(-1)[sl].unsqueeze(1))
        start = end
    out.backward(dout.float())
    return out.detach(), xs.grad, w1s.grad, w2s.grad, ss.grad


def _tile_errors(got, ref, tile=256):
    """Relative Frobenius error of every tile x tile block of every expert's [rows, cols]
    matrix (edge blocks included), as a tensor [E, row blocks, column blocks]."""
    E, rows, cols = ref.shape
    pr, pc = -rows % tile, -cols % tile
    diff = torch.nn.functional.pad((got.float() - ref).pow(2), (0, pc, 0, pr))
    base = torch.nn.functional.pad(ref.pow(2), (0, pc, 0, pr))
    shape = (E, (rows + pr) // tile, tile, (cols + pc) // tile, tile)
    return (diff.view(shape).sum((2, 4)) / base.view(shape).sum((2, 4)).clamp_min(1e-30)).sqrt()


def _check(name, T, d, ff, E, k, zipf, seed):
    from moe_explore.functional.topk_moe import routed_experts
    x, dout, w1, w2, scores, idx = _inputs(T, d, ff, E, k, zipf, seed)
    counts = torch.bincount(idx.flatten(), minlength=E)
    print(f"{name}: rows per expert {counts.min().item()}..{counts.max().item()}", flush=True)
    if zipf is not None:
        assert counts.min() < 64 and counts.max() > 8 * counts.float().mean() / 4, \
            "the routing is not skewed enough to test the balanced deal"
    xc = x.cuda().requires_grad_(True)
    w1c, w2c = w1.requires_grad_(True), w2.requires_grad_(True)
    sc = scores.cuda().requires_grad_(True)
    out = routed_experts(xc, w1c, w2c, sc, idx.cuda(), E, k, "swiglu")
    out.backward(dout.cuda())
    torch.cuda.synchronize()
    for t in (out, xc.grad, w1c.grad, w2c.grad, sc.grad):
        assert torch.isfinite(t.float()).all()

    # --- tokens: out, dX, dscores against the oracle with the full weights
    gen = torch.Generator().manual_seed(seed + 1)
    sel = _token_subset(idx, E, 24, gen)
    w1_cpu, w2_cpu = w1.detach().cpu(), w2.detach().cpu()
    ref_out, ref_dx, _, _, ref_ds = moe_ref.experts_backward(
        x[sel], w1_cpu, w2_cpu, scores[sel], idx[sel], E, k, "swiglu", dout[sel])
    sel_c = sel.cuda()
    assert_parity(out.detach()[sel_c], ref_out, torch.bfloat16, f"{name}: out", tol=BF16_TOL)
    assert_parity(xc.grad[sel_c], ref_dx, torch.bfloat16, f"{name}: dX", tol=BF16_TOL)
    assert_parity(sc.grad[sel_c], ref_ds, torch.bfloat16, f"{name}: dscores", tol=BF16_TOL)

    # --- GLU columns: dW1 / dW2 slices of every expert against the oracle over all tokens
    edge = [0, 1, 127, 128, 255, 256, ff - 129, ff - 128, ff - 2, ff - 1]
    rnd = torch.randperm(ff, generator=gen)[:6].tolist()
    J = torch.tensor(sorted(set(j for j in edge + rnd if 0 <= j < ff)))
    cols = torch.stack((2 * J, 2 * J + 1), dim=1).flatten()        # gate, up of every j in J
    _, _, ref_dw1, ref_dw2, _ = moe_ref.experts_backward(
        x, w1_cpu[:, :, cols], w2_cpu[:, J, :], scores, idx, E, k, "swiglu", dout)
    got_dw1 = w1c.grad[:, :, cols.cuda()].float().cpu()
    got_dw2 = w2c.grad[:, J.cuda(), :].float().cpu()
    assert_parity(got_dw1, ref_dw1, torch.bfloat16, f"{name}: dW1 columns", tol=BF16_TOL)
    assert_parity(got_dw2, ref_dw2, torch.bfloat16, f"{name}: dW2 rows", tol=BF16_TOL)
    # every expert on its own: a misplaced or dropped tile of a small expert would vanish in
    # the norm over all experts
    for e in range(E):
        if counts[e] == 0:
            assert (w1c.grad[e] == 0).all() and (w2c.grad[e] == 0).all(), f"expert {e} has no rows"
            continue
        assert_parity(got_dw1[e], ref_dw1[e], torch.bfloat16, f"{name}: dW1 expert {e} "
                      f"({counts[e].item()} rows)", tol=BF16_TOL)
        assert_parity(got_dw2[e], ref_dw2[e], torch.bfloat16, f"{name}: dW2 expert {e} "
                      f"({counts[e].item()} rows)", tol=BF16_TOL)
    # --- every element: the fp32 PyTorch loop on the GPU, pinned to the oracle on the same
    # restrictions, then compared with the HIP results as whole tensors, per expert and per tile
    t_out, t_dx, t_dw1, t_dw2, t_ds = _torch_fp32_on_gpu(x.cuda(), w1.detach(), w2.detach(), scores.cuda(),
                                                          idx.cuda(), dout.cuda(), E, k)
    for what, got, want in (("out", t_out[sel_c], ref_out), ("dX", t_dx[sel_c], ref_dx),
                            ("dscores", t_ds[sel_c], ref_ds),
                            ("dW1 columns", t_dw1[:, :, cols.cuda()], ref_dw1),
                            ("dW2 rows", t_dw2[:, J.cuda(), :], ref_dw2)):
        assert_parity(got.cpu(), want, torch.float32, f"{name}: GPU fp32 loop vs oracle, {what}", tol=1e-4)
    assert_parity(out.detach(), t_out, torch.bfloat16, f"{name}: out, all tokens", tol=BF16_TOL)
    assert_parity(xc.grad, t_dx, torch.bfloat16, f"{name}: dX, all tokens", tol=BF16_TOL)
    assert_parity(sc.grad, t_ds, torch.bfloat16, f"{name}: dscores, all tokens", tol=BF16_TOL)
    assert_parity(w1c.grad, t_dw1, torch.bfloat16, f"{name}: dW1, whole", tol=BF16_TOL)
    assert_parity(w2c.grad, t_dw2, torch.bfloat16, f"{name}: dW2, whole", tol=BF16_TOL)
    live = (counts > 0).cuda()
    for what, got, want in (("dW1", w1c.grad, t_dw1), ("dW2", w2c.grad, t_dw2)):
        err = _tile_errors(got, want)[live]
        worst = err.max().item()
        assert worst <= BF16_TOL, f"{name}: {what}: a 256 x 256 tile is off by {worst:.3e} " \
                                  f"(expert, row block, column block) = {tuple((err == err.max()).nonzero()[0].tolist())}"
    # rows of 256 tokens of out / dX likewise (a dropped row block of a small expert)
    for what, got, want in (("out", out.detach(), t_out), ("dX", xc.grad, t_dx)):
        err = _tile_errors(got[None], want[None])
        assert err.max().item() <= BF16_TOL, f"{name}: {what}: a 256 x 256 tile is off by {err.max().item():.3e}"


def test_backward_config1_mixtral_full_size():
    _check("config 1", 4096, 4096, 14336, 8, 2, None, seed=11)


def test_backward_config2_olmoe_full_size():
    _check("config 2", 8192, 2048, 1024, 64, 8, None, seed=12)


def test_backward_config3_zipf_full_size():
    _check("config 3", 16384, 2048, 1408, 64, 6, 1.2, seed=13)
