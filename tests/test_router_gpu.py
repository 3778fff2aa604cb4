"""Fused router kernel (moe_router_topk / moe_router_bwd through the package's
topk_router / ernie_router) against the CPU oracle's restatement of the reference's
routers (router.py:17-54).

Selections are compared where the oracle's own decision is not a near-tie: the k-th and
(k+1)-th largest selection keys must differ by more than the rounding noise of the logits
for a token to be checked index by index; every token is checked for valid, distinct
indices and for scores that match the oracle's scores of the experts the kernel chose."""
import pytest
import torch

from oracle import moe_ref
from tests.util import seeded

pytestmark = pytest.mark.gpu

# (T, d, E, topk)
SHAPES = [(512, 256, 8, 2), (1000, 512, 64, 8), (96, 1024, 128, 8), (70, 264, 256, 16),
          (33, 72, 5, 3), (2048, 2048, 64, 6), (64, 128, 4, 4), (1, 64, 8, 2)]
# more than 256 experts: two chunks of 256 handled by different wavefronts
MANY_EXPERTS = [(200, 512, 384, 8), (100, 1024, 512, 16), (77, 256, 500, 6), (130, 2048, 320, 8), (40, 512, 257, 4)]


def _inputs(T, d, E, dtype, seed, w_dtype=None):
    g = seeded(seed)
    x = torch.randn((T, d), generator=g).to(dtype)
    w = (torch.randn((d, E), generator=g) * d ** -0.5).to(w_dtype or dtype)
    return x, w


def _check(scores, idx, x, w, topk, softmax_first, normalize, bias=None):
    """scores/idx from the GPU (already on the CPU) against the oracle on the same inputs."""
    T, E = x.size(0), w.size(1)
    dtype = x.dtype
    assert idx.dtype == torch.int64 and scores.dtype == dtype
    assert idx.shape == scores.shape == (T, topk)
    assert (idx >= 0).all() and (idx < E).all()
    assert (torch.sort(idx, -1).values.diff(dim=-1) > 0).all(), "an expert chosen twice"
    if bias is None:
        logits = (x @ w).float()   # matmul in the input dtype, as router.py:22
        key = torch.softmax(logits, -1) if softmax_first else logits
        probs = key
    else:
        logits = x.float() @ w
        probs = torch.softmax(logits, -1)
        key = probs + bias
    # index parity where the oracle's choice is clear of rounding noise: the logits carry
    # an error of a few ulps of their dtype (other summation order), relative to the key
    srt = torch.sort(key, -1, descending=True).values
    kth = srt[:, topk - 1]
    noise = 4 * max(torch.finfo(dtype).eps, 16 * torch.finfo(torch.float32).eps) * \
        (kth.abs() if (softmax_first or bias is not None) else srt[:, 0].abs().clamp_min(1.0))
    if topk < E:
        clear = (kth - srt[:, topk]) > noise
    else:
        clear = torch.ones(T, dtype=torch.bool)
    # every token: the chosen experts are top-k up to the noise (none below the k-th key by
    # more than it, and no expert above the k-th key by more than it left out)
    chosen_mask = torch.zeros((T, E), dtype=torch.bool).scatter_(1, idx, True)
    assert (torch.gather(key, 1, idx) >= (kth - noise)[:, None]).all()
    assert not ((key > (kth + noise)[:, None]) & ~chosen_mask).any()
    want_idx = torch.topk(key, topk, -1).indices
    assert torch.equal(torch.sort(idx[clear], -1).values, torch.sort(want_idx[clear], -1).values)
    # the kernel lists the experts in descending key order (up to the same noise)
    chosen = torch.gather(key, 1, idx)
    assert (chosen.diff(dim=-1) <= 4 * noise[:, None] + 1e-6).all()
    # scores of the experts the kernel chose, computed the oracle's way
    if bias is None and not softmax_first:
        raw = torch.softmax(torch.gather(logits, 1, idx), -1)
    else:
        raw = torch.gather(probs, 1, idx)
    if bias is not None:
        raw = raw / raw.sum(-1, keepdim=True).clamp_min(1e-12)
    elif normalize:
        raw = raw / raw.sum(-1, keepdim=True)
    tol = {torch.float32: 2e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    torch.testing.assert_close(scores.float(), raw.to(dtype).float(), rtol=tol, atol=tol * 0.1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("softmax_first,normalize", [(True, True), (True, False), (False, False)])
def test_topk_router_matches_oracle(shape, dtype, softmax_first, normalize):
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router, _fused_supported
    T, d, E, topk = shape
    x, w = _inputs(T, d, E, dtype, seed=T + E)
    assert _fused_supported(x.cuda(), w.cuda(), topk, False)
    s, i = topk_router(x.cuda(), TopkRouterParams(w.cuda(), topk, softmax_first, normalize))
    _check(s.cpu(), i.cpu(), x, w, topk, softmax_first, normalize)
    # the oracle's own entry point agrees with the reading of it above
    so, io = moe_ref.topk_router(x.float(), w.float(), topk, softmax_first, normalize)
    assert so.shape == s.shape and io.shape == i.shape


@pytest.mark.parametrize("E,topk", [(16, 4), (64, 8), (160, 6)])
def test_masked_logits_are_chosen_last_and_never_twice(E, topk):
    """Top-k before the softmax over tokens with fewer than k finite logits (a feature that
    overflows to -inf for most experts): the finite experts are chosen, the rest of the k are
    distinct experts with logit -inf and score 0 -- in every form of the selection (keys in
    registers up to 16 experts a lane, in LDS beyond)."""
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router, _fused_supported
    T, d = 96, 64
    x, w = _inputs(T, d, E, torch.bfloat16, seed=E)
    finite = [3, E - 2]
    x[:, 0] = 1e38                       # times -100, summed in fp32: -inf
    w[0, :] = -100.0
    w[0, finite] = 0.0
    x, w = x.cuda(), w.cuda()
    assert _fused_supported(x, w, topk, False)
    s, i = topk_router(x, TopkRouterParams(w, topk, False, False))
    s, i = s.float().cpu(), i.cpu()
    assert (torch.sort(i, -1).values.diff(dim=-1) > 0).all(), "an expert chosen twice"
    assert (i >= 0).all() and (i < E).all()
    chosen = torch.zeros((T, E), dtype=torch.bool).scatter_(1, i, True)
    assert chosen[:, finite].all(), "a finite logit was passed over for a masked one"
    is_finite = torch.zeros(E, dtype=torch.bool)
    is_finite[finite] = True
    assert (s[~is_finite[i]] == 0).all()
    torch.testing.assert_close(s.sum(-1), torch.ones(T), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", MANY_EXPERTS)
@pytest.mark.parametrize("softmax_first,normalize", [(True, True), (False, False)])
def test_topk_router_more_than_256_experts(shape, dtype, softmax_first, normalize):
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router, _fused_supported
    T, d, E, topk = shape
    x, w = _inputs(T, d, E, dtype, seed=T + E)
    assert _fused_supported(x.cuda(), w.cuda(), topk, False)
    s, i = topk_router(x.cuda(), TopkRouterParams(w.cuda(), topk, softmax_first, normalize))
    _check(s.cpu(), i.cpu(), x, w, topk, softmax_first, normalize)


def test_ernie_router_and_backward_with_384_experts():
    """The bias path, the saved logits and the gradient of the scores with 384 experts."""
    from moe_explore.params import ErnieRouterParams, TopkRouterParams
    from moe_explore.router import ernie_router, topk_router
    T, d, E, topk = 150, 512, 384, 8
    x, w = _inputs(T, d, E, torch.bfloat16, seed=384, w_dtype=torch.float32)
    bias = torch.randn(E, generator=seeded(5)) * 0.01
    s, i = ernie_router(x.cuda(), ErnieRouterParams(w.cuda(), bias.cuda(), topk))
    _check(s.cpu(), i.cpu(), x, w, topk, True, True, bias=bias)
    xg = x.float().clone().cuda().requires_grad_(True)
    wg = w.clone().cuda().requires_grad_(True)
    sg, ig = topk_router(xg, TopkRouterParams(wg, topk, True, True))
    g = torch.randn(sg.shape, generator=seeded(6))
    sg.backward(g.cuda())
    # fp32 router: 1e-5 against autograd in fp64 (logits rounded to fp32 as the kernel's are)
    xr = x.double().requires_grad_(True)
    wr = w.double().requires_grad_(True)
    logits = xr @ wr
    logits = logits + (logits.float().double() - logits).detach()
    pr = torch.softmax(logits, -1)
    sr = torch.gather(pr, 1, ig.cpu())
    sr = sr / sr.sum(-1, keepdim=True)
    sr.backward(g.double())
    assert moe_ref.rel_fro(xg.grad.cpu(), xr.grad) <= 1e-5
    assert moe_ref.rel_fro(wg.grad.cpu(), wr.grad) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES[:5])
def test_ernie_router_matches_oracle(shape, dtype):
    from moe_explore.params import ErnieRouterParams
    from moe_explore.router import ernie_router
    T, d, E, topk = shape
    x, w = _inputs(T, d, E, dtype, seed=3 * T + E, w_dtype=torch.float32)
    bias = torch.randn(E, generator=seeded(5)) * 0.05
    s, i = ernie_router(x.cuda(), ErnieRouterParams(w.cuda(), bias.cuda(), topk))
    _check(s.cpu(), i.cpu(), x, w, topk, True, True, bias=bias)
    so, io = moe_ref.ernie_router(x, w, bias, topk)
    both = torch.sort(i.cpu(), -1).values == torch.sort(io, -1).values
    assert both.all(-1).float().mean() > 0.97


def test_logits_output_and_strided_weight():
    """The saved logits are the dtype-rounded x @ w; a transposed-view weight ([E, d] storage,
    as nn.Linear keeps it) gives the same result as a contiguous one."""
    from moe_explore.router import _fused_forward
    from moe_explore import _C
    T, d, E, topk = 300, 512, 64, 4
    x, w = _inputs(T, d, E, torch.bfloat16, seed=9)
    flags = _C.ROUTER_SOFTMAX_FIRST | _C.ROUTER_NORMALIZE
    s1, i1, l1 = _fused_forward(x.cuda(), w.cuda(), None, topk, flags, True)
    wt = w.t().contiguous().cuda().t()   # same values, strides (1, d)
    assert wt.stride() == (1, d)
    s2, i2, l2 = _fused_forward(x.cuda(), wt, None, topk, flags, True)
    assert torch.equal(i1, i2) and torch.equal(s1, s2) and torch.equal(l1, l2)
    want = (x.float() @ w.float())
    torch.testing.assert_close(l1.cpu(), want, rtol=1e-2, atol=1e-2)
    assert torch.equal(l1.cpu(), l1.cpu().to(torch.bfloat16).float()), "logits not rounded to bf16"


@pytest.mark.parametrize("mode", ["softmax_first_norm", "softmax_first", "topk_first", "ernie"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_backward_matches_autograd(mode, dtype):
    """dx and dW of the fused router against torch.autograd through the oracle's formulation,
    with the selection of the GPU run handed over (so that a tie cannot differ)."""
    from moe_explore.params import ErnieRouterParams, TopkRouterParams
    from moe_explore.router import router
    T, d, E, topk = 257, 128, 16, 4
    w_dtype = torch.float32 if mode == "ernie" else dtype
    x, w = _inputs(T, d, E, dtype, seed=21, w_dtype=w_dtype)
    bias = torch.randn(E, generator=seeded(6)) * 0.05
    g = torch.randn((T, topk), generator=seeded(7)).to(dtype)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    if mode == "ernie":
        params = ErnieRouterParams(wg, bias.cuda(), topk)
    else:
        params = TopkRouterParams(wg, topk, mode != "topk_first", mode == "softmax_first_norm")
    s, i = router(xg, params)
    s.backward(g.cuda())
    idx = i.cpu()
    # oracle: autograd through the same formulas with the same selection, in fp64 for the
    # fp32 router (held to 1e-5) and in fp32 for the 16-bit one
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    xr, wr = x.to(cd).requires_grad_(True), w.to(cd).requires_grad_(True)
    logits = xr @ wr
    if mode != "ernie":
        # the reference's matmul returns the logits in the dtype of x (router.py:22); rounding
        # has no gradient of its own (straight through)
        logits = logits + (logits.to(dtype).to(cd) - logits).detach()
    if mode == "topk_first":
        sr = torch.softmax(torch.gather(logits, 1, idx), -1)
    else:
        sr = torch.gather(torch.softmax(logits, -1), 1, idx)
        if mode == "softmax_first_norm":
            sr = sr / sr.sum(-1, keepdim=True)
        elif mode == "ernie":
            sr = sr / sr.sum(-1, keepdim=True).clamp_min(1e-12)
    sr.backward(g.to(cd))
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert moe_ref.rel_fro(xg.grad.cpu(), xr.grad) <= tol
    assert moe_ref.rel_fro(wg.grad.cpu(), wr.grad) <= tol


def test_unsupported_shapes_take_the_aten_path():
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router, _fused_supported
    x, w = _inputs(64, 100, 6, torch.bfloat16, seed=1)   # d % 8 != 0
    assert not _fused_supported(x.cuda(), w.cuda(), 2, False)
    s, i = topk_router(x.cuda(), TopkRouterParams(w.cuda(), 2, True, True))
    so, io = moe_ref.topk_router(x, w, 2, True, True)
    assert s.shape == so.shape and i.shape == io.shape


@pytest.mark.parametrize("E,topk", [(256, 8), (160, 6), (128, 8), (100, 4)])
def test_topk_router_many_tokens_and_65_to_256_experts(E, topk):
    """More 32-token blocks than compute units and 65-256 experts: the kernel forms with 64
    tokens a workgroup (129-256 experts: two groups of wavefronts, 128 experts each)."""
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router
    T, d = 32 * 300 + 17, 256
    x, w = _inputs(T, d, E, torch.bfloat16, seed=E)
    s, i = topk_router(x.cuda(), TopkRouterParams(w.cuda(), topk, True, True))
    _check(s.cpu(), i.cpu(), x, w, topk, True, True)


def test_router_weight_gradient_with_many_tokens():
    """From 8192 tokens on the router's weight gradient is a sum of partial products over token
    groups from the K-grouped kernel: against fp32 autograd with the same selection, at the bf16 bar."""
    from moe_explore.params import TopkRouterParams
    from moe_explore.router import topk_router
    T, d, E, topk = 8192 + 77, 256, 64, 8
    x, w = _inputs(T, d, E, torch.bfloat16, seed=31)
    g = torch.randn((T, topk), generator=seeded(8)).to(torch.bfloat16)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    s, i = topk_router(xg, TopkRouterParams(wg, topk, True, True))
    s.backward(g.cuda())
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    logits = xr @ wr
    logits = logits + (logits.to(torch.bfloat16).float() - logits).detach()
    sr = torch.gather(torch.softmax(logits, -1), 1, i.cpu())
    sr = sr / sr.sum(-1, keepdim=True)
    sr.backward(g.float())
    assert moe_ref.rel_fro(wg.grad.cpu(), wr.grad) <= 2e-2
    assert moe_ref.rel_fro(xg.grad.cpu(), xr.grad) <= 2e-2


@pytest.mark.parametrize("in_16_bits", [False, True])
def test_ernie_router_gradients_with_many_tokens(in_16_bits):
    """fp32 router weight under bf16 activations, 8192 tokens and more.  By default the weight
    gradient comes from fp32 products (1e-5 against autograd in fp64 with the same selection;
    dx leaves in bf16, at the bf16 bar); on request the backward products run on 16-bit
    operands (dW over token groups on the K-grouped kernel, returned in fp32), at the bf16 bar."""
    from moe_explore import router as router_module
    from moe_explore.params import ErnieRouterParams
    from moe_explore.router import ernie_router
    T, d, E, topk = 8192 + 33, 256, 64, 6
    x, w = _inputs(T, d, E, torch.bfloat16, seed=41, w_dtype=torch.float32)
    bias = torch.randn(E, generator=seeded(9)) * 0.05
    g = torch.randn((T, topk), generator=seeded(10)).to(torch.bfloat16)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    router_module.fp32_router_backward_in_16_bits(in_16_bits)
    try:
        s, i = ernie_router(xg, ErnieRouterParams(wg, bias.cuda(), topk))
        s.backward(g.cuda())
    finally:
        router_module.fp32_router_backward_in_16_bits(False)
    assert wg.grad.dtype == torch.float32 and xg.grad.dtype == torch.bfloat16
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    logits = xr @ wr
    logits = logits + (logits.float().double() - logits).detach()   # the kernel's fp32 logits
    sr = torch.gather(torch.softmax(logits, -1), 1, i.cpu())
    sr = sr / sr.sum(-1, keepdim=True).clamp_min(1e-12)
    sr.backward(g.double())
    assert moe_ref.rel_fro(wg.grad.cpu(), wr.grad) <= (2e-2 if in_16_bits else 1e-5)
    assert moe_ref.rel_fro(xg.grad.cpu(), xr.grad) <= 2e-2
