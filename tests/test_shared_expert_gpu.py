"""Rows f2 of the layer: the shared-expert branch (reference topk_moe.py:56-62: every token
through S dense FFNs whose outputs are summed over S and added to the routed output), experts
without an activation, and separate gate / up weights (GLUParams) interleaved once."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity, randn, seeded

pytestmark = pytest.mark.gpu


def _shared_ref(x, up, down, act):
    """h = x @ up[s]; h = act(h); h = h @ down[s]; sum over s (topk_moe.py:58-61), in the
    dtype of x (callers pass fp32 for 16-bit layers and fp64 for fp32 layers)."""
    out = torch.zeros(x.size(0), down.size(-1), dtype=x.dtype)
    for s in range(up.size(0)):
        out = out + moe_ref.activation(x @ up[s], act) @ down[s]
    return out


@pytest.mark.parametrize("S,act,dtype,T,d,ffs", [
    (1, "swiglu", torch.bfloat16, 300, 256, 384),
    (2, "swiglu", torch.bfloat16, 1100, 256, 192),
    (3, "silu", torch.float16, 200, 128, 96),
    (2, "geglu", torch.float32, 150, 64, 80),
    (1, "gelu", torch.float32, 64, 32, 48),
])
def test_shared_expert_forward_backward(S, act, dtype, T, d, ffs):
    from moe_explore.functional.topk_moe import topk_moe_forward
    from moe_explore.params import MLPParams, MOEParams, SharedExpertParams, TopkRouterParams
    g = seeded(S * 100 + T)
    E, k, ff = 8, 2, 128
    glu = "glu" in act
    x = randn((T, d), g, dtype)
    w1 = randn((E, d, 2 * ff if glu else ff), g, dtype, 0.1)
    w2 = randn((E, ff, d), g, dtype, 0.1)
    wr = randn((d, E), g, dtype, 0.1)
    up = randn((S, d, 2 * ffs if glu else ffs), g, dtype, 0.1)
    down = randn((S, ffs, d), g, dtype, 0.1)
    dout = randn((T, d), g, dtype)
    xc = x.cuda().requires_grad_(True)
    upc, downc = up.cuda().requires_grad_(True), down.cuda().requires_grad_(True)
    params = MOEParams(TopkRouterParams(wr.cuda(), k, True, True), MLPParams(w1.cuda(), w2.cuda(), act),
                       E, k, SharedExpertParams(upc, downc, act))
    out = topk_moe_forward(xc, params)
    assert out.shape == (T, d) and out.dtype == dtype
    plain = topk_moe_forward(x.cuda(), MOEParams(params.router_params, params.expert_params, E, k))
    out.backward(dout.cuda())
    # the oracle of the shared branch alone: routed part subtracted on both sides
    cd = torch.float64 if dtype == torch.float32 else torch.float32
    xr = x.to(cd).requires_grad_(True)
    upr, downr = up.to(cd).requires_grad_(True), down.to(cd).requires_grad_(True)
    ref = _shared_ref(xr, upr, downr, act)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    # (a difference of two layer outputs: each carries its own rounding, hence twice the bar)
    assert_parity((out.detach().to(cd) - plain.to(cd)), ref.detach(), dtype, "shared branch", tol=2 * tol)
    # gradients of the shared weights come from the shared branch alone
    ref.backward(dout.to(cd))
    assert_parity(upc.grad, upr.grad, dtype, "d up_weight", tol=tol)
    assert_parity(downc.grad, downr.grad, dtype, "d down_weight", tol=tol)
    # dX of the whole layer = routed part (own test elsewhere) + shared part
    x2 = x.cuda().requires_grad_(True)
    topk_moe_forward(x2, MOEParams(params.router_params, params.expert_params, E, k)).backward(dout.cuda())
    assert_parity(xc.grad.to(cd) - x2.grad.to(cd), xr.grad, dtype, "dX of the shared branch", tol=2 * tol)


def test_shared_expert_two_dimensional_weights_are_one_expert():
    from moe_explore.functional.topk_moe import shared_experts
    from moe_explore.params import SharedExpertParams
    g = seeded(2)
    x = randn((96, 64), g, torch.bfloat16)
    up, down = randn((64, 2 * 80), g, torch.bfloat16, 0.1), randn((80, 64), g, torch.bfloat16, 0.1)
    out = shared_experts(x.cuda(), SharedExpertParams(up.cuda(), down.cuda(), "swiglu"))
    assert_parity(out, _shared_ref(x.float(), up[None].float(), down[None].float(), "swiglu"), torch.bfloat16,
                  "2-D shared weights")


@pytest.mark.parametrize("dtype,T,d,ff,E,k", [
    (torch.float32, 200, 64, 96, 8, 2), (torch.bfloat16, 1300, 256, 320, 4, 2), (torch.float16, 300, 128, 128, 16, 4),
])
def test_experts_without_activation_forward_backward(dtype, T, d, ff, E, k):
    """MLPParams.activation = None is a legal layer (params.py:11-15): the experts are two
    linear maps.  dH = s * G, s * A = s * H, dscore = <G, H>."""
    from moe_explore.functional.topk_moe import routed_experts
    g = seeded(T + ff)
    x = randn((T, d), g, dtype)
    w1, w2 = randn((E, d, ff), g, dtype, 0.1), randn((E, ff, d), g, dtype, 0.1)
    scores, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k, True, True, dtype)
    dout = randn((T, d), g, dtype)
    xc, w1c, w2c, sc = (t.cuda().requires_grad_(True) for t in (x, w1, w2, scores))
    out = routed_experts(xc, w1c, w2c, sc, idx.cuda(), E, k, None)
    out.backward(dout.cuda())
    ref_out, dx, dw1, dw2, ds = moe_ref.experts_backward(
        x, w1, w2, scores, idx, E, k, None, dout,
        compute_dtype=torch.float64 if dtype == torch.float32 else torch.float32)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for name, got, want in (("out", out, ref_out), ("dx", xc.grad, dx), ("dw1", w1c.grad, dw1),
                            ("dw2", w2c.grad, dw2), ("dscores", sc.grad, ds)):
        assert_parity(got, want, dtype, name, tol=tol)


def test_separate_gate_up_weights():
    """GLUParams (params.py:16-21, the Hugging Face layout): interleaved on every call, so an
    update of gate or up by any route is seen; gradients come back per tensor."""
    from moe_explore.functional import topk_moe as layer
    from moe_explore.params import GLUInterleavedParams, GLUParams, MOEParams, TopkRouterParams
    g = seeded(31)
    T, d, ff, E, k = 256, 128, 192, 8, 2
    dt = torch.bfloat16
    x = randn((T, d), g, dt).cuda()
    gate, up = randn((E, d, ff), g, dt, 0.1).cuda(), randn((E, d, ff), g, dt, 0.1).cuda()
    down = randn((E, ff, d), g, dt, 0.1).cuda()
    rp = TopkRouterParams(randn((d, E), g, dt, 0.1).cuda(), k, True, True)
    ep = GLUParams(gate, up, down, "swiglu")
    w_a, _, _ = layer.expert_weights(ep)
    assert torch.equal(w_a[:, :, 0::2], gate) and torch.equal(w_a[:, :, 1::2], up)
    out = layer.topk_moe_forward(x, MOEParams(rp, ep, E, k))
    same = layer.topk_moe_forward(x, MOEParams(rp, layer.to_interleaved(ep), E, k))
    assert isinstance(layer.to_interleaved(ep), GLUInterleavedParams)
    assert torch.equal(out, same)
    # updates that leave the version counter alone (through .data, as optimisers with master
    # weights do) are seen as well: no copy outlives a call
    gate.data.mul_(0.5)
    up.data.copy_(up.data * 2)
    w_c, _, _ = layer.expert_weights(ep)
    assert torch.equal(w_c[:, :, 0::2], gate) and torch.equal(w_c[:, :, 1::2], up)
    # gradients: d gate / d up are the even / odd columns of d weight1
    gate.requires_grad_(True)
    up.requires_grad_(True)
    dout = randn((T, d), g, dt).cuda()
    layer.topk_moe_forward(x, MOEParams(rp, ep, E, k)).backward(dout)
    w1 = layer.interleave_glu_weights(gate.detach(), up.detach()).requires_grad_(True)
    layer.topk_moe_forward(x, MOEParams(rp, GLUInterleavedParams(w1, down, "swiglu"), E, k)).backward(dout)
    assert torch.equal(gate.grad, w1.grad[:, :, 0::2]) and torch.equal(up.grad, w1.grad[:, :, 1::2])
