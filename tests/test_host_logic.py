"""Host-side mirror of the reference's Python API: records, router, activations,
test helpers; all plain PyTorch on the CPU."""
import dataclasses

import pytest
import torch
import torch.nn.functional as F

from util import seeded


def test_param_records_keep_the_reference_field_order():
    from moe_explore.params import (MLPParams, GLUParams, GLUInterleavedParams, TopkRouterParams,
                                    ErnieRouterParams, MOEParams)
    from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams
    names = lambda c: [f.name for f in dataclasses.fields(c)]
    assert names(MLPParams) == ["weight1", "weight2", "activation"]
    assert names(GLUParams) == ["gate_weight", "up_weight", "down_weight", "activation"]
    assert names(GLUInterleavedParams) == ["interleaved_weight", "down_weight", "activation"]
    assert names(TopkRouterParams) == ["router_weight", "topk", "softmax_before_topk", "normalize_routing"]
    assert names(ErnieRouterParams) == ["router_weight", "bias", "topk"]
    assert names(MOEParams)[:4] == ["router_params", "expert_params", "num_experts", "topk"]
    assert names(MGroupedGEMMParams) == ["weight", "group_indices", "permute_indices", "gather", "scatter",
                                         "num_tokens", "topk", "shared_weight", "scales", "activation"]


def test_activation_enum_behaves_like_a_string():
    from moe_explore.functional.activation import Activation, activation
    assert Activation.SWIGLU == "swiglu" and "glu" in Activation.GEGLU
    assert "silu" in [a.value for a in Activation]
    x = torch.randn((4, 8), generator=seeded(0))
    assert torch.equal(activation(x, "silu"), F.silu(x))
    assert torch.equal(activation(x, Activation.GELU), F.gelu(x))
    assert torch.equal(activation(x, "swiglu"), F.silu(x[:, 0::2]) * x[:, 1::2])
    with pytest.raises(AssertionError):
        activation(x, "relu")


def test_routers_on_cpu():
    from moe_explore.params import TopkRouterParams, ErnieRouterParams
    from moe_explore.router import router
    g = seeded(1)
    x = torch.randn((17, 32), generator=g)
    wr = torch.randn((32, 8), generator=g)
    s, i = router(x, TopkRouterParams(wr, 2, True, True))
    assert s.shape == (17, 2) and i.dtype == torch.int64
    torch.testing.assert_close(s.sum(-1), torch.ones(17))
    s, i = router(x, ErnieRouterParams(wr, torch.zeros(8), 3))
    torch.testing.assert_close(s.sum(-1), torch.ones(17))
    with pytest.raises(ValueError):
        router(x, object())


def test_topk_moe_torch_matches_the_oracle_on_cpu():
    from moe_explore.functional.topk_moe import topk_moe_torch
    from moe_explore.params import MOEParams, MLPParams, TopkRouterParams
    from oracle import moe_ref
    g = seeded(2)
    T, d, ff, E, k = 64, 32, 48, 8, 2
    x = torch.randn((T, d), generator=g)
    w1 = torch.randn((E, d, 2 * ff), generator=g) * 0.1
    w2 = torch.randn((E, ff, d), generator=g) * 0.1
    wr = torch.randn((d, E), generator=g)
    params = MOEParams(TopkRouterParams(wr, k, True, False), MLPParams(w1, w2, "swiglu"), E, k)
    out = topk_moe_torch(x, params)
    ref, _, _ = moe_ref.topk_moe(x, wr, w1, w2, E, k, "swiglu")
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)


def test_testing_helpers():
    from moe_explore import testing
    gi = testing.random_groups(100, 5, "cpu")
    assert gi[0] == 0 and gi[-1] == 100 and (gi[1:] >= gi[:-1]).all() and gi.dtype == torch.int32
    s, i = testing.perfect_routing(16, 4, 2, "cpu", torch.float32)
    assert torch.bincount(i, minlength=4).tolist() == [8, 8, 8, 8]
    s, i = testing.random_zipf_routing(4096, 64, 6, "cpu", torch.float32, generator=seeded(3))
    c = torch.bincount(i.reshape(-1), minlength=64)
    assert c.max() > 10 * max(int(c.min()), 1)
    w = testing.uniform_weight_init((4, 8, 16), "cpu", torch.float32)
    assert w.abs().max() <= (3 ** 0.5) * (2 / 24) ** 0.5
    a = torch.ones(4, 4)
    testing.assert_close(a, a.clone())
    with pytest.raises(AssertionError):
        testing.assert_close(a, a + 1)


@pytest.mark.parametrize("gather,scatter,act", [(False, False, None), (True, False, "swiglu"),
                                                (False, True, None), (False, False, "gelu")])
def test_package_op_level_loop_matches_the_oracle(gather, scatter, act):
    """moe_explore.testing.torch_grouped_matmul_gather_scatter (the reference's comparison
    implementation, testing.py:9-50, as the package ships it) against the oracle's."""
    from moe_explore.testing import torch_grouped_matmul_gather_scatter
    from moe_explore.triton_kernels.m_grouped_gemm import MGroupedGEMMParams
    from oracle import moe_ref
    g = seeded(5)
    T, E, k, K, N = 40, 4, 2, 16, 24
    _, idx = moe_ref.route_from_logits(torch.randn((T, E), generator=g), k)
    gi, ind = moe_ref.get_token_indices(idx, k, E, zero_prefix=True)
    rows = T if gather else T * k
    a = torch.randn((rows, K), generator=g)
    w = torch.randn((E, K, N), generator=g)
    scales = torch.rand((T, k), generator=g) if scatter else None
    p = MGroupedGEMMParams(w, gi, ind if (gather or scatter) else None, gather, scatter,
                           T if (gather or scatter) else rows, k, scales=scales, activation=act)
    out = torch_grouped_matmul_gather_scatter(a, p)
    ref = moe_ref.grouped_matmul_gather_scatter(a, w, gi, p.permute_indices, gather, scatter, T, k,
                                                scales, act)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)


def test_separate_gate_up_weights_are_never_served_stale_on_cpu():
    """Whatever route an update takes (in place, through .data, which leaves the version
    counter alone, or a new storage), the next call interleaves the values of that moment."""
    from moe_explore.functional import topk_moe as layer
    from moe_explore.params import GLUParams
    g = seeded(6)
    gate, up, down = (torch.randn(s, generator=g) for s in ((3, 8, 6), (3, 8, 6), (3, 6, 8)))
    ep = GLUParams(gate, up, down, "swiglu")
    w_a = layer.expert_weights(ep)[0]
    assert torch.equal(w_a[..., 0::2], gate) and torch.equal(w_a[..., 1::2], up)
    up.add_(1.0)
    assert torch.equal(layer.expert_weights(ep)[0][..., 1::2], up)
    version = gate._version
    gate.data.mul_(2.0)
    up.data.copy_(torch.randn(3, 8, 6, generator=g))
    assert gate._version == version
    w_b = layer.expert_weights(ep)[0]
    assert torch.equal(w_b[..., 0::2], gate) and torch.equal(w_b[..., 1::2], up)
    gate.requires_grad_(True)
    gate.data.add_(1.0)
    w_c = layer.expert_weights(ep)[0]
    assert torch.equal(w_c.detach()[..., 0::2], gate.detach())
    w_c.sum().backward()
    assert torch.equal(gate.grad, torch.ones_like(gate))
    assert layer.to_interleaved(ep).interleaved_weight.shape == (3, 8, 12)


def test_stage_ranges_are_off_by_default_and_nest():
    from moe_explore import tracing
    assert not tracing.enabled()
    with tracing.scope("router"):
        pass


@pytest.mark.parametrize("gather", [False, True])
def test_grouped_glu_helper_matches_the_interleaved_oracle(gather):
    """testing.torch_grouped_glu (separate gate / up weights, testing.py:52-85) against the oracle's
    grouped product on the interleaved weight with the GLU epilogue."""
    from types import SimpleNamespace
    from moe_explore.functional.activation import glu_form
    from moe_explore.testing import torch_grouped_glu
    from oracle import moe_ref
    g = torch.Generator().manual_seed(9)
    T, E, k, K, N = 37, 5, 2, 24, 16
    gate = torch.randn((E, K, N), generator=g)
    up = torch.randn((E, K, N), generator=g)
    w = torch.stack((gate, up), dim=-1).reshape(E, K, 2 * N)
    if gather:
        idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
        gi, perm = moe_ref.get_token_indices(idx, k, E, zero_prefix=True)
        a = torch.randn((T, K), generator=g)
    else:
        perm = None
        gi = torch.tensor([0, 4, 4, 20, 30, 37], dtype=torch.int32)
        a = torch.randn((37, K), generator=g)
    for act in ("silu", "gelu"):
        p = SimpleNamespace(gate_weight=gate, up_weight=up, group_indices=gi, permute_indices=perm,
                            gather=gather, topk=k if gather else 1, activation=act)
        got = torch_grouped_glu(a, p)
        want = moe_ref.grouped_matmul_gather_scatter(a, w, gi, perm, gather=gather, topk=k if gather else 1,
                                                     activation_name=glu_form(act))
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
