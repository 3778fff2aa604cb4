"""Independent end-to-end oracle: the sparse-MoE blocks of the locally installed
`transformers` modelling code (OLMoE, Mixtral, Qwen3-MoE, Ernie-4.5: the four the reference's
hf_moe_reference.py:15-120 wraps, Ernie here also WITH its shared experts, which the
reference switches off at :84-86), built from locally constructed configs
with seeded random weights (nothing is fetched), against the HIP layer on the same
weights.  The reference does the same against released configs (tests/test_hf.py:75-90,
hf_moe_reference.py); its weight mapping is mirrored here: separate gate / up weights
interleaved into the even / odd columns of weight1 (tests/test_hf.py:52-73)."""
import pytest
import torch

from oracle import moe_ref
from util import assert_parity

transformers = pytest.importorskip("transformers")


def _block(kind, hidden, inter, E, k, norm, shared=0):
    if kind == "olmoe":
        from transformers.models.olmoe.configuration_olmoe import OlmoeConfig
        from transformers.models.olmoe.modeling_olmoe import OlmoeSparseMoeBlock
        cfg = OlmoeConfig(hidden_size=hidden, intermediate_size=inter, num_experts=E,
                          num_experts_per_tok=k, norm_topk_prob=norm, hidden_act="silu")
        if not hasattr(cfg, "num_local_experts"):
            cfg.num_local_experts = E
        blk = OlmoeSparseMoeBlock(cfg)
    elif kind == "qwen3":
        from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
        from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock
        cfg = Qwen3MoeConfig(hidden_size=hidden, moe_intermediate_size=inter, intermediate_size=inter,
                             num_experts=E, num_experts_per_tok=k, norm_topk_prob=norm, hidden_act="silu")
        blk = Qwen3MoeSparseMoeBlock(cfg)
    elif kind == "ernie":
        from transformers.models.ernie4_5_moe.configuration_ernie4_5_moe import Ernie4_5_MoeConfig
        from transformers.models.ernie4_5_moe.modeling_ernie4_5_moe import Ernie4_5_MoeSparseMoeBlock
        cfg = Ernie4_5_MoeConfig(hidden_size=hidden, moe_intermediate_size=inter, intermediate_size=inter,
                                 moe_num_experts=E, moe_k=k, moe_num_shared_experts=shared,
                                 hidden_act="silu", use_bias=False)
        blk = Ernie4_5_MoeSparseMoeBlock(cfg)
    else:
        from transformers.models.mixtral.configuration_mixtral import MixtralConfig
        from transformers.models.mixtral.modeling_mixtral import MixtralSparseMoeBlock
        cfg = MixtralConfig(hidden_size=hidden, intermediate_size=inter, num_local_experts=E,
                            num_experts_per_tok=k, hidden_act="silu", router_jitter_noise=0.0)
        blk = MixtralSparseMoeBlock(cfg)
    g = torch.Generator().manual_seed(1234)
    with torch.no_grad():
        for name, prm in blk.named_parameters():
            if name.endswith("e_score_correction_bias"):
                # a selection bias of the size of the probabilities (1 / E): changes who is chosen
                prm.copy_(torch.rand(prm.shape, generator=g) * (2.0 / E))
            else:
                prm.copy_(torch.randn(prm.shape, generator=g) * (0.5 if prm.dim() == 2 else 0.05))
    return blk.eval().float()


def _moe_params(blk, k, norm, device, dtype):
    """HF layout -> this package's: router weight [d, E]; gate_up_proj [E, 2ff, d] (gate rows
    first) -> gate / up [E, d, ff]; down_proj [E, d, ff] -> [E, ff, d]; Ernie: fp32 router
    weight and selection bias, shared experts (one MLP of width S * ff: gate_proj / up_proj /
    down_proj) -> interleaved up_weight [1, d, 2 S ff], down_weight [1, S ff, d]."""
    from moe_explore.params import (ErnieRouterParams, GLUParams, MOEParams, SharedExpertParams,
                                    TopkRouterParams)
    E, two_ff, d = blk.experts.gate_up_proj.shape
    ff = two_ff // 2
    gu = blk.experts.gate_up_proj.detach()
    gate = gu[:, :ff, :].transpose(1, 2).contiguous()
    up = gu[:, ff:, :].transpose(1, 2).contiguous()
    down = blk.experts.down_proj.detach().transpose(1, 2).contiguous()
    wr = blk.gate.weight.detach().t().contiguous()
    cast = lambda t: t.to(device=device, dtype=dtype)
    statics = getattr(blk.gate, "moe_statics", None)
    if statics is not None:
        bias = statics.e_score_correction_bias.detach().reshape(-1)
        rp = ErnieRouterParams(wr.to(device=device, dtype=torch.float32),
                               bias.to(device=device, dtype=torch.float32), k)
    else:
        rp = TopkRouterParams(cast(wr), k, softmax_before_topk=True, normalize_routing=norm)
    sp = None
    mlp = getattr(blk, "shared_experts", None)
    if mlp is not None:
        sg, su = mlp.gate_proj.weight.detach().t(), mlp.up_proj.weight.detach().t()   # [d, S ff]
        w = torch.stack((sg, su), dim=-1).reshape(d, -1)                               # even = gate
        sp = SharedExpertParams(cast(w.unsqueeze(0).contiguous()),
                                cast(mlp.down_proj.weight.detach().t().unsqueeze(0).contiguous()), "swiglu")
    return MOEParams(rp, GLUParams(cast(gate), cast(up), cast(down), "swiglu"), E, k, sp)


def _oracle_layer(x, p):
    """The CPU oracle on the parameter record of `_moe_params` (fp32): router of either kind,
    expert loop, shared experts as dense fp32 matmuls."""
    from moe_explore.params import ErnieRouterParams
    ep, rp = p.expert_params, p.router_params
    E, d, ff = ep.gate_weight.shape
    w1 = torch.empty((E, d, 2 * ff))
    w1[:, :, 0::2], w1[:, :, 1::2] = ep.gate_weight, ep.up_weight
    if isinstance(rp, ErnieRouterParams):
        scores, idx = moe_ref.ernie_router(x, rp.router_weight, rp.bias, rp.topk)
    else:
        scores, idx = moe_ref.topk_router(x, rp.router_weight, rp.topk, rp.softmax_before_topk,
                                          rp.normalize_routing)
    out = moe_ref.experts_forward(x, w1, ep.down_weight, scores, idx, E, p.topk, "swiglu")
    sp = p.shared_expert_params
    if sp is not None:
        for s in range(sp.up_weight.size(0)):
            out = out + moe_ref.activation(x @ sp.up_weight[s], "swiglu") @ sp.down_weight[s]
    return out, scores, idx


BLOCKS = [("olmoe", False, 0), ("olmoe", True, 0), ("mixtral", True, 0), ("qwen3", False, 0),
          ("qwen3", True, 0), ("ernie", True, 0), ("ernie", True, 2)]


@pytest.mark.parametrize("kind,norm,shared", BLOCKS)
def test_oracle_matches_transformers_block(kind, norm, shared):
    """Pins the CPU oracle's layer (both routers, GLU column layout, per-expert loop, combine)
    against an implementation written by someone else."""
    hidden, inter, E, k, seq = 128, 160, 8, 2, 64
    blk = _block(kind, hidden, inter, E, k, norm, shared)
    x = torch.randn((1, seq, hidden), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        ref = blk(x)
    ref = ref[0] if isinstance(ref, tuple) else ref
    out, _, _ = _oracle_layer(x[0], _moe_params(blk, k, norm, "cpu", torch.float32))
    assert_parity(out, ref.reshape(seq, hidden), torch.float32, f"oracle vs {kind} block", tol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,norm,shared", BLOCKS)
def test_layer_matches_transformers_block_fp32(kind, norm, shared):
    from moe_explore.functional.topk_moe import topk_moe_forward
    hidden, inter, E, k, seq = 256, 320, 8, 2, 96
    blk = _block(kind, hidden, inter, E, k, norm, shared)
    x = torch.randn((1, seq, hidden), generator=torch.Generator().manual_seed(7))
    # the block itself in fp64 is the reference of the fp32 layer (1e-5)
    import copy
    with torch.no_grad():
        ref = copy.deepcopy(blk).double()(x.double())
    ref = ref[0] if isinstance(ref, tuple) else ref
    out = topk_moe_forward(x[0].cuda(), _moe_params(blk, k, norm, "cuda", torch.float32))
    assert_parity(out, ref.reshape(seq, hidden), torch.float32, f"{kind} block, fp32", tol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("E,k,shared", [(64, 6, 2), (16, 4, 0)])
def test_ernie_block_bf16(E, k, shared):
    """The Ernie-4.5 shape family end to end in bf16 (fp32 router with a selection bias, top-6
    of 64, two shared experts) against the block in fp32 on bf16-rounded weights.  The fused
    router's selection is checked first; tokens whose k-th and (k+1)-th keys nearly tie may
    legitimately differ, so the outputs are compared on the tokens where both chose alike."""
    from moe_explore.functional.topk_moe import topk_moe_forward
    from moe_explore.router import router
    hidden, inter, seq = 512, 256, 400
    blk = _block("ernie", hidden, inter, E, k, True, shared)
    with torch.no_grad():
        for name, prm in blk.named_parameters():
            if "gate.weight" not in name and "bias" not in name:
                prm.copy_(prm.to(torch.bfloat16).float())
    x = torch.randn((seq, hidden), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    params = _moe_params(blk, k, True, "cuda", torch.bfloat16)
    out = topk_moe_forward(x.cuda(), params)
    _, idx = router(x.cuda(), params.router_params)
    with torch.no_grad():
        ref = blk(x.float().unsqueeze(0))
        _, _, ref_idx = blk.gate(x.float())
    ref = (ref[0] if isinstance(ref, tuple) else ref).reshape(seq, hidden)
    same = (torch.sort(idx.cpu(), -1).values == torch.sort(ref_idx, -1).values).all(-1)
    assert same.float().mean() > 0.97, "router selections differ on more than near-ties"
    assert_parity(out.cpu()[same], ref[same], torch.bfloat16, "ernie block, bf16", tol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["olmoe", "mixtral"])
def test_experts_match_transformers_experts_bf16(kind):
    """bf16 on the GPU against the block's expert module in fp32 on bf16-rounded weights,
    with the routing decisions handed over (a bf16 router may break near-ties differently)."""
    from moe_explore.functional.topk_moe import expert_weights, routed_experts
    from moe_explore.router import router
    hidden, inter, E, k, seq = 512, 384, 8, 2, 300
    blk = _block(kind, hidden, inter, E, k, True)
    with torch.no_grad():
        for prm in blk.parameters():
            prm.copy_(prm.to(torch.bfloat16).float())
    x = torch.randn((seq, hidden), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    params = _moe_params(blk, k, True, "cuda", torch.bfloat16)
    scores, idx = router(x.cuda(), params.router_params)
    w1, w2, act = expert_weights(params.expert_params)
    out = routed_experts(x.cuda(), w1, w2, scores, idx, E, k, act)
    with torch.no_grad():
        ref = blk.experts(x.float(), idx.cpu(), scores.float().cpu())
    assert_parity(out, ref, torch.bfloat16, f"{kind} experts, bf16", tol=2e-2)


def _hf_case(model, hidden, inter, E, k, dev, dtype):
    """(config, MOEParams, forward function of moe_explore.hf_moe_reference) of one model family;
    the expert record carries the model's hidden_act ("silu"), as the reference's test builds it."""
    from moe_explore import hf_moe_reference as hf
    from moe_explore.params import MOEParams
    from moe_explore.testing import random_ernie_router, random_glu, random_topk_router
    experts = random_glu(E, hidden, inter, "silu", dev, dtype)
    if model == "olmoe":
        from transformers.models.olmoe.configuration_olmoe import OlmoeConfig
        cfg = OlmoeConfig(hidden_size=hidden, intermediate_size=inter, num_experts=E,
                          num_experts_per_tok=k, norm_topk_prob=False, hidden_act="silu")
        router, forward = random_topk_router(E, hidden, k, True, False, dev, dtype), hf.olmoe_forward
    elif model == "qwen3":
        from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
        cfg = Qwen3MoeConfig(hidden_size=hidden, moe_intermediate_size=inter, intermediate_size=inter,
                             num_experts=E, num_experts_per_tok=k, norm_topk_prob=True, hidden_act="silu")
        router, forward = random_topk_router(E, hidden, k, True, True, dev, dtype), hf.qwen3_moe_forward
    else:
        from transformers.models.ernie4_5_moe.configuration_ernie4_5_moe import Ernie4_5_MoeConfig
        cfg = Ernie4_5_MoeConfig(hidden_size=hidden, moe_intermediate_size=inter, intermediate_size=inter,
                                 moe_num_experts=E, moe_k=k, moe_num_shared_experts=2, hidden_act="silu",
                                 use_bias=False)
        router, forward = random_ernie_router(E, hidden, k, dev, dtype), hf.ernie4_5_moe_forward
    return cfg, MOEParams(router, experts, E, k), forward


@pytest.mark.parametrize("model", ["olmoe", "qwen3", "ernie"])
def test_package_hf_reference_forward_functions_cpu(model):
    """moe_explore.hf_moe_reference (the reference's hf_moe_reference.py:16-120) on the CPU in fp32
    against the package's topk_moe_torch and against the oracle, on the same parameter record."""
    from moe_explore.functional.topk_moe import topk_moe_torch
    hidden, inter, E, k, T = 64, 32, 8, 2, 40
    torch.manual_seed(3)
    cfg, params, forward = _hf_case(model, hidden, inter, E, k, "cpu", torch.float32)
    x = torch.randn((T, hidden))
    ref = forward(cfg, x.unsqueeze(0), params).squeeze(0)
    assert_parity(topk_moe_torch(x, params), ref, torch.float32, f"{model}: topk_moe_torch vs transformers")
    ep = params.expert_params
    want, _, _ = _oracle_layer(x, type(params)(params.router_params, type(ep)(
        ep.gate_weight, ep.up_weight, ep.down_weight, "swiglu"), E, k))
    assert_parity(ref, want, torch.float32, f"{model}: transformers vs oracle")


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["olmoe", "qwen3", "ernie"])
def test_package_hf_reference_forward_functions(model):
    """The package's own counterpart of the reference's hf_moe_reference.py (its *_forward
    functions on a config and a MOEParams record) against topk_moe_forward on the same record,
    as the reference's tests/test_hf.py:75-99 does with released configs; here the configs are
    built locally at a reduced size, bf16 on the GPU, the reference's comparison rule."""
    from moe_explore.functional.topk_moe import topk_moe_forward
    from moe_explore.testing import assert_close
    hidden, inter, E, k, T = 256, 128, 16, 4, 200
    dev, dtype = "cuda", torch.bfloat16
    torch.manual_seed(11)
    cfg, params, forward = _hf_case(model, hidden, inter, E, k, dev, dtype)
    x = torch.randn((T, hidden), device=dev, dtype=dtype)
    ref = forward(cfg, x.unsqueeze(0), params).squeeze(0)
    out = topk_moe_forward(x, params)
    assert ref.isfinite().all() and out.isfinite().all()
    assert_close(ref, out)
