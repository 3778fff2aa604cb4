"""Sparse-MoE blocks of the installed ``transformers`` modelling code, loaded with the
weights of a ``MOEParams`` record, as independent implementations to compare the layer
with (the reference's ``hf_moe_reference.py:16-120``: ``Olmoe``, ``Qwen3Moe``,
``Ernie4_5_Moe`` and one ``*_forward`` function each, used by its ``tests/test_hf.py``).

The blocks are plain PyTorch and run wherever the input lives.  ``params.expert_params``
is a ``GLUParams`` (separate gate / up weights ``[E, d, ff]``, down ``[E, ff, d]``), the
router weight ``[d, E]``; both expert layouts that ``transformers`` has shipped are
filled: a list of expert MLPs with ``gate_proj`` / ``up_proj`` / ``down_proj`` (what the
reference wrote against), and one experts module with stacked ``gate_up_proj
[E, 2 ff, d]`` (gate rows first) and ``down_proj [E, d, ff]``.
"""
import torch
from transformers.models.ernie4_5_moe.configuration_ernie4_5_moe import Ernie4_5_MoeConfig
from transformers.models.ernie4_5_moe.modeling_ernie4_5_moe import Ernie4_5_MoeSparseMoeBlock
from transformers.models.olmoe.configuration_olmoe import OlmoeConfig
from transformers.models.olmoe.modeling_olmoe import OlmoeSparseMoeBlock
from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

from moe_explore.params import MOEParams


def _fill(block, router_weight, gate_weight, up_weight, down_weight, router_bias=None):
    """Copies [d, E] / [E, d, ff] / [E, ff, d] weights into ``block`` (see the module text)."""
    with torch.no_grad():
        # (the Ernie router keeps its weight and its selection bias in fp32 whatever the block's dtype)
        gate_dtype = torch.float32 if router_bias is not None else block.gate.weight.dtype
        block.gate.weight.data = router_weight.t().contiguous().to(gate_dtype)
        if router_bias is not None:
            statics = block.moe_statics if hasattr(block, "moe_statics") else block.gate.moe_statics
            statics.e_score_correction_bias.data = router_bias.to(torch.float32).reshape(
                statics.e_score_correction_bias.shape)
        experts = block.experts
        if hasattr(experts, "gate_up_proj"):
            stacked = torch.cat((gate_weight.transpose(1, 2), up_weight.transpose(1, 2)), dim=1)
            experts.gate_up_proj.data = stacked.contiguous().to(experts.gate_up_proj.dtype)
            experts.down_proj.data = down_weight.transpose(1, 2).contiguous().to(experts.down_proj.dtype)
        else:
            for e, mlp in enumerate(experts):
                mlp.gate_proj.weight.data = gate_weight[e].t().contiguous()
                mlp.up_proj.weight.data = up_weight[e].t().contiguous()
                mlp.down_proj.weight.data = down_weight[e].t().contiguous()


def _run(block, input, params, router_bias=None):
    block = block.to(device=input.device, dtype=input.dtype)
    ep = params.expert_params
    _fill(block, params.router_params.router_weight, ep.gate_weight, ep.up_weight, ep.down_weight,
          router_bias)
    with torch.no_grad():
        out = block(input)
    return out[0] if isinstance(out, tuple) else out   # older versions also return the router logits


class Olmoe(OlmoeSparseMoeBlock):
    def init_weights(self, router_weight, gate_weight, up_weight, down_weight):
        _fill(self, router_weight, gate_weight, up_weight, down_weight)


class Qwen3Moe(Qwen3MoeSparseMoeBlock):
    def init_weights(self, router_weight, gate_weight, up_weight, down_weight):
        _fill(self, router_weight, gate_weight, up_weight, down_weight)


class Ernie4_5_Moe(Ernie4_5_MoeSparseMoeBlock):
    """Without shared experts, as the reference builds it (``hf_moe_reference.py:84-86``); the
    layer's own shared-expert branch is compared with the full block in this build's tests."""

    def __init__(self, config):
        config.moe_num_shared_experts = 0
        super().__init__(config)

    def init_weights(self, router_weight, router_bias, gate_weight, up_weight, down_weight):
        _fill(self, router_weight, gate_weight, up_weight, down_weight, router_bias)


def olmoe_forward(olmoe_config: OlmoeConfig, input: torch.Tensor, params: MOEParams):
    return _run(Olmoe(olmoe_config), input, params)


def qwen3_moe_forward(qwen3_config: Qwen3MoeConfig, input: torch.Tensor, params: MOEParams):
    return _run(Qwen3Moe(qwen3_config), input, params)


def ernie4_5_moe_forward(ernie4_5_config: Ernie4_5_MoeConfig, input: torch.Tensor, params: MOEParams):
    return _run(Ernie4_5_Moe(ernie4_5_config), input, params, params.router_params.bias)
