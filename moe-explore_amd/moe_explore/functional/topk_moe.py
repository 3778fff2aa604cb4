"""The MoE layer (reference ``functional/topk_moe.py:10-102``).

``topk_moe_forward`` runs router -> routing preprocessing -> grouped GEMM with
fused gather and activation -> grouped GEMM fused with the top-k weighted
combine, all on HIP kernels and without a host synchronisation.  When a
gradient is required it records an autograd node whose backward runs the
transposed M-grouped GEMMs (dX), the K-grouped GEMMs (dW) and the activation
gradient; the reference itself is forward-only.

``topk_moe_torch`` is the plain-PyTorch per-expert loop that the reference ships
as its comparison implementation (``:67-102``); it is not used by the HIP path.
"""
import torch

from moe_explore.params import MOEParams, MLPParams, GLUParams, GLUInterleavedParams
from moe_explore.tracing import scope
from moe_explore.functional.activation import activation, activation_name, glu_form, is_glu
from moe_explore.functional.scale_and_reduce import scale_and_reduce
from moe_explore.router import router
from moe_explore.expert_permute import get_token_indices
from moe_explore.hip_kernels.row_gather_scatter import row_gather, row_gather_kmajor
from moe_explore.hip_kernels.m_grouped_gemm import (
    MGroupedGEMMParams,
    m_grouped_gemm,
    k_grouped_gemm,
    act_bwd,
    m_grouped_gemm_glu_bwd,
)


def interleave_glu_weights(gate_weight, up_weight):
    """[E, d, ff] gate and up -> [E, d, 2*ff] with gate in the even and up in the odd
    columns, the layout the GLU epilogue reads (``functional/activation.py:19-20``)."""
    e, d, ff = gate_weight.shape
    out = torch.empty((e, d, 2 * ff), device=gate_weight.device, dtype=gate_weight.dtype)
    out[:, :, 0::2] = gate_weight
    out[:, :, 1::2] = up_weight
    return out


def to_interleaved(ep):
    """Load-time conversion of separate gate / up weights (``params.py:16-21``, the layout of
    Hugging Face checkpoints) into the record the kernels read directly.  Training code
    should convert once and keep the result as its parameter: the weight gradient then
    comes back in the same interleaved layout and nothing is copied per step."""
    if isinstance(ep, GLUParams):
        return GLUInterleavedParams(interleave_glu_weights(ep.gate_weight, ep.up_weight),
                                    ep.down_weight, glu_form(ep.activation))
    return ep


class _InterleaveFunction(torch.autograd.Function):
    """Differentiable interleave: the gradient of weight1 goes back to gate and up as its
    even and odd columns."""

    @staticmethod
    def forward(ctx, gate, up):
        return interleave_glu_weights(gate, up)

    @staticmethod
    def backward(ctx, dw):
        return dw[:, :, 0::2], dw[:, :, 1::2]


def expert_weights(ep):
    """(weight1, weight2, activation) of any of the reference's FFN parameter records.
    Separate gate / up weights are interleaved on every call (one pass over the two tensors):
    no copy is kept between calls, because nothing a tensor exposes tells whether its storage
    has been written since (updates through ``.data``, graph replays and raw kernels leave the
    version counter alone).  ``to_interleaved`` converts once, at load time."""
    if isinstance(ep, MLPParams):
        return ep.weight1, ep.weight2, ep.activation
    if isinstance(ep, GLUInterleavedParams):
        return ep.interleaved_weight, ep.down_weight, glu_form(ep.activation)
    if isinstance(ep, GLUParams):
        gate, up = ep.gate_weight, ep.up_weight
        if torch.is_grad_enabled() and (gate.requires_grad or up.requires_grad):
            w1 = _InterleaveFunction.apply(gate, up)
        else:
            w1 = interleave_glu_weights(gate.detach(), up.detach())
        return w1, ep.down_weight, glu_form(ep.activation)
    raise ValueError(f"Unsupported expert parameter type: {type(ep)}")


def _ksplit_for(rows, num_experts, n, k):
    """Cuts K in two when the output has so few 256 x 256 tiles that the last round of
    workgroups would leave most of the 256 CUs idle, and K is long enough to pay for a
    second partial store."""
    tiles = ((rows + 255) // 256 + num_experts // 2) * ((n + 255) // 256)
    if k >= 4096 and k % 128 == 0 and tiles < 1024 and (tiles % 256) not in (0,) and \
            (tiles % 256) < 160:
        return 2
    return 1


# intermediate width below which the dW2 kernel gathers its token rows itself (see backward)
_FUSED_GATHER_BELOW_FF = 1280


def _dw2(a_scaled, dout, gi, idx, topk):
    """dW2 = (s*A)^T dOut over every expert's positions.  The token rows are gathered first,
    feature-major (one 25 us pass over R x d): the K-grouped kernel then reads that operand from
    LDS with plain 16-byte loads instead of transpose loads.  The kernel can also gather by
    itself, but then has to wait for the row ids of every K step, and with them for the copies
    it keeps in flight: 10-15 % slower.  That is still the cheaper way for narrow experts: the
    pass over R x d costs ~330 / ff of the GEMM it serves (ff = 1024: a third), so below
    ff = 1280 the kernel gathers dout itself (OLMoE shape, T = 8192: 0.362 -> 0.316 ms; Qwen3
    shape, T = 32000: 1.09 -> 0.91 ms; ff = 1408 the same either way)."""
    if a_scaled.size(1) < _FUSED_GATHER_BELOW_FF:
        return k_grouped_gemm(a_scaled, dout, gi, idx, topk, gather_b=True)
    dw2 = None
    dt = row_gather_kmajor(dout, idx, topk, gi)
    if dt is not None:
        dw2 = k_grouped_gemm(a_scaled, dt, gi, b_kmajor=True)
    if dw2 is None:  # a shape the feature-major path does not take
        dw2 = k_grouped_gemm(a_scaled, row_gather(dout, idx, topk), gi)
    return dw2


def _dw1(x, dh, gi, idx, topk):
    """dW1 = Xg^T dH; the gathered token rows feature-major where the kernel takes them (-10 %
    at the Mixtral shape; its GEMM is twice as long as dW2's, so it always gathers first)."""
    dw1 = None
    xt = row_gather_kmajor(x, idx, topk, gi)
    if xt is not None:
        dw1 = k_grouped_gemm(xt, dh, gi, a_kmajor=True)
    if dw1 is None:
        dw1 = k_grouped_gemm(row_gather(x, idx, topk), dh, gi)
    return dw1


class _ExpertsFunction(torch.autograd.Function):
    """Routed experts + combine: ``out[t] = sum_j scores[t,j] * FFN_e(t,j)(x[t])``."""

    @staticmethod
    def forward(ctx, x, w1, w2, scores, group_indices, indices, act, topk):
        T = x.size(0)
        need_grad = any(ctx.needs_input_grad[:4])
        p1 = MGroupedGEMMParams(w1, group_indices, indices, True, False, T, topk, activation=act)
        with scope("fused_grouped_glu"):
            if need_grad and act is not None:
                a, h = m_grouped_gemm(x, p1, save_preact=True)
            else:
                a = m_grouped_gemm(x, p1)
                h = a if need_grad else None  # identity activation: A is its own pre-activation
        # down projection stored in slot order, then the top-k weighted sum
        # (reference topk_moe.py:36-54); the fp32-atomic fused combine of
        # m_grouped_gemm(combine=True) is slower than this second pass on MI355X
        p2 = MGroupedGEMMParams(w2, group_indices, indices, False, True, T, topk, scales=scores)
        ks = _ksplit_for(T * topk, w2.size(0), w2.size(2), w2.size(1))
        with scope("down_grouped_gemm"):
            y = m_grouped_gemm(a, p2, ksplit=ks)
        ks = y.size(0) // (T * topk) if T else 1
        with scope("scale_and_reduce"):
            out = scale_and_reduce(y, scores, T, topk, y.size(1), nsplit=ks)
        if need_grad:
            ctx.save_for_backward(x, w1, w2, scores, group_indices, indices, h)
            ctx.act, ctx.topk = act, topk
        return out

    @staticmethod
    def backward(ctx, dout):
        x, w1, w2, scores, gi, idx, h = ctx.saved_tensors
        act, topk, T = ctx.act, ctx.topk, x.size(0)
        dout = dout.contiguous()
        # G[p] = dout[token(p)] @ w2[e]^T
        need_dscore = ctx.needs_input_grad[3]
        fused = None
        if is_glu(act):
            # G is turned into dH, s*A and dscore in the GEMM's epilogue and never stored
            pf = MGroupedGEMMParams(w2, gi, idx, True, False, T, topk, scales=scores)
            fused = m_grouped_gemm_glu_bwd(dout, pf, h, act, transpose_weight=True,
                                           want_dscale=need_dscore)
        if fused is not None:
            dh, a_scaled, dscale = fused
        else:
            pg = MGroupedGEMMParams(w2, gi, idx, True, False, T, topk)
            g = m_grouped_gemm(dout, pg, transpose_weight=True)
            # (identity activation: dH = s * G, s * A = s * H, dscore = <G, H>)
            dh, a_scaled, dscale = act_bwd(h, g, act, row_scale=scores, permute_indices=idx,
                                           want_y_scaled=True, want_dscale=need_dscore)
        dw1 = dw2 = dx = dscores = None
        # dW2, dW1 and dX share no output, but they run one after the other on the calling stream:
        # forked onto side streams of equal priority the hardware deals the compute units out
        # among the three resident-workgroup launches from the start (not only in the last
        # round of each), the launches lose the L2 locality of their tile order, and the step
        # is 8 % slower (Mixtral shape: 8.76 -> 9.5 ms).
        if ctx.needs_input_grad[2]:
            dw2 = _dw2(a_scaled, dout, gi, idx, topk)
        if ctx.needs_input_grad[1]:
            dw1 = _dw1(x, dh, gi, idx, topk)
        if ctx.needs_input_grad[0]:
            px = MGroupedGEMMParams(w1, gi, idx, False, True, T, topk, scales=None)
            ks = _ksplit_for(T * topk, w1.size(0), w1.size(1), w1.size(2))
            dxg = m_grouped_gemm(dh, px, transpose_weight=True, ksplit=ks)
            ks = dxg.size(0) // (T * topk) if T else 1
            dx = scale_and_reduce(dxg, None, T, topk, dxg.size(1), nsplit=ks)
        if need_dscore:
            dscores = dscale.view(scores.shape).to(scores.dtype)
        return dx, dw1, dw2, dscores, None, None, None, None


def routed_experts(x, weight1, weight2, topk_scores, topk_indices, num_experts, topk, act):
    """Experts + combine for given routing decisions (differentiable in ``x``, the
    weights and ``topk_scores``)."""
    with scope("get_token_indices"):
        p = get_token_indices(topk_indices, topk, num_experts, zero_prefix=True)
    return _ExpertsFunction.apply(x, weight1, weight2, topk_scores, p.group_indices, p.indices,
                                  activation_name(act), topk)


def shared_experts(input, sp):
    """The reference's shared-expert branch (``topk_moe.py:56-62``): every token through each
    of the S shared FFNs, summed over S (its ``h.sum(0)`` over stacked ``[S, d, ff]`` /
    ``[S, ff, d]`` weights; 2-D weights are one shared expert).  Runs on the grouped-GEMM
    kernels as S experts that every token is routed to with weight 1, so the forward is two
    grouped GEMMs and the backward the routed experts' own."""
    up, down = sp.up_weight, sp.down_weight
    if up.dim() == 2:
        up, down = up.unsqueeze(0), down.unsqueeze(0)
    assert up.dim() == 3 and down.dim() == 3 and up.size(0) == down.size(0)
    S, T = up.size(0), input.size(0)
    ones = torch.ones((T, S), device=input.device, dtype=input.dtype)
    ids = torch.arange(S, device=input.device, dtype=torch.int64).expand(T, S)
    return routed_experts(input, up, down, ones, ids, S, S, sp.activation)


def topk_moe_forward(input: torch.Tensor, params: MOEParams, autotune_mode=None):
    w1, w2, act = expert_weights(params.expert_params)
    with scope("router"):
        topk_scores, topk_indices = router(input, params.router_params)
    out = routed_experts(input, w1, w2, topk_scores, topk_indices, params.num_experts,
                         params.topk, act)
    sp = getattr(params, "shared_expert_params", None)
    if sp is not None:
        with scope("shared_expert"):
            out = out + shared_experts(input, sp)
    return out


def topk_moe_torch(input, params: MOEParams, autotune_mode=None):
    """Per-expert PyTorch loop (``topk_moe.py:67-102``), any device.  Scales and
    accumulates in the input dtype, expert by expert, as the reference does."""
    w1, w2, act = expert_weights(params.expert_params)
    topk_scores, topk_indices = router(input, params.router_params)
    flat_expert_weights = topk_scores.reshape(-1, 1)
    flat = topk_indices.reshape(-1)
    indices = torch.sort(flat, stable=True).indices
    ends = torch.bincount(flat, minlength=params.num_experts).cumsum(0).tolist()
    expert_cache = torch.zeros_like(input)
    start = 0
    for expert_id, end in enumerate(ends):
        if start == end:
            continue
        sl = indices[start:end]
        tok = sl // params.topk
        h = input[tok] @ w1[expert_id]
        if act is not None:
            h = activation(h, act)
        y = h @ w2[expert_id]
        y.mul_(flat_expert_weights[sl])
        expert_cache.scatter_reduce_(0, tok.view(-1, 1).repeat(1, input.shape[-1]), y, reduce="sum")
        start = end
    return expert_cache
