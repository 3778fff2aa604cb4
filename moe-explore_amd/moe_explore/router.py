"""Routers (reference ``router.py:5-54``).

On the GPU ``topk_router`` and ``ernie_router`` run as one fused HIP kernel (logits,
fp32 softmax, top-k, renormalisation, cast) with a second small kernel for the gradient
of the scores with respect to the logits; of the two skinny matmuls of the backward pass dx
stays on ATen and the weight gradient runs on the K-grouped kernel from 8192 tokens on.
Shapes outside the kernel's reach (more than 512 experts, top-k above 16, rows that cannot be
read 16 bytes at a time) and CPU tensors take the ATen formulation
below, which is the reference's own.
"""
import torch
from torch import nn

from moe_explore import _C
from moe_explore.params import RouterParams, TopkRouterParams, ErnieRouterParams


def softmax(x):
    return nn.functional.softmax(x, dim=-1, dtype=torch.float32)


def router(input: torch.Tensor, params: RouterParams):
    if isinstance(params, TopkRouterParams):
        return topk_router(input, params)
    elif isinstance(params, ErnieRouterParams):
        return ernie_router(input, params)
    raise ValueError(f"Unsupported router type: {type(params)}")


def _fused_flags(softmax_before_topk, normalize_routing, ernie):
    return ((_C.ROUTER_SOFTMAX_FIRST if softmax_before_topk else 0)
            | (_C.ROUTER_NORMALIZE if normalize_routing else 0)
            | (_C.ROUTER_ERNIE if ernie else 0))


def _fused_supported(x, weight, topk, ernie):
    if not (x.is_cuda and weight.is_cuda) or x.dim() != 2 or weight.dim() != 2:
        return False
    if x.dtype not in _C._DTYPES or weight.dtype not in _C._DTYPES:
        return False
    if weight.dtype != torch.float32 and weight.dtype != x.dtype:
        return False
    if ernie and weight.dtype != torch.float32:
        return False
    d, E = weight.shape
    f32 = torch.float32 in (x.dtype, weight.dtype)
    vec = 4 if f32 else 8
    return (x.size(1) == d and 0 < E <= 512 and 1 <= topk <= min(E, 16) and d % vec == 0
            and x.stride(1) == 1 and x.stride(0) % vec == 0
            and x.data_ptr() % (vec * x.element_size()) == 0)


def _fused_forward(x, weight, bias, topk, flags, want_logits):
    lib = _C.load()
    T, d = x.shape
    E = weight.size(1)
    scores = torch.empty((T, topk), dtype=x.dtype, device=x.device)
    idx = torch.empty((T, topk), dtype=torch.int64, device=x.device)
    logits = torch.empty((T, E), dtype=torch.float32, device=x.device) if want_logits else None
    xd, wd = _C.dtype_code(x.dtype), _C.dtype_code(weight.dtype)
    ws_bytes = lib.moe_router_workspace_bytes(d, E, xd, wd)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    st = lib.moe_router_topk(
        x.data_ptr(), x.stride(0), weight.data_ptr(), weight.stride(0), weight.stride(1),
        _C.ptr(bias), scores.data_ptr(), idx.data_ptr(), _C.ptr(logits), T, d, E, topk, flags,
        xd, wd, ws.data_ptr(), ws.numel(), _C.stream_of(x))
    _C.check(st, "moe_router_topk")
    return scores, idx, logits


_token_group_bounds = {}
_MANY_TOKENS = 8192  # from here on the router's weight gradient runs over token groups

# An fp32 router weight (Ernie: "float32 for everything in the router", router.py:43) gets its
# gradient from fp32 products at every token count.  Callers that prefer speed can ask for
# 16-bit operands from _MANY_TOKENS tokens on; nothing switches by itself.
_fp32_router_backward_in_16_bits = False


def fp32_router_backward_in_16_bits(enabled: bool):
    """Opt in to (or out of) 16-bit operands for the backward products of an fp32 router
    weight under 16-bit activations from 8192 tokens on: about 2e-3 relative error on the
    weight gradient instead of 1e-6, 0.35 ms less at T = 32000, d = 2560.  Off by default."""
    global _fp32_router_backward_in_16_bits
    _fp32_router_backward_in_16_bits = bool(enabled)


def _router_weight_grad(x, dlogits, out_dtype):
    """``x^T @ dlogits`` ([T, d]^T [T, E] -> [d, E]).  A reduction over many tokens into a small
    matrix, which the library's GEMM runs on a few compute units (T = 32000, d = 2048, E = 128:
    109 us).  From 8192 tokens on the tokens are cut into as many groups as fill the GPU and the
    K-grouped weight-gradient kernel computes one partial product a group (55 us with the sum of
    the partials; 16-bit operands only: its partials are rounded to 16 bits, 2e-3 relative)."""
    T, d = x.shape
    E = dlogits.size(1)
    if (x.dtype in (torch.bfloat16, torch.float16) and dlogits.dtype == x.dtype and out_dtype == x.dtype
            and T >= _MANY_TOKENS and d % 8 == 0 and E % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0):
        from moe_explore.gpu_utils import get_gpu_sm_count
        from moe_explore.hip_kernels.m_grouped_gemm import k_grouped_gemm
        groups = max(1, min(T // 64, -(-get_gpu_sm_count(x.device) // -(-d // 256))))
        key = (T, groups, x.device)
        bounds = _token_group_bounds.get(key)
        if bounds is None:
            step = T // groups // 64 * 64
            bounds = torch.tensor([i * step for i in range(groups)] + [T], dtype=torch.int32, device=x.device)
            if len(_token_group_bounds) > 64:
                _token_group_bounds.clear()
            _token_group_bounds[key] = bounds
        return k_grouped_gemm(x, dlogits, bounds).float().sum(0)
    return x.to(out_dtype).t() @ dlogits


class _FusedRouter(torch.autograd.Function):
    """scores, indices = router(x, weight); differentiable in x and weight through the
    scores (the selection itself has no gradient)."""

    @staticmethod
    def forward(ctx, x, weight, bias, topk, flags):
        need = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        scores, idx, logits = _fused_forward(x, weight, bias, topk, flags, need)
        if need:
            ctx.save_for_backward(x, weight, idx, logits)
            ctx.flags, ctx.topk = flags, topk
        ctx.mark_non_differentiable(idx)
        return scores, idx

    @staticmethod
    def backward(ctx, dscores, _didx):
        x, weight, idx, logits = ctx.saved_tensors
        T, E = logits.shape
        ernie = bool(ctx.flags & _C.ROUTER_ERNIE)
        # the top-k router's logits have the dtype of x; Ernie's are fp32
        out_dtype = torch.float32 if (ernie or weight.dtype == torch.float32) else x.dtype
        dscores = dscores.contiguous()
        dlogits = torch.empty((T, E), dtype=out_dtype, device=x.device)
        st = _C.load().moe_router_bwd(
            logits.data_ptr(), idx.data_ptr(), dscores.data_ptr(), dlogits.data_ptr(), T, E,
            ctx.topk, ctx.flags, _C.dtype_code(dscores.dtype), _C.dtype_code(out_dtype),
            _C.stream_of(x))
        _C.check(st, "moe_router_bwd")
        dx = dw = None
        if (_fp32_router_backward_in_16_bits and out_dtype == torch.float32
                and x.dtype in (torch.bfloat16, torch.float16) and T >= _MANY_TOKENS):
            # fp32 router weight under 16-bit activations (Ernie), many tokens, on request
            # (fp32_router_backward_in_16_bits): the two products of the backward pass on 16-bit
            # operands, as for a 16-bit router.  In fp32 they cost an upcast copy of x and of dx
            # (T = 32000, d = 2560: 0.6 ms a step against 0.25 ms); dx leaves in 16 bits either
            # way, but dW then carries the 2e-3 of 16-bit partial products instead of 1e-6.
            dl16 = dlogits.to(x.dtype)
            if ctx.needs_input_grad[0]:
                dx = dl16 @ weight.t().to(x.dtype)
            if ctx.needs_input_grad[1]:
                dw = _router_weight_grad(x, dl16, x.dtype).to(weight.dtype)
            return dx, dw, None, None, None
        if ctx.needs_input_grad[0]:
            dx = (dlogits @ weight.t().to(out_dtype)).to(x.dtype)
        if ctx.needs_input_grad[1]:
            dw = _router_weight_grad(x, dlogits, out_dtype).to(weight.dtype)
        return dx, dw, None, None, None


def topk_router(input: torch.Tensor, router_params: TopkRouterParams):
    weight = router_params.router_weight
    if _fused_supported(input, weight, router_params.topk, False):
        flags = _fused_flags(router_params.softmax_before_topk, router_params.normalize_routing, False)
        return _FusedRouter.apply(input, weight, None, router_params.topk, flags)
    logits = input @ router_params.router_weight
    return route_from_logits(
        logits,
        router_params.topk,
        softmax_before_topk=router_params.softmax_before_topk,
        normalize_routing=router_params.normalize_routing,
        dtype=input.dtype,
    )


def route_from_logits(logits, topk, softmax_before_topk=True, normalize_routing=False, dtype=None):
    """The part of ``topk_router`` after the logits matmul (``router.py:23-34``);
    split out so that benchmarks can feed synthetic logits directly."""
    dtype = logits.dtype if dtype is None else dtype
    if softmax_before_topk:
        logits = softmax(logits)
    topk_scores, topk_indices = torch.topk(logits, k=topk, dim=-1, sorted=False)
    if not softmax_before_topk:
        topk_scores = softmax(topk_scores)
    if normalize_routing:
        topk_scores = topk_scores / topk_scores.sum(dim=-1, keepdim=True)
    return topk_scores.to(dtype), topk_indices


def ernie_router(input: torch.Tensor, router_params: ErnieRouterParams):
    assert router_params.router_weight.dtype is torch.float32
    if _fused_supported(input, router_params.router_weight, router_params.topk, True):
        bias = router_params.bias.to(device=input.device, dtype=torch.float32).reshape(-1).contiguous()
        assert bias.numel() == router_params.router_weight.size(1)
        return _FusedRouter.apply(input, router_params.router_weight, bias, router_params.topk,
                                  _fused_flags(True, True, True))
    with torch.autocast(device_type=input.device.type, enabled=False):
        logits = input.float() @ router_params.router_weight
        weights = softmax(logits)
        _, topk_indices = torch.topk(weights + router_params.bias, k=router_params.topk, dim=-1, sorted=False)
        weights = torch.gather(weights, index=topk_indices, dim=-1)
        weights = weights / torch.clamp(weights.sum(dim=-1, keepdim=True), min=1e-12)
        return weights.to(input.dtype), topk_indices
