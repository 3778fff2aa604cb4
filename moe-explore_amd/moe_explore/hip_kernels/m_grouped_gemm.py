"""M-grouped and K-grouped GEMM wrappers.

``m_grouped_gemm`` / ``MGroupedGEMMParams`` keep the reference's signature and
output rules (``triton_kernels/m_grouped_gemm.py:16-31, 332-393``).  The keyword
arguments after ``autotune_mode`` are this library's additions: the fused
weighted scatter-add combine, the saved pre-activation and the weight-transposed
product used by the backward pass.
"""
from dataclasses import dataclass
from typing import Callable, Optional

import torch

from moe_explore import _C
from moe_explore.functional.activation import activation_name, is_glu
from .autotune_config import AutotuneMode


@dataclass
class MGroupedGEMMParams:
    weight: torch.Tensor
    group_indices: torch.Tensor
    permute_indices: Optional[torch.Tensor]
    gather: bool
    scatter: bool
    # Pre-routing token count when gathering or scattering, else the number of
    # input rows (reference m_grouped_gemm.py:23-27).
    num_tokens: int
    topk: int
    shared_weight: Optional[torch.Tensor] = None
    scales: Optional[torch.Tensor] = None
    activation: Optional[Callable] = None


def _weight_view(weight, transpose_weight):
    """[E, K, N] view of the weight whose K or N stride is 1."""
    w = weight.transpose(1, 2) if transpose_weight else weight
    if w.stride(2) != 1 and w.stride(1) != 1:
        w = w.contiguous()
    if w.size(0) > 1 and w.stride(0) < 0:
        w = w.contiguous()
    return w


def _group_indices(group_indices):
    gi = group_indices
    if gi.dtype != torch.int32:
        gi = gi.to(torch.int32)
    return gi.contiguous()


def m_grouped_gemm(
    token: torch.Tensor,
    params: MGroupedGEMMParams,
    autotune_mode: Optional[AutotuneMode] = None,
    *,
    combine: bool = False,
    save_preact: bool = False,
    transpose_weight: bool = False,
    out: Optional[torch.Tensor] = None,
    ksplit: int = 1,
):
    """``out[rows of expert e] = epilogue(token[rows] @ weight[e])``.

    Reference behaviour: ``gather`` reads token row ``permute_indices[p] // topk``
    for sorted position ``p``; ``scatter`` stores row ``p`` at
    ``permute_indices[p]``; ``scales`` is carried but not applied
    (``topk_moe.py:36-54`` applies it afterwards).

    Additions: ``combine=True`` (with ``scatter``) fuses that afterwards step:
    the result is the ``[num_tokens, N]`` top-k combination
    ``sum_j scales[t, j] * row(t, j)`` accumulated in fp32 (``scales=None`` sums
    unweighted).  ``save_preact=True`` also returns the rows before the epilogue.
    ``transpose_weight=True`` multiplies by ``weight[e]^T`` (weight is ``[E, N, K]``).
    ``ksplit > 1`` cuts K into that many parts that run as separate tiles; the result
    then has ``ksplit`` stacked partial copies (``[ksplit * rows, N]``) for
    ``scale_and_reduce(..., nsplit=ksplit)`` to add.  Falls back to one part when the
    shape does not allow the split.
    """
    assert token.dim() == 2
    assert params.weight.dim() == 3
    w = _weight_view(params.weight, transpose_weight)
    assert token.size(1) == w.size(1)
    assert autotune_mode is None or autotune_mode in AutotuneMode
    if params.gather or params.scatter:
        assert params.permute_indices is not None
    assert not (combine and not params.scatter), "combine=True needs scatter=True"
    assert not (combine and params.gather), "gather and the fused combine exclude each other"
    _C.require_cuda(token, w, params.group_indices, params.permute_indices)

    num_tokens = params.num_tokens
    e, k, n = w.size()
    if params.gather or params.scatter:
        out_rows = num_tokens * params.topk
    else:
        out_rows = num_tokens
    act = activation_name(params.activation)
    out_cols = n // 2 if is_glu(act) else n

    if token.stride(1) != 1 and token.size(1) > 1:
        token = token.contiguous()
    gi = _group_indices(params.group_indices)
    assert gi.numel() == e + 1, "group_indices must have num_experts + 1 entries"
    perm = params.permute_indices
    if perm is not None:
        perm = perm.contiguous()
        assert perm.numel() == out_rows, "permute_indices must have num_tokens * topk entries"
    if not params.gather:
        assert token.size(0) >= out_rows or params.scatter, "fewer input rows than num_tokens"
    if params.scatter:
        assert token.size(0) == out_rows, "scatter expects num_tokens * topk input rows"

    flags = 0
    if params.gather:
        flags |= _C.GEMM_GATHER_A
    scales = None
    if combine:
        flags |= _C.GEMM_SCATTER_ADD
        acc = torch.zeros((num_tokens, out_cols), device=token.device, dtype=torch.float32)
        c, c_rows = acc, num_tokens
        if params.scales is not None:
            scales = params.scales.to(token.dtype).contiguous().view(-1)
            assert scales.numel() == out_rows
    else:
        if params.scatter:
            flags |= _C.GEMM_SCATTER_C
        if ksplit > 1 and (act is not None or save_preact or k % (64 * ksplit) != 0
                           or token.dtype == torch.float32):
            ksplit = 1
        if out is None:
            out = torch.empty((ksplit * out_rows, out_cols), device=token.device, dtype=token.dtype)
        else:
            assert ksplit == 1
            assert out.shape == (out_rows, out_cols) and out.dtype == token.dtype and out.stride(1) == 1
        c, c_rows = out, out_rows
    preact = None
    if save_preact:
        assert not params.scatter, "the pre-activation is stored in sorted order only"
        flags |= _C.GEMM_SAVE_PREACT
        preact = torch.empty((out_rows, n), device=token.device, dtype=token.dtype)

    a_rows = token.size(0) if (params.gather or params.scatter) else min(token.size(0), out_rows)
    if combine:
        ksplit = 1

    def launch(parts):
        return _C.load().moe_m_grouped_gemm(
            token.data_ptr(), a_rows, token.stride(0),
            w.data_ptr(), w.stride(0), w.stride(1), w.stride(2),
            c.data_ptr(), c_rows, c.stride(0),
            _C.ptr(preact), 0 if preact is None else preact.stride(0),
            gi.data_ptr(), _C.ptr(perm), 0 if perm is None else _C.idx_bytes(perm), _C.ptr(scales),
            e, k, n, params.topk, flags, _C.act_code(act), _C.dtype_code(token.dtype),
            parts, c_rows * c.stride(0) if parts > 1 else 0, _C.stream_of(token))

    st = launch(ksplit)
    if st == -2 and ksplit > 1:  # MOE_ERR_UNSUPPORTED: this shape cannot be split
        ksplit = 1
        out = c = out[:out_rows]
        st = launch(1)
    _C.check(st, "moe_m_grouped_gemm")

    if combine:
        if out is None:
            out = torch.empty((num_tokens, out_cols), device=token.device, dtype=token.dtype)
        if token.dtype == torch.float32:
            out = acc if out is None else out.copy_(acc)
        else:
            st = _C.load().moe_cast_from_f32(acc.data_ptr(), acc.stride(0), out.data_ptr(),
                                             out.stride(0), num_tokens, out_cols,
                                             _C.dtype_code(token.dtype), _C.stream_of(token))
            _C.check(st, "moe_cast_from_f32")
    if save_preact:
        return out, preact
    return out


def k_grouped_gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    group_indices: torch.Tensor,
    permute_indices: Optional[torch.Tensor] = None,
    topk: int = 1,
    gather_a: bool = False,
    gather_b: bool = False,
    a_kmajor: bool = False,
    b_kmajor: bool = False,
):
    """Expert weight gradient: ``out[e] = a_e^T @ b_e`` with the contraction over
    expert ``e``'s sorted positions.  ``gather_a`` / ``gather_b`` read that operand's
    row for position ``p`` at ``permute_indices[p] // topk``.  ``a_kmajor`` / ``b_kmajor``:
    that operand is the feature-major matrix ``row_gather_kmajor`` returns (the fast path
    for the gathered token rows); only the MFMA kernel reads that layout, and when it does not
    take the shape (widths or strides not multiples of 8, unaligned pointers, no positions)
    the call returns ``None`` and the caller gathers with ``row_gather`` instead.  No
    reference counterpart (the reference is forward-only)."""
    assert a.dim() == 2 and b.dim() == 2 and a.dtype == b.dtype
    assert not (gather_a and gather_b) and not (a_kmajor and b_kmajor)
    assert not ((a_kmajor or b_kmajor) and (gather_a or gather_b))
    _C.require_cuda(a, b, group_indices, permute_indices)
    if a.stride(1) != 1 and a.size(1) > 1:
        a = a.contiguous()
    if b.stride(1) != 1 and b.size(1) > 1:
        b = b.contiguous()
    gi = _group_indices(group_indices)
    e = gi.numel() - 1
    flags = (_C.KGEMM_GATHER_A if gather_a else 0) | (_C.KGEMM_GATHER_B if gather_b else 0) | \
        (_C.KGEMM_A_KMAJOR if a_kmajor else 0) | (_C.KGEMM_B_KMAJOR if b_kmajor else 0)
    perm = None
    if gather_a or gather_b:
        assert permute_indices is not None
        perm = permute_indices.contiguous()
        assert perm.numel() == (b.size(0) if gather_a else a.size(0))
    elif not (a_kmajor or b_kmajor):
        assert a.size(0) == b.size(0)
    # a K-major operand is [features, columns]
    ka = a.size(0) if a_kmajor else a.size(1)
    nb = b.size(0) if b_kmajor else b.size(1)
    out = torch.empty((e, ka, nb), device=a.device, dtype=a.dtype)
    st = _C.load().moe_k_grouped_gemm(
        a.data_ptr(), a.size(1) if a_kmajor else a.size(0), a.stride(0), b.data_ptr(),
        b.size(1) if b_kmajor else b.size(0), b.stride(0), out.data_ptr(),
        gi.data_ptr(), _C.ptr(perm), 0 if perm is None else _C.idx_bytes(perm), e, ka,
        nb, topk, flags, _C.dtype_code(a.dtype), _C.stream_of(a))
    if st == -2 and (a_kmajor or b_kmajor):  # MOE_ERR_UNSUPPORTED
        return None
    _C.check(st, "moe_k_grouped_gemm")
    return out


def m_grouped_gemm_glu_bwd(dy_tokens, params: MGroupedGEMMParams, h, act, transpose_weight=False,
                           want_dscale=False):
    """``m_grouped_gemm`` (plain or gathered, no activation) followed by ``act_bwd`` in one
    launch: the product ``G`` (the gradient of the GLU output, per sorted position) is never
    stored.  ``params.scales`` are the routing weights by slot, ``params.permute_indices``
    the slot ids (the kernel wants the weights by sorted position and returns dscale by
    position: both permutations happen here).  Returns ``(dh, y_scaled, dscale or None)`` as ``act_bwd`` does with
    ``want_y_scaled``, or ``None`` when the shape is outside the fused kernel's reach (the
    caller then runs the two steps)."""
    name = activation_name(act)
    assert is_glu(name) and params.activation is None and not params.scatter
    _C.require_cuda(dy_tokens, params.weight, params.group_indices, params.permute_indices, h)
    if dy_tokens.dtype not in (torch.bfloat16, torch.float16) or h.dtype != dy_tokens.dtype:
        return None
    w = _weight_view(params.weight, transpose_weight)
    e, k, n = w.shape
    if dy_tokens.stride(1) != 1 or h.stride(1) != 1 or w.stride(1) != 1:
        return None
    P, n2 = h.shape
    assert n2 == 2 * n and dy_tokens.size(1) == k
    perm = params.permute_indices
    perm = None if perm is None else perm.contiguous()
    flags = _C.GEMM_GATHER_A if params.gather else 0
    assert P == (params.num_tokens * params.topk if params.gather else params.num_tokens)
    dh = torch.empty_like(h, memory_format=torch.contiguous_format)
    ys = torch.empty((P, n), device=h.device, dtype=h.dtype)
    ds = torch.zeros(P, device=h.device, dtype=torch.float32) if want_dscale else None
    rs = None
    if params.scales is not None:
        rs = params.scales.to(h.dtype).reshape(-1)
        rs = (rs if perm is None else rs[perm]).contiguous()
    gi = params.group_indices
    assert gi.dtype == torch.int32 and gi.numel() == e + 1
    st = _C.load().moe_m_grouped_gemm_glu_bwd(
        dy_tokens.data_ptr(), dy_tokens.size(0), dy_tokens.stride(0), w.data_ptr(), w.stride(0),
        w.stride(1), w.stride(2), h.data_ptr(), h.stride(0), dh.data_ptr(), dh.stride(0),
        ys.data_ptr(), ys.stride(0), _C.ptr(ds), gi.data_ptr(), _C.ptr(perm),
        0 if perm is None else _C.idx_bytes(perm), _C.ptr(rs), P, e, k, n, params.topk, flags,
        _C.act_code(name), _C.dtype_code(h.dtype), _C.stream_of(h))
    if st == -2:  # MOE_ERR_UNSUPPORTED
        return None
    _C.check(st, "moe_m_grouped_gemm_glu_bwd")
    if ds is not None and perm is not None:  # position order -> slot order
        ds = torch.empty_like(ds).index_copy_(0, perm.to(torch.int64), ds)
    return dh, ys, ds


def act_bwd(h, dy, act, row_scale=None, permute_indices=None, want_y_scaled=False, want_dscale=False):
    """Gradient of the expert activation (see ``moe_act_bwd`` in the C header).
    Returns ``(dh, y_scaled or None, dscale or None)``."""
    assert h.dim() == 2 and dy.dim() == 2 and h.dtype == dy.dtype
    _C.require_cuda(h, dy, row_scale, permute_indices)
    name = activation_name(act)
    h = h if h.stride(1) == 1 else h.contiguous()
    dy = dy if dy.stride(1) == 1 else dy.contiguous()
    R, N = h.shape
    assert dy.shape == (R, N // 2 if is_glu(name) else N)
    dh = torch.empty_like(h, memory_format=torch.contiguous_format)
    ys = torch.empty_like(dy, memory_format=torch.contiguous_format) if want_y_scaled else None
    ds = torch.zeros(R, device=h.device, dtype=torch.float32) if want_dscale else None
    rs = None if row_scale is None else row_scale.to(h.dtype).contiguous().view(-1)
    perm = None if permute_indices is None else permute_indices.contiguous()
    st = _C.load().moe_act_bwd(
        h.data_ptr(), h.stride(0), dy.data_ptr(), dy.stride(0), dh.data_ptr(), dh.stride(0),
        _C.ptr(rs), _C.ptr(perm), 0 if perm is None else _C.idx_bytes(perm), _C.ptr(ys),
        0 if ys is None else ys.stride(0), _C.ptr(ds), R, N, _C.act_code(name),
        _C.dtype_code(h.dtype), _C.stream_of(h))
    _C.check(st, "moe_act_bwd")
    return dh, ys, ds
