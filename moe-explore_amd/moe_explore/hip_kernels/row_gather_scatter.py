"""Row gather / row scatter (reference ``triton_kernels/row_gather_scatter.py``)."""
import torch

from moe_explore import _C


def _rows(t):
    return t if t.stride(1) == 1 or t.size(1) <= 1 else t.contiguous()


def row_gather(tokens: torch.Tensor, gather_indices: torch.Tensor, index_div: int = 1):
    """``out[r, :] = tokens[gather_indices[r] // index_div, :]``
    (``row_gather_scatter.py:36-58``; ``index_div`` folds the ``indices // topk`` of
    ``expert_permute.py:51`` into the kernel)."""
    assert tokens.ndim == 2
    assert gather_indices.ndim == 1
    _C.require_cuda(tokens, gather_indices)
    tokens = _rows(tokens)
    gather_indices = gather_indices.contiguous()
    out = torch.empty((gather_indices.size(0), tokens.size(1)), device=tokens.device, dtype=tokens.dtype)
    if out.numel() == 0:
        return out
    assert tokens.size(0) > 0, "gather from an empty matrix"
    st = _C.load().moe_row_gather(
        tokens.data_ptr(), tokens.size(0), tokens.stride(0), gather_indices.data_ptr(),
        _C.idx_bytes(gather_indices), int(index_div), out.data_ptr(), out.stride(0), out.size(0),
        out.size(1), tokens.element_size(), _C.stream_of(tokens))
    _C.check(st, "moe_row_gather")
    return out


def row_scatter(tokens: torch.Tensor, scatter_indices: torch.Tensor):
    """``out[scatter_indices[r], :] = tokens[r, :]`` for a permutation
    ``scatter_indices`` (``row_gather_scatter.py:91-116``)."""
    assert tokens.ndim == 2
    assert scatter_indices.ndim == 1
    assert scatter_indices.size(0) == tokens.size(0)
    _C.require_cuda(tokens, scatter_indices)
    tokens = _rows(tokens)
    scatter_indices = scatter_indices.contiguous()
    out = torch.empty((tokens.size(0), tokens.size(1)), device=tokens.device, dtype=tokens.dtype)
    if out.numel() == 0:
        return out
    st = _C.load().moe_row_scatter(
        tokens.data_ptr(), tokens.stride(0), scatter_indices.data_ptr(), _C.idx_bytes(scatter_indices),
        out.data_ptr(), out.size(0), out.stride(0), tokens.size(0), tokens.size(1),
        tokens.element_size(), _C.stream_of(tokens))
    _C.check(st, "moe_row_scatter")
    return out


def row_gather_kmajor(tokens: torch.Tensor, gather_indices: torch.Tensor, index_div: int,
                      group_indices: torch.Tensor):
    """Gathered token rows, feature-major, for the weight-gradient GEMM
    (``k_grouped_gemm(..., a_kmajor=True)`` / ``b_kmajor=True``):
    ``out[f, qs(e) + (p - lo(e))] = tokens[gather_indices[p] // index_div, f]`` for the sorted
    positions ``p`` of expert ``e``, where ``qs(e) = 64 * (lo(e) // 64 + e)`` and every
    segment is followed by zeros up to the next multiple of 64 columns.  Returns ``None`` when
    the kernel does not take the operand (not a 16-bit dtype, widths not multiples of 8):
    the caller then gathers with ``row_gather``.  No reference counterpart."""
    assert tokens.ndim == 2 and gather_indices.ndim == 1
    _C.require_cuda(tokens, gather_indices, group_indices)
    if tokens.dtype not in (torch.bfloat16, torch.float16):
        return None
    tokens = _rows(tokens)
    gather_indices = gather_indices.contiguous()
    assert group_indices.dtype == torch.int32
    gi = group_indices.contiguous()
    P, E = gather_indices.numel(), gi.numel() - 1
    lib = _C.load()
    cols = lib.moe_kmajor_columns(P, E)
    out = torch.empty((tokens.size(1), cols), device=tokens.device, dtype=tokens.dtype)
    if P == 0 or out.numel() == 0:
        return out
    st = lib.moe_row_gather_kmajor(
        tokens.data_ptr(), tokens.size(0), tokens.stride(0), gather_indices.data_ptr(),
        _C.idx_bytes(gather_indices), int(index_div), gi.data_ptr(), E, P, out.data_ptr(),
        out.stride(0), tokens.size(1), _C.dtype_code(tokens.dtype), _C.stream_of(tokens))
    if st == -2:  # MOE_ERR_UNSUPPORTED
        return None
    _C.check(st, "moe_row_gather_kmajor")
    return out
