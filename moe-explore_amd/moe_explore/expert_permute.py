"""Routing preprocessing and the unfused permute helpers
(reference ``expert_permute.py:8-68``)."""
from dataclasses import dataclass
from typing import Tuple, Union

import torch

from moe_explore import _C
from moe_explore.hip_kernels.row_gather_scatter import row_gather, row_scatter
from moe_explore.functional.scale_and_reduce import scale_and_reduce


@dataclass
class GroupedTokens:
    tokens: torch.Tensor
    group_indices: torch.Tensor
    indices: torch.Tensor


@dataclass
class PermToGroupIndices:
    group_indices: torch.Tensor
    indices: torch.Tensor


def get_token_indices(expert_indices, topk, num_experts, zero_prefix=False):
    """Sorts flat slot ids by expert and returns the expert offsets.

    ``indices`` (int64 ``[R]``) lists slot ids ``s = t*topk + j`` expert by expert,
    ascending inside an expert (the stable order; the reference's ``argsort`` leaves
    the order inside an expert unspecified, ``expert_permute.py:27``).
    ``group_indices`` is int32 ``[E+1]`` starting at 0 when ``zero_prefix`` else the
    int64 ``[E]`` inclusive prefix sum (``:31-36``).  One device pass, no host sync.
    """
    _C.require_cuda(expert_indices)
    flat = expert_indices.reshape(-1)
    if flat.dtype not in (torch.int32, torch.int64):
        flat = flat.to(torch.int64)
    flat = flat.contiguous()
    R, E = flat.numel(), int(num_experts)
    dev = flat.device
    lib = _C.load()
    indices = torch.empty(R, dtype=torch.int64, device=dev)
    group_indices = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inclusive = None if zero_prefix else torch.empty(E, dtype=torch.int64, device=dev)
    ws_bytes = lib.moe_route_workspace_bytes(R, E)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    st = lib.moe_route_preprocess(
        flat.data_ptr(), _C.idx_bytes(flat), R, E, indices.data_ptr(), group_indices.data_ptr(),
        _C.ptr(inclusive), ws.data_ptr(), ws.numel(), _C.stream_of(flat))
    _C.check(st, "moe_route_preprocess")
    return PermToGroupIndices(
        group_indices=group_indices if zero_prefix else inclusive,
        indices=indices,
    )


def get_token_indices_into(expert_indices, num_experts, indices_out, group_indices_out,
                           inclusive_out=None):
    """``get_token_indices`` for callers that may not allocate (HIP graph capture, serving
    loops with a fixed memory plan): the results go to the caller's tensors (``indices_out``
    int64 ``[R]``, ``group_indices_out`` int32 ``[E+1]``, optionally ``inclusive_out`` int64
    ``[E]``) and the per-chunk counts to a 4 MiB buffer inside the library, so nothing is
    allocated here or there.  ``expert_indices`` must already be a contiguous int32 / int64
    tensor.  Calls on one device share that buffer: keep them on one stream.  Raises
    ``MoeHipError`` when ``ceil(R / 512) * E`` exceeds 2**20 words."""
    _C.require_cuda(expert_indices, indices_out, group_indices_out, inclusive_out)
    assert expert_indices.is_contiguous() and expert_indices.dtype in (torch.int32, torch.int64)
    R, E = expert_indices.numel(), int(num_experts)
    assert indices_out.dtype == torch.int64 and indices_out.numel() == R and indices_out.is_contiguous()
    assert group_indices_out.dtype == torch.int32 and group_indices_out.numel() == E + 1
    assert inclusive_out is None or (inclusive_out.dtype == torch.int64 and inclusive_out.numel() == E)
    st = _C.load().moe_route_preprocess_noalloc(
        expert_indices.data_ptr(), _C.idx_bytes(expert_indices), R, E, indices_out.data_ptr(),
        group_indices_out.data_ptr(), _C.ptr(inclusive_out), _C.stream_of(expert_indices))
    _C.check(st, "moe_route_preprocess_noalloc")
    return PermToGroupIndices(group_indices=group_indices_out, indices=indices_out)


def expert_input_permute(tokens: torch.Tensor, expert_indices: torch.Tensor, num_experts: int,
                         topk: int) -> GroupedTokens:
    indices = get_token_indices(expert_indices, topk, num_experts, zero_prefix=True)
    output = row_gather(tokens, indices.indices, index_div=topk)
    return GroupedTokens(tokens=output, group_indices=indices.group_indices, indices=indices.indices)


def expert_output_permute(grouped_tokens: GroupedTokens, expert_scores: torch.Tensor, topk: int,
                          output_shape: Union[Tuple[int], torch.Size]) -> torch.Tensor:
    tokens = row_scatter(grouped_tokens.tokens, grouped_tokens.indices)
    return scale_and_reduce(tokens, expert_scores, expert_scores.size(0), topk, tokens.size(1))
