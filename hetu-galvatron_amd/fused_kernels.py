"""TE-2.1-style fused permutation API on the HIP kernels.

Mirrors the three names the reference imports at moe/moe_utils.py:10 from moe/fused_kernels.py:
`moe_permute` (:398-438), `moe_unpermute` (:10-53) and `moe_sort_chunks_by_index` (:762-782).

`row_id_map` is opaque to callers in that API (it is only handed from moe_permute to
moe_unpermute).  Here it is the token-major destination table, int32 [T,E]: entry (t,e) is the row
of token t inside expert e's block of the permuted tensor, or -1.  `row_id_map_reference_layout`
converts it to the reference's int64 [E,T] layout for comparisons.

Beyond the reference: map_type='index' is supported, and unpermute without probs has a backward.
"""
from __future__ import annotations

import warnings
from typing import Tuple

import torch

from . import ops
from .moe_utils import _PermuteRows, _UnpermuteRows, _SortChunks


def row_id_map_reference_layout(row_id_map: torch.Tensor) -> torch.Tensor:
    """int32 [T,E] destination table -> int64 [E,T] (layout of triton_make_row_id_map,
    moe/fused_kernels.py:514-541)."""
    return row_id_map.t().contiguous().to(torch.int64)


def _index_to_mask(routing_idx: torch.Tensor, num_experts: int) -> torch.Tensor:
    mask = torch.zeros((routing_idx.shape[0], num_experts), dtype=torch.bool, device=routing_idx.device)
    mask.scatter_(1, routing_idx.long(), True)
    return mask


def moe_permute(inp: torch.Tensor, routing_map: torch.Tensor, num_out_tokens: int = -1,
                max_token_num: int = -1, map_type: str = "mask",
                num_experts: int = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Permute the tokens by expert.  routing_map: [T,E] mask (bool / int) for map_type='mask', or
    [T,topK] expert indices for map_type='index' (needs num_experts)."""
    if map_type not in ("mask", "index"):
        raise ValueError("map_type should be one of 'mask' or 'index'")
    if not inp.numel():
        return inp, torch.tensor([], device=inp.device)
    assert inp.is_cuda and routing_map.is_cuda, "the fused permute needs GPU tensors"
    assert inp.size(0) == routing_map.size(0), "Permute not possible"
    if map_type == "index":
        assert num_experts is not None, "map_type='index' needs num_experts"
        routing_map = _index_to_mask(routing_map, num_experts)
    assert num_out_tokens is not None, "num_out_tokens must be provided to the fused permute function."
    if torch.is_tensor(num_out_tokens):
        num_out_tokens = int(num_out_tokens.item())
    if num_out_tokens < 0:
        # "no tokens are dropped": the size is data dependent, one host read
        num_out_tokens = int(routing_map.bool().sum().item())
    plan = ops.permute_plan(routing_map, num_out_tokens, want_sorted=False)
    out = _PermuteRows.apply(inp.contiguous(), plan.dst_map, plan.n_out, False)
    return out, plan.dst_map


def moe_unpermute(inp: torch.Tensor, row_id_map: torch.Tensor, merging_probs: torch.Tensor = None,
                  restore_shape: torch.Size = None, map_type: str = "mask",
                  probs: torch.Tensor = None) -> torch.Tensor:
    """Unpermute (and optionally merge with probabilities), fp32 accumulation."""
    if probs is not None:
        if merging_probs is not None:
            raise ValueError("Both merging_probs and probs kwarg are provided. probs is deprecated.")
        warnings.warn("probs kwarg is deprecated. Use merging_probs kwarg instead.")
        merging_probs = probs
    if map_type not in ("mask", "index"):
        raise ValueError("map_type should be one of 'mask' or 'index'")
    if not inp.numel():
        return inp
    assert inp.is_cuda and row_id_map.is_cuda, "the fused unpermute needs GPU tensors"
    assert row_id_map.dtype == torch.int32 and row_id_map.dim() == 2, \
        "row_id_map must be the table returned by moe_permute"
    num_tokens = row_id_map.shape[0]
    if restore_shape is not None:
        assert restore_shape[0] == num_tokens and restore_shape[1] == inp.shape[1]
    if merging_probs is not None:
        merging_probs = merging_probs.contiguous()
    return _UnpermuteRows.apply(inp.contiguous(), row_id_map, merging_probs, num_tokens, False)


def moe_sort_chunks_by_index(inp: torch.Tensor, split_sizes: torch.Tensor,
                             sorted_index: torch.Tensor) -> torch.Tensor:
    """Split `inp` along dim 0 by split_sizes and concatenate the chunks in sorted_index order."""
    if not inp.numel():
        return inp
    assert split_sizes.numel() == sorted_index.numel()
    return _SortChunks.apply(inp.contiguous(), split_sizes, sorted_index)
