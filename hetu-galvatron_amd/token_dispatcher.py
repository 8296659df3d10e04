"""Token dispatchers with the reference's interface (galvatron/core/runtime/moe/token_dispatcher.py),
local (EP = TP = 1) branches only: this build runs on one GPU and has no collectives.

    MoEAllGatherTokenDispatcher   token_dispatcher.py:116-284
    MoEAlltoAllTokenDispatcher    token_dispatcher.py:287-740

Both keep per-call state on `self` between token_permutation and token_unpermutation, as the
reference does, so one dispatcher instance serves one layer call at a time.

`tokens_per_expert` is returned as a DEVICE int64 tensor that carries the device-side
expert-offset table (attribute `_gmoe_offsets`): the grouped GEMM walks that table directly, so the
blocking device-to-host copy the reference makes once per layer (token_dispatcher.py:205,
:702-740) disappears.  `tokens_per_expert.cpu()` still gives the reference's value.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import ops
from .config import MoEConfig
from .moe_utils import _PermuteRows, _UnpermuteRows, get_capacity


class MoETokenDispatcher:
    def __init__(self, config: MoEConfig, ep_group=None, tp_of_ep_group=None, tp_and_ep_group=None):
        for g in (ep_group, tp_of_ep_group, tp_and_ep_group):
            assert g is None, "expert / tensor parallel groups need collectives (single GPU build)"
        self.config = config
        self.shared_experts = None
        self.tp_size = 1
        self.ep_size = 1

    def token_permutation(self, tokens, probs, routing_map):
        raise NotImplementedError("Dispatch function not implemented.")

    def token_unpermutation(self, expert_output, bias=None, residual=None, shared=None):
        raise NotImplementedError("Restore function not implemented.")

    def set_shared_experts(self, shared_experts):
        self.shared_experts = shared_experts


def _attach_offsets(counts: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    counts._gmoe_offsets = offsets
    return counts


class MoEAllGatherTokenDispatcher(MoETokenDispatcher):
    """Dropless dispatch to the local experts (all experts on one GPU)."""

    def __init__(self, num_local_experts: int, local_expert_indices: List[int], config: MoEConfig,
                 ep_group=None, tp_of_ep_group=None, tp_and_ep_group=None, layer_idx: int = None):
        super().__init__(config, ep_group, tp_of_ep_group, tp_and_ep_group)
        self.num_local_experts = num_local_experts
        assert self.num_local_experts > 0, "Expected at least one expert"
        self.local_expert_indices = local_expert_indices
        assert len(self.local_expert_indices) > 0, "Expected at least one local expert index"
        self.router_topk = config.moe_router_topk
        self.add_bias = config.add_bias_linear
        self.layer_idx = layer_idx

    def token_permutation(self, hidden_states, probs, routing_map):
        self.hidden_shape = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, self.hidden_shape[-1])
        self.hidden_shape_before_permute = hidden_states.shape
        e0, e1 = self.local_expert_indices[0], self.local_expert_indices[-1] + 1
        if e0 == 0 and e1 == routing_map.shape[1]:
            self.local_map, self.local_probs = routing_map.contiguous(), probs.contiguous()
        else:
            self.local_map = routing_map[:, e0:e1].contiguous()
            self.local_probs = probs[:, e0:e1].contiguous()
        T = hidden_states.shape[0]
        dropless = self.config.moe_expert_capacity_factor is None and e1 - e0 == routing_map.shape[1]
        # Rows of the permuted buffer, without reading the map on the host: every token keeps its k
        # experts when nothing is dropped; otherwise an upper bound (the rows past the experts' last
        # offset are zero-filled and never read: the grouped GEMM walks the offset table, the combine
        # the destination map), where the reference synchronises to size the buffer exactly
        # (token_dispatcher.py:205).
        n_out = T * min(self.router_topk, e1 - e0)
        cap = self.config.moe_expert_capacity_factor
        if cap is not None:
            n_out = min(n_out, (e1 - e0) * get_capacity(T * self.router_topk, routing_map.shape[1], cap))
        plan = ops.permute_plan(self.local_map, n_out, want_sorted=False)
        self._plan = plan
        # the same flag goes to the scatter and to the combine (whose backward fills the gradient
        # of the permuted rows): with a capacity factor >= 1 the bound above is T*k, yet tokens may
        # have been dropped and the rows past the last offset exist
        self._zero_fill = not dropless
        permuted = _PermuteRows.apply(hidden_states.contiguous(), plan.dst_map, n_out, self._zero_fill)
        self.reversed_local_input_permutation_mapping = plan.dst_map
        return permuted, _attach_offsets(plan.tokens_per_expert, plan.expert_offsets)

    def token_unpermutation(self, hidden_states, bias=None, residual=None, shared=None):
        """`shared` and `residual` (extensions of the reference's signature): tensors of the
        layer-input shape (the shared experts' output, the layer's residual) added to the combined
        rows in the same pass, in that order, each with the rounding of a separate add."""
        plan = self._plan
        unpermuted_bias = None
        if self.add_bias:
            # token_dispatcher.py:246-258, 277-283: the bias rows take the same gate weighting and
            # combine as the expert output, returned beside it and not added
            assert bias is not None
            if bias.dim() == 1:  # a single local expert hands back its [H] bias (moe/mlp.py:184-186)
                from .mlp import expand_bias
                bias = expand_bias(bias, plan.n_out)
            unpermuted_bias = _UnpermuteRows.apply(bias.contiguous(), plan.dst_map, self.local_probs,
                                                   plan.num_tokens, self._zero_fill, None, None)
            unpermuted_bias = unpermuted_bias.view(self.hidden_shape)
        else:
            assert bias is None, "the experts returned a bias although add_bias_linear is off"
        if residual is not None:
            residual = residual.reshape(plan.num_tokens, -1).contiguous()
        if shared is not None:
            shared = shared.reshape(plan.num_tokens, -1).contiguous()
        # gate weighting and the k-way reduction in one pass, fp32 accumulation
        # (token_dispatcher.py:233-244 does a multiply followed by scatter_add_)
        out = _UnpermuteRows.apply(hidden_states.contiguous(), plan.dst_map, self.local_probs,
                                   plan.num_tokens, self._zero_fill, residual, shared)
        return out.view(self.hidden_shape), unpermuted_bias


class MoEAlltoAllTokenDispatcher(MoETokenDispatcher):
    """AlltoAll dispatcher at EP = TP = 1: permute -> (identity exchange) -> experts -> unpermute with
    the gate weighting inside unpermute (token_dispatcher.py:510-689)."""

    def __init__(self, num_local_experts: int, local_expert_indices: List[int], config: MoEConfig,
                 ep_group=None, tp_of_ep_group=None, tp_and_ep_group=None, layer_idx: int = None):
        super().__init__(config, ep_group, tp_of_ep_group, tp_and_ep_group)
        self.layer_idx = layer_idx
        self.num_local_experts = num_local_experts
        self.num_experts = config.num_moe_experts
        assert self.num_local_experts > 0, "Expected at least one expert"
        assert len(local_expert_indices) == self.num_local_experts, "Invalid local expert indices"
        for i in range(len(local_expert_indices) - 1):
            assert local_expert_indices[i] == local_expert_indices[i + 1] - 1, \
                "local_expert_indices must be continous"
        assert self.num_local_experts == self.num_experts, "EP > 1 needs collectives (single GPU build)"
        self.local_expert_indices = local_expert_indices
        self.drop_and_pad = config.moe_pad_expert_input_to_capacity
        if self.drop_and_pad:
            assert config.moe_expert_capacity_factor is not None
        self.capacity = None

    def preprocess(self, routing_map: torch.Tensor):
        """Output size of the permutation (token_dispatcher.py:379-508, local branch)."""
        T = routing_map.size(0)
        if self.drop_and_pad:
            self.capacity = get_capacity(T * self.config.moe_router_topk, self.num_experts,
                                         self.config.moe_expert_capacity_factor)
            self.num_out_tokens = self.capacity * self.num_experts
        elif self.config.moe_expert_capacity_factor is not None:
            # tokens were dropped: an upper bound instead of a host read of the map (the rows past
            # the experts' last offset are zero-filled and never read)
            self.capacity = None
            self.num_out_tokens = min(T * self.config.moe_router_topk, self.num_experts * get_capacity(
                T * self.config.moe_router_topk, self.num_experts, self.config.moe_expert_capacity_factor))
        else:
            self.num_out_tokens = T * self.config.moe_router_topk

    def token_permutation(self, hidden_states, probs, routing_map):
        self.hidden_shape = hidden_states.shape
        self.probs = probs
        self.routing_map = routing_map
        assert probs.dim() == 2, "Expected 2D tensor for probs"
        assert routing_map.dim() == 2, "Expected 2D tensor for token2expert mask"
        assert routing_map.dtype == torch.bool, "Expected bool tensor for mask"
        hidden_states = hidden_states.reshape(-1, self.hidden_shape[-1])
        self.preprocess(routing_map)
        self.hidden_shape_before_permute = hidden_states.shape
        plan = ops.permute_plan(routing_map, self.num_out_tokens,
                                capacity=self.capacity if self.drop_and_pad else 0, want_sorted=False)
        self._plan = plan
        bounded = self.config.moe_expert_capacity_factor is not None
        permuted = _PermuteRows.apply(hidden_states.contiguous(), plan.dst_map, plan.n_out,
                                      plan.padded or bounded)
        self.reversed_local_input_permutation_mapping = plan.dst_map
        return permuted, _attach_offsets(plan.tokens_per_expert, plan.expert_offsets)

    def token_unpermutation(self, hidden_states, bias: Optional[torch.Tensor] = None, residual=None,
                            shared=None):
        assert bias is None, "Bias is not supported in MoEAlltoAllTokenDispatcher"
        plan = self._plan
        if residual is not None:
            residual = residual.reshape(plan.num_tokens, -1).contiguous()
        if shared is not None:
            shared = shared.reshape(plan.num_tokens, -1).contiguous()
        out = _UnpermuteRows.apply(hidden_states.contiguous(), plan.dst_map, self.probs.contiguous(),
                                   plan.num_tokens,
                                   plan.padded or self.config.moe_expert_capacity_factor is not None,
                                   residual, shared)
        return out.view(self.hidden_shape), None
