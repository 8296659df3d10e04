"""`GalvatronMoERouter` / `GalvatronMoEMLP` with the reference's forward contracts
(galvatron/core/runtime/models/moe_modules.py:33-128) on one GPU:

    probs, routing_map = GalvatronMoERouter(config)(hidden_states[S,B,H])
    out = GalvatronMoEMLP(config)(hidden_states, mlp_residual, probs, routing_map)
        = unpermute(experts(permute(hidden_states))) [+ shared experts] + mlp_residual
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .config import MoEConfig
from .mlp import GroupedMLP, SequentialMLP, SharedExpertMLP
from .router import TopKRouter
from .token_dispatcher import MoEAllGatherTokenDispatcher, MoEAlltoAllTokenDispatcher


class GalvatronMoERouter(nn.Module):
    def __init__(self, config: MoEConfig, layer_idx: int = 1, device=None):
        super().__init__()
        self.layer_idx = layer_idx
        self.init_method_std = config.init_method_std
        self.router = TopKRouter(config=config)
        self.router.set_layer_idx(layer_idx)
        if device is not None:
            self.router.to(device)
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.normal_(self.router.weight, mean=0.0, std=self.init_method_std)
        if getattr(self.router, "expert_bias", None) is not None:
            self.router.expert_bias.zero_()
        if getattr(self.router, "local_tokens_per_expert", None) is not None:
            self.router.local_tokens_per_expert.zero_()

    def forward(self, hidden_states):
        return self.router(hidden_states)


class GalvatronMoEMLP(nn.Module):
    def __init__(self, config: MoEConfig, layer_idx: int = 1, ep_group=None, tp_of_ep_group=None,
                 tp_and_ep_group=None, device=None):
        super().__init__()
        assert ep_group is None and tp_of_ep_group is None and tp_and_ep_group is None, \
            "expert parallel groups need collectives (single GPU build)"
        self.layer_idx = layer_idx
        self.num_local_experts = config.num_moe_experts
        self.local_expert_indices = list(range(self.num_local_experts))
        kwargs = dict(num_local_experts=self.num_local_experts,
                      local_expert_indices=self.local_expert_indices, config=config,
                      layer_idx=layer_idx)
        if config.moe_token_dispatcher_type == "allgather":
            self.token_dispatcher = MoEAllGatherTokenDispatcher(**kwargs)
        elif config.moe_token_dispatcher_type == "alltoall":
            self.token_dispatcher = MoEAlltoAllTokenDispatcher(**kwargs)
        elif config.moe_token_dispatcher_type == "alltoall_seq":
            assert False, "alltoall_seq is deprecated"
        elif config.moe_token_dispatcher_type == "flex":
            raise ValueError("the flex (DeepEP) dispatcher needs multi-GPU communication")
        else:
            raise ValueError(f"Unsupported MoE dispatcher type: {config.moe_token_dispatcher_type}")
        if config.moe_grouped_gemm:
            self.experts = GroupedMLP(self.num_local_experts, config, layer_idx=layer_idx, device=device)
        else:
            # the layout the reference's checkpoints load into (models/moe_modules.py:97-105)
            self.experts = SequentialMLP(self.num_local_experts, config, layer_idx=layer_idx,
                                         device=device)
        self.shared_experts = None
        if config.moe_shared_expert_intermediate_size is not None:
            self.shared_experts = SharedExpertMLP(config, device=device)
        self.shared_expert_overlap = bool(config.moe_shared_expert_overlap) \
            and self.shared_experts is not None

    def forward(self, hidden_states, mlp_residual, probs, routing_map):
        shared = self.shared_experts
        if self.shared_expert_overlap:
            shared.pre_forward_comm(hidden_states)  # the stages run on the shared experts' stream
        dispatched_input, tokens_per_expert = self.token_dispatcher.token_permutation(
            hidden_states, probs, routing_map)
        if self.shared_expert_overlap:
            shared.linear_fc1_forward_and_act()
        expert_output, mlp_bias = self.experts(dispatched_input, tokens_per_expert)
        shared_out = None
        if self.shared_expert_overlap:
            shared.linear_fc2_forward()
            shared.post_forward_comm()
            shared_out = shared.get_output()
        elif shared is not None:
            shared_out = shared(hidden_states)
        # `output += shared_expert_output` (moe/token_dispatcher.py:686-688) and
        # `... + mlp_residual` (models/moe_modules.py:124-127) happen inside the combine kernel, with
        # the roundings of the separate adds
        fuse = lambda t: t is None or t.dtype == expert_output.dtype  # noqa: E731
        if fuse(shared_out) and fuse(mlp_residual):
            out, _ = self.token_dispatcher.token_unpermutation(expert_output, mlp_bias,
                                                               residual=mlp_residual, shared=shared_out)
            return out
        out, _ = self.token_dispatcher.token_unpermutation(expert_output, mlp_bias)
        if shared_out is not None:
            out = out + shared_out
        if mlp_residual is not None:
            out = out + mlp_residual
        return out
