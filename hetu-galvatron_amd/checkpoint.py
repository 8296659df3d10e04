"""Expert-weight layouts: Hugging Face Mixtral (`w1`, `w3`, `w2` per expert), SequentialMLP
(`linear_fc1 [2F,H]`, `linear_fc2 [H,F]` per expert) and GroupedMLP (`weight1 [H, E*2F]` viewed
`[E,H,2F]`, `weight2 [E*F, H]` viewed `[E,F,H]`).

The reference loads Hugging Face checkpoints only into SequentialMLP (checkpoint/moe_adapter.py:
193-222: linear_fc1 = cat([w1, w3], dim 0), linear_fc2 = w2) and raises NotImplementedError for
the grouped layout (moe_adapter.py:195-196); the grouped form is the same matrices transposed per
expert, gate (w1) columns first, then up (w3) columns, as GroupedMLP.forward reads them
(moe/mlp.py:103-112).  The router gate, the expert bias and the pre-router norm load from the keys
the reference reads (moe_adapter.py:181-191).  Pure tensor reshaping: runs on any device.
"""
from __future__ import annotations

from typing import Dict, Sequence, Tuple

import torch

HF_EXPERT_KEY = "block_sparse_moe.experts.%d.%s.weight"


def fc_weights_from_hf(checkpoint: Dict[str, torch.Tensor], expert: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(linear_fc1 [2F,H], linear_fc2 [H,F]) of one expert (moe_adapter.py:209-222 at TP size 1)."""
    w1 = checkpoint[HF_EXPERT_KEY % (expert, "w1")]
    w3 = checkpoint[HF_EXPERT_KEY % (expert, "w3")]
    w2 = checkpoint[HF_EXPERT_KEY % (expert, "w2")]
    assert w1.shape == w3.shape and w2.shape == (w1.shape[1], w1.shape[0])
    return torch.cat([w1, w3], dim=0), w2


def grouped_from_fc(fc1: Sequence[torch.Tensor], fc2: Sequence[torch.Tensor]):
    """Per-expert linear_fc1 [2F,H] / linear_fc2 [H,F] -> (weight1 [H, E*2F], weight2 [E*F, H])
    whose memory, viewed [E,H,2F] / [E,F,H], holds expert e's matrices transposed."""
    E = len(fc1)
    assert E == len(fc2) and E > 0
    F2, H = fc1[0].shape
    w1 = torch.stack([w.t() for w in fc1], dim=0).contiguous()      # [E,H,2F]
    w2 = torch.stack([w.t() for w in fc2], dim=0).contiguous()      # [E,F,H]
    assert w2.shape == (E, F2 // 2, H)
    return w1.view(H, E * F2), w2.view(E * (F2 // 2), H)


def fc_from_grouped(weight1: torch.Tensor, weight2: torch.Tensor, num_experts: int):
    """Inverse of grouped_from_fc: lists of linear_fc1 [2F,H] and linear_fc2 [H,F]."""
    H = weight1.shape[0]
    w1 = weight1.contiguous().view(num_experts, H, -1)
    w2 = weight2.contiguous().view(num_experts, -1, H)
    return ([w1[e].t().contiguous() for e in range(num_experts)],
            [w2[e].t().contiguous() for e in range(num_experts)])


def grouped_from_hf(checkpoint: Dict[str, torch.Tensor], expert_indices: Sequence[int]):
    """Hugging Face Mixtral layer state -> GroupedMLP (weight1, weight2) for the given global
    expert indices (the branch the reference leaves unimplemented)."""
    pairs = [fc_weights_from_hf(checkpoint, e) for e in expert_indices]
    return grouped_from_fc([p[0] for p in pairs], [p[1] for p in pairs])


def hf_from_grouped(weight1: torch.Tensor, weight2: torch.Tensor, expert_indices: Sequence[int]):
    """GroupedMLP weights -> Hugging Face Mixtral keys for the given global expert indices."""
    fc1, fc2 = fc_from_grouped(weight1, weight2, len(expert_indices))
    out = {}
    for e, a, b in zip(expert_indices, fc1, fc2):
        half = a.shape[0] // 2
        out[HF_EXPERT_KEY % (e, "w1")] = a[:half].contiguous()
        out[HF_EXPERT_KEY % (e, "w3")] = a[half:].contiguous()
        out[HF_EXPERT_KEY % (e, "w2")] = b
    return out


@torch.no_grad()
def load_experts_from_hf(checkpoint: Dict[str, torch.Tensor], experts, local_expert_indices: Sequence[int]):
    """Fill a GroupedMLP or a SequentialMLP from a Hugging Face Mixtral layer state."""
    if hasattr(experts, "local_experts"):
        for expert, e in zip(experts.local_experts, local_expert_indices):
            fc1, fc2 = fc_weights_from_hf(checkpoint, e)
            expert.linear_fc1.weight.copy_(fc1.to(expert.linear_fc1.weight))
            expert.linear_fc2.weight.copy_(fc2.to(expert.linear_fc2.weight))
        return
    w1, w2 = grouped_from_hf(checkpoint, local_expert_indices)
    experts.weight1.copy_(w1.to(experts.weight1))
    experts.weight2.copy_(w2.to(experts.weight2))


@torch.no_grad()
def copy_sequential_to_grouped(sequential, grouped) -> None:
    w1, w2 = grouped_from_fc([e.linear_fc1.weight for e in sequential.local_experts],
                             [e.linear_fc2.weight for e in sequential.local_experts])
    grouped.weight1.copy_(w1.to(grouped.weight1))
    grouped.weight2.copy_(w2.to(grouped.weight2))


@torch.no_grad()
def copy_grouped_to_sequential(grouped, sequential) -> None:
    fc1, fc2 = fc_from_grouped(grouped.weight1, grouped.weight2, grouped.num_local_experts)
    for expert, a, b in zip(sequential.local_experts, fc1, fc2):
        expert.linear_fc1.weight.copy_(a.to(expert.linear_fc1.weight))
        expert.linear_fc2.weight.copy_(b.to(expert.linear_fc2.weight))


HF_ROUTER_KEY = "block_sparse_moe.gate.weight"
HF_EXPERT_BIAS_KEY = "block_sparse_moe.expert_bias"
HF_PRE_ROUTER_NORM_KEY = "post_attention_layernorm.weight"


@torch.no_grad()
def load_router_from_hf(checkpoint: Dict[str, torch.Tensor], router_module) -> None:
    """Gate weight [E,H] (and the expert bias when both sides have one) of a Hugging Face Mixtral
    layer state into a GalvatronMoERouter or a TopKRouter (moe_adapter.py:186-190)."""
    router = router_module.router if hasattr(router_module, "router") else router_module
    router.weight.copy_(checkpoint[HF_ROUTER_KEY].to(router.weight))
    bias = getattr(router, "expert_bias", None)
    if bias is not None and HF_EXPERT_BIAS_KEY in checkpoint:
        bias.copy_(checkpoint[HF_EXPERT_BIAS_KEY].to(bias))


@torch.no_grad()
def load_pre_router_norm_from_hf(checkpoint: Dict[str, torch.Tensor], norm_module) -> None:
    """`post_attention_layernorm.weight` into the pre-router norm (moe_adapter.py:181-183); accepts
    the norm itself or the PreRouterNorm wrapper."""
    norm = getattr(norm_module, "pre_router_norm", norm_module)
    norm.weight.copy_(checkpoint[HF_PRE_ROUTER_NORM_KEY].to(norm.weight))


@torch.no_grad()
def load_moe_layer_from_hf(checkpoint: Dict[str, torch.Tensor], router_module, mlp_module,
                           pre_router_norm=None) -> None:
    """One Hugging Face Mixtral decoder layer's MoE part into this package's modules: router gate,
    experts (grouped or sequential) and, when given, the pre-router norm."""
    load_router_from_hf(checkpoint, router_module)
    load_experts_from_hf(checkpoint, mlp_module.experts, mlp_module.local_expert_indices)
    if pre_router_norm is not None:
        load_pre_router_norm_from_hf(checkpoint, pre_router_norm)


def hf_from_moe_layer(router_module, mlp_module, pre_router_norm=None) -> Dict[str, torch.Tensor]:
    """The inverse: the Hugging Face keys of the layer's MoE part from the modules' parameters."""
    router = router_module.router if hasattr(router_module, "router") else router_module
    out = {HF_ROUTER_KEY: router.weight.detach().clone()}
    if getattr(router, "expert_bias", None) is not None:
        out[HF_EXPERT_BIAS_KEY] = router.expert_bias.detach().clone()
    experts = mlp_module.experts
    if hasattr(experts, "local_experts"):
        for e, expert in zip(mlp_module.local_expert_indices, experts.local_experts):
            fc1 = expert.linear_fc1.weight.detach()
            half = fc1.shape[0] // 2
            out[HF_EXPERT_KEY % (e, "w1")] = fc1[:half].clone()
            out[HF_EXPERT_KEY % (e, "w3")] = fc1[half:].clone()
            out[HF_EXPERT_KEY % (e, "w2")] = expert.linear_fc2.weight.detach().clone()
    else:
        out.update(hf_from_grouped(experts.weight1.detach(), experts.weight2.detach(),
                                   mlp_module.local_expert_indices))
    if pre_router_norm is not None:
        norm = getattr(pre_router_norm, "pre_router_norm", pre_router_norm)
        out[HF_PRE_ROUTER_NORM_KEY] = norm.weight.detach().clone()
    return out
