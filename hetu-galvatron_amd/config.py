"""The subset of the reference's model arguments the MoE layer reads, with the same field names and
defaults (galvatron/core/runtime/args_schema.py:126-156, :243 for init_method_std), so that a
`GalvatronModelArgs` instance can be passed wherever a `MoEConfig` is expected."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional

import torch
import torch.nn.functional as F


@dataclass
class MoEConfig:
    hidden_size: int = 4096
    num_moe_experts: int = 8
    moe_ffn_hidden_size: int = 14336
    moe_router_topk: int = 2
    moe_router_load_balancing_type: str = "aux_loss"  # none | aux_loss | seq_aux_loss | sinkhorn
    moe_router_score_function: str = "softmax"        # softmax | sigmoid
    moe_router_pre_softmax: bool = False
    moe_router_topk_scaling_factor: Optional[float] = None
    moe_router_num_groups: Optional[int] = None
    moe_router_group_topk: Optional[int] = None
    moe_router_enable_expert_bias: bool = False
    moe_router_dtype: Optional[str] = None            # None | fp32 | fp64
    moe_aux_loss_coeff: float = 0.0
    moe_z_loss_coeff: Optional[float] = None
    moe_token_dispatcher_type: str = "allgather"      # allgather | alltoall
    moe_expert_capacity_factor: Optional[float] = None
    moe_pad_expert_input_to_capacity: bool = False
    moe_token_drop_policy: str = "probs"
    moe_input_jitter_eps: Optional[float] = None
    moe_permute_fusion: bool = True
    moe_shared_expert_intermediate_size: Optional[int] = None
    moe_shared_expert_overlap: bool = False
    moe_grouped_gemm: bool = True
    gated_linear_unit: bool = True
    activation_func: Callable = F.silu
    add_bias_linear: bool = False
    bias_activation_fusion: bool = False              # args_schema.py:120
    activation_func_fp8_input_store: bool = False     # args_schema.py:121
    params_dtype: torch.dtype = torch.bfloat16
    calculate_per_token_loss: bool = False
    deterministic_mode: bool = False
    num_layers: int = 1
    init_method_std: float = 0.02
    normalization: str = "RMSNorm"                   # args_schema.py:115
    norm_epsilon: float = 1e-5                        # args_schema.py:116
