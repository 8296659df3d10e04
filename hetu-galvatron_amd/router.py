"""`Router` / `TopKRouter` with the reference's interface (galvatron/core/runtime/moe/router.py),
routing through the HIP top-k kernel.

forward(input [S,B,H]) -> (probs [T,E], routing_map [T,E] bool), T = S*B with token index s*B+b.
The gate projection is a plain dense GEMM and goes to the BLAS library (F.linear), as in the
reference (router.py:49-68); everything after the logits is one HIP kernel forward and one backward:
score function, top-k, gates, routing map, per-expert counts, and the statistics and gradients of the
load-balancing loss (router.py:193-231, 278-314) and of the z-loss (router.py:316-348).
"""
from __future__ import annotations

from functools import partial

import torch

from . import ops
from .config import MoEConfig
from .moe_utils import (
    MoEAuxLossAutoScaler,
    _RouteTopK,
    apply_expert_capacity,
    save_to_aux_losses_tracker,
    sequence_load_balancing_loss_func,
    sinkhorn,
)


class _GateProjection(torch.autograd.Function):
    """F.linear(input.to(router_dtype), weight.to(router_dtype)) (router.py:49-68) on the HIP gate
    kernels; gradients come back in the dtypes of input and weight, as autograd of the casts gives."""

    @staticmethod
    def forward(ctx, x, weight, router_dtype):
        x = x.contiguous()
        ctx.save_for_backward(x, weight)
        return ops.gate_fwd(x, weight, out_dtype=router_dtype)

    @staticmethod
    def backward(ctx, dlogits):
        x, weight = ctx.saved_tensors
        dx, dw = ops.gate_bwd(dlogits.contiguous(), x, weight, need_dx=ctx.needs_input_grad[0],
                              need_dw=ctx.needs_input_grad[1])
        return dx, dw, None


class Router(torch.nn.Module):
    """Base router: owns the gate weight [num_experts, hidden] (router.py:22-68)."""

    def __init__(self, config: MoEConfig) -> None:
        super().__init__()
        self.config = config
        self.num_experts = config.num_moe_experts
        self.layer_idx = None
        self.weight = torch.nn.Parameter(
            torch.empty((config.num_moe_experts, config.hidden_size), dtype=torch.float32))
        self.weight.data = self.weight.data.to(dtype=config.params_dtype)
        self.calculate_per_token_loss = config.calculate_per_token_loss

    def gating(self, input: torch.Tensor) -> torch.Tensor:
        if self.weight.device.type == "cpu":
            self.weight.data = self.weight.data.to(device=torch.cuda.current_device())
        router_dtype = input.dtype
        if self.config.moe_router_dtype == "fp32":
            router_dtype = torch.float32
        elif self.config.moe_router_dtype == "fp64":
            router_dtype = torch.float64
        if router_dtype != torch.float64 and input.is_cuda and ops.gate_supported(input, self.weight):
            # small expert counts: the HIP gate projection; an fp32 router gets fp32 logits straight
            # from the 16-bit operands (their products are exact in fp32, so no operand is cast)
            return _GateProjection.apply(input, self.weight, router_dtype)
        return torch.nn.functional.linear(input.to(router_dtype), self.weight.to(router_dtype))

    def routing(self, logits: torch.Tensor):
        raise NotImplementedError("Routing function not implemented.")

    def forward(self, input: torch.Tensor):
        raise NotImplementedError("Forward function not implemented.")

    def set_layer_idx(self, layer_idx: int):
        self.layer_idx = layer_idx


class TopKRouter(Router):
    """Route each token to its top-k experts (router.py:100-437)."""

    def __init__(self, config: MoEConfig) -> None:
        super().__init__(config=config)
        self.topk = config.moe_router_topk
        self.routing_type = config.moe_router_load_balancing_type
        self.score_function = config.moe_router_score_function
        self.input_jitter = None
        self.enable_expert_bias = config.moe_router_enable_expert_bias
        if self.enable_expert_bias:
            self.register_buffer("local_tokens_per_expert",
                                 torch.zeros(config.num_moe_experts, dtype=torch.float32),
                                 persistent=False)
            self.register_buffer("expert_bias", torch.zeros(config.num_moe_experts, dtype=torch.float32))
        else:
            self.local_tokens_per_expert = None
            self.expert_bias = None
        # value of the auxiliary losses of the last forward (device scalars), for logging and tests
        self.last_aux_loss = None
        self.last_z_loss = None

    def _maintain_float32_expert_bias(self):
        if getattr(self, "expert_bias", None) is not None and self.expert_bias.dtype != torch.float32:
            self.expert_bias.data = self.expert_bias.data.to(torch.float32)

    def apply_input_jitter(self, input: torch.Tensor):
        eps = self.config.moe_input_jitter_eps
        if eps is None:
            return input
        if self.input_jitter is None:
            self.input_jitter = torch.distributions.uniform.Uniform(
                torch.tensor(1.0 - eps, device=input.device),
                torch.tensor(1.0 + eps, device=input.device)).rsample
        return input * self.input_jitter(input.shape)

    # -- routing variants -------------------------------------------------------------------------
    def _route(self, logits, aux_coeff: float, z_coeff):
        """One fused kernel: top-k + gates + counts (+ loss statistics when a coefficient is set)."""
        cfg = self.config
        T, E = logits.shape
        train = self.training and torch.is_grad_enabled()
        per_token = float(T) if self.calculate_per_token_loss else 1.0
        aux_scale = z_scale = 0.0
        if train and aux_coeff:
            # d/dlogits of aux = sum_e P_e f_e * E*coeff/(T^2 k)   (moe_utils.py:55-58)
            aux_scale = E * aux_coeff / (T * T * self.topk) * per_token
        if train and z_coeff is not None:
            # d/dlogits of z = coeff * mean_t lse_t^2             (moe_utils.py:126)
            z_scale = z_coeff / T * per_token
        want_stats = aux_scale != 0.0 or z_scale != 0.0
        bias = self.expert_bias if self.score_function == "sigmoid" else None
        if bias is not None:
            bias = bias.detach().to(torch.float32).contiguous()
        probs, routing_map, counts, stats = _RouteTopK.apply(
            logits.contiguous(), self.topk, self.score_function, cfg.moe_router_pre_softmax,
            cfg.moe_router_topk_scaling_factor, bias, cfg.moe_router_num_groups,
            cfg.moe_router_group_topk, aux_scale, z_scale, want_stats)
        if want_stats:
            with torch.no_grad():
                if aux_scale != 0.0:
                    aux = torch.sum(stats[:E] * counts) * (E * aux_coeff / (T * T * self.topk))
                    self.last_aux_loss = aux
                    save_to_aux_losses_tracker("load_balancing_loss", aux / aux_coeff, self.layer_idx,
                                               cfg.num_layers)
                if z_scale != 0.0:
                    z = stats[E] * (z_coeff / T)
                    self.last_z_loss = z
                    save_to_aux_losses_tracker("z_loss", z / z_coeff, self.layer_idx, cfg.num_layers)
        if cfg.moe_expert_capacity_factor is not None:
            probs, routing_map = apply_expert_capacity(
                probs, routing_map, self.topk, cfg.moe_expert_capacity_factor,
                cfg.moe_pad_expert_input_to_capacity, cfg.moe_token_drop_policy)
        return probs, routing_map, counts

    def sinkhorn_load_balancing(self, logits: torch.Tensor):
        """router.py:140-171; selection by torch.topk on the normalised costs."""

        def _activation(lg):
            if self.topk == 1:
                return torch.sigmoid(lg)
            return torch.softmax(lg, dim=-1, dtype=torch.float32).type_as(lg)

        assert self.config.moe_aux_loss_coeff == 0, "Sinkhorn routing does not support aux loss."
        if self.training:
            with torch.no_grad():
                norm_logits = sinkhorn(logits.to(dtype=torch.float32))
                _, indices = torch.topk(norm_logits, k=self.topk, dim=1)
            logits = _activation(logits)
        else:
            logits = _activation(logits)
            _, indices = torch.topk(logits, k=self.topk, dim=1)
        rmap = torch.zeros_like(logits).int().scatter(1, indices, 1).bool()
        return logits * rmap, rmap

    def seq_aux_loss_load_balancing(self, logits, bsz: int, seq_length: int, z_coeff):
        """router.py:233-276: routing by the fused kernel, per-sequence loss with torch ops."""
        probs, routing_map, _ = self._route(logits, 0.0, z_coeff)
        coeff = self.config.moe_aux_loss_coeff
        if self.training and torch.is_grad_enabled() and coeff != 0:
            if self.score_function == "softmax":
                scores = torch.softmax(logits, dim=-1, dtype=torch.float32)
            else:
                scores = torch.sigmoid(logits)
                scores = scores / (scores.sum(dim=-1, keepdim=True) + 1e-20) if self.topk > 1 else scores
            aux_loss = sequence_load_balancing_loss_func(
                probs=scores, routing_map=routing_map, batch_size=bsz, seq_length=seq_length,
                topk=self.topk, moe_aux_loss_coeff=coeff)
            self.last_aux_loss = aux_loss.detach()
            save_to_aux_losses_tracker("load_balancing_loss", aux_loss / coeff, self.layer_idx,
                                       self.config.num_layers)
            if self.calculate_per_token_loss:
                aux_loss = aux_loss * probs.shape[0]
            probs = MoEAuxLossAutoScaler.apply(probs, aux_loss)
        return probs, routing_map

    def routing(self, logits: torch.Tensor):
        """router.py:371-421."""
        seq_length, bsz = logits.shape[:2]
        logits = logits.view(-1, self.config.num_moe_experts)
        z_coeff = self.config.moe_z_loss_coeff
        if self.routing_type == "sinkhorn":
            if z_coeff is not None and self.training and torch.is_grad_enabled():
                from .moe_utils import z_loss_func
                z = z_loss_func(logits, z_coeff)
                self.last_z_loss = z.detach()
                logits = MoEAuxLossAutoScaler.apply(
                    logits, z * logits.shape[0] if self.calculate_per_token_loss else z)
            scores, routing_map = self.sinkhorn_load_balancing(logits)
        elif self.routing_type == "aux_loss":
            scores, routing_map, _ = self._route(logits, self.config.moe_aux_loss_coeff, z_coeff)
        elif self.routing_type == "seq_aux_loss":
            scores, routing_map = self.seq_aux_loss_load_balancing(logits, bsz, seq_length, z_coeff)
        elif self.routing_type == "none":
            scores, routing_map, _ = self._route(logits, 0.0, z_coeff)
        else:
            raise ValueError(f"Unsupported MoE routing type: {self.routing_type}")
        if self.enable_expert_bias and torch.is_grad_enabled():
            with torch.no_grad():
                self.local_tokens_per_expert += routing_map.sum(dim=0)
        return scores, routing_map

    def forward(self, input: torch.Tensor):
        """router.py:423-438."""
        self._maintain_float32_expert_bias()
        input = self.apply_input_jitter(input)
        logits = self.gating(input)
        if logits.dim() == 2:  # [T,H] input: treat as S=T, B=1
            logits = logits.unsqueeze(1)
        return self.routing(logits)
