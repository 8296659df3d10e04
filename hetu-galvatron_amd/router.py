"""`Router` / `TopKRouter` with the reference's interface (galvatron/core/runtime/moe/router.py),
routing through the HIP top-k kernel.

forward(input [S,B,H]) -> (probs [T,E], routing_map [T,E] bool), T = S*B with token index s*B+b.
The gate projection (router.py:49-68) runs on the HIP gate kernels; everything after the logits is
one HIP kernel forward and one backward: score function, top-k, gates, routing map, per-expert
counts, and the statistics and gradients of the load-balancing loss (router.py:193-231, 278-314)
and of the z-loss (router.py:316-348).  The loss values, the logging tracker and the token counts of
the expert-bias scheme are updated by one bookkeeping launch on the device; the sequence-level
loss (router.py:233-276) and sinkhorn routing (router.py:140-171) have their own kernels.
"""
from __future__ import annotations

import torch

from . import ops
from .config import MoEConfig
from .moe_utils import (
    MoEAuxLossAutoScaler,
    _RouteTopK,
    _SeqAuxLoss,
    apply_expert_capacity,
    aux_losses_tracker_slot,
    save_to_aux_losses_tracker,
    z_loss_func,
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
        if router_dtype == torch.float64:
            raise ValueError("moe_router_dtype='fp64' is not supported: the gate projection runs on "
                             "the HIP kernels, which compute in fp32")
        weight = self.weight
        if weight.dtype != input.dtype:
            # F.linear(input.to(rd), weight.to(rd)): the casts stay torch's (and autograd's), the
            # product is the HIP kernels'
            input, weight = input.to(router_dtype), weight.to(router_dtype)
        if not ops.gate_supported(input, weight):
            raise ValueError("gate projection: unsupported operands (dtype %s / %s, hidden size %d, "
                             "%d experts)" % (input.dtype, weight.dtype, input.shape[-1], weight.shape[0]))
        # an fp32 router gets fp32 logits straight from 16-bit operands (their products are exact
        # in fp32, so no operand is cast)
        return _GateProjection.apply(input, weight, router_dtype)

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
        """Multiply the router input by noise drawn uniformly from [1 - eps, 1 + eps)
        (router.py:350-369); nothing happens when `moe_input_jitter_eps` is unset."""
        eps = self.config.moe_input_jitter_eps
        if eps is None:
            return input
        # the reference samples in fp32 (torch.distributions.Uniform of fp32 bounds), so a 16-bit
        # input is promoted to fp32 by the product
        noise = torch.empty(input.shape, dtype=torch.float32, device=input.device)
        return input * noise.uniform_(1.0 - eps, 1.0 + eps)

    # -- routing variants -------------------------------------------------------------------------
    def _route(self, logits, aux_coeff: float, z_coeff, selection=None, score_function=None,
               pre_softmax=None, plain=False):
        """One fused kernel: top-k + gates + counts (+ loss statistics when a coefficient is set),
        then one bookkeeping launch for the loss values, the tracker and the running token counts.
        `selection` [T,E] fp32 replaces the scores in the top-k; `plain` switches off scaling factor,
        groups, bias and capacity (sinkhorn routing uses none of them)."""
        cfg = self.config
        T, E = logits.shape
        score_function = score_function or self.score_function
        pre_softmax = cfg.moe_router_pre_softmax if pre_softmax is None else pre_softmax
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
        bias = None if plain or score_function != "sigmoid" else self.expert_bias
        if bias is not None:
            bias = bias.detach().to(torch.float32).contiguous()
        probs, routing_map, counts, stats = _RouteTopK.apply(
            logits.contiguous(), self.topk, score_function, pre_softmax,
            None if plain else cfg.moe_router_topk_scaling_factor, bias,
            None if plain else cfg.moe_router_num_groups, None if plain else cfg.moe_router_group_topk,
            aux_scale, z_scale, want_stats, selection)
        capacity = None if plain else cfg.moe_expert_capacity_factor
        # running token counts of the expert-bias scheme (router.py:415-419): the kernel's histogram,
        # unless tokens are dropped afterwards
        count_here = self.enable_expert_bias and torch.is_grad_enabled() and capacity is None
        if want_stats or count_here:
            with torch.no_grad():
                dev = logits.device
                track_aux, track_z = aux_scale != 0.0, z_scale != 0.0
                aux, z = ops.router_bookkeeping(
                    stats if want_stats else None, counts, E,
                    aux_factor=E * aux_coeff / (T * T * self.topk) if track_aux else 0.0,
                    z_factor=z_coeff / T if track_z else 0.0, want_aux=track_aux, want_z=track_z,
                    aux_slot=aux_losses_tracker_slot("load_balancing_loss", self.layer_idx,
                                                     cfg.num_layers, dev) if track_aux else None,
                    aux_slot_scale=1.0 / aux_coeff if track_aux else 1.0,
                    z_slot=aux_losses_tracker_slot("z_loss", self.layer_idx, cfg.num_layers, dev)
                    if track_z else None,
                    z_slot_scale=1.0 / z_coeff if track_z and z_coeff else 1.0,
                    local_tokens=self.local_tokens_per_expert if count_here else None)
                if track_aux:
                    self.last_aux_loss = aux
                if track_z:
                    self.last_z_loss = z
        if capacity is not None:
            probs, routing_map = apply_expert_capacity(
                probs, routing_map, self.topk, capacity, cfg.moe_pad_expert_input_to_capacity,
                cfg.moe_token_drop_policy)
            if self.enable_expert_bias and torch.is_grad_enabled():
                with torch.no_grad():
                    self.local_tokens_per_expert += routing_map.sum(dim=0)
        return probs, routing_map, counts

    # -- the reference's step-by-step methods ------------------------------------------------------
    # `routing` above goes through `_route`, where the loss statistics and gradients are part of the
    # routing kernels.  The methods the reference composes its routing from are kept for callers and
    # subclasses that use them one by one; they give the same values on the same device kernels.
    def compute_routing_scores_for_aux_loss(self, logits: torch.Tensor) -> torch.Tensor:
        """router.py:173-191: fp32 softmax over all experts, or the sigmoid scores divided by their
        sum per token (top-1: plain sigmoid).  The routing kernel with k = E: every expert selected."""
        E = logits.shape[-1]
        if self.score_function == "softmax":
            return _RouteTopK.apply(logits.float().contiguous(), E, "softmax", True, None, None, None,
                                    None)[0]
        if self.score_function == "sigmoid":
            if self.topk > 1:
                return _RouteTopK.apply(logits.contiguous(), E, "sigmoid", False, None, None, None,
                                        None)[0]
            return torch.sigmoid(logits)
        raise ValueError(f"Invalid score_function: {self.score_function}")

    def aux_loss_load_balancing(self, logits: torch.Tensor):
        """router.py:193-231: top-k routing with the switch load-balancing loss attached."""
        probs, routing_map, _ = self._route(logits, self.config.moe_aux_loss_coeff, None)
        return probs, routing_map

    def apply_load_balancing_loss(self, activation: torch.Tensor, load_balancing_loss_func):
        """router.py:278-314: evaluate the loss, log it, attach its gradient to `activation`."""
        coeff = self.config.moe_aux_loss_coeff
        if coeff == 0:
            return activation
        aux_loss = load_balancing_loss_func(moe_aux_loss_coeff=coeff, sequence_partition_group=None)
        save_to_aux_losses_tracker("load_balancing_loss", aux_loss / coeff, self.layer_idx,
                                   self.config.num_layers)
        if self.calculate_per_token_loss:
            aux_loss = aux_loss * activation.shape[0]
        return MoEAuxLossAutoScaler.apply(activation, aux_loss)

    def apply_z_loss(self, logits: torch.Tensor):
        """router.py:316-348: attach the z-loss to the logits (training with gradients only)."""
        coeff = self.config.moe_z_loss_coeff
        if coeff is not None and self.training and torch.is_grad_enabled():
            z_loss = z_loss_func(logits, coeff)
            scale_up = logits.shape[0] if self.calculate_per_token_loss else 1.0
            logits = MoEAuxLossAutoScaler.apply(logits, z_loss * scale_up)
            save_to_aux_losses_tracker("z_loss", z_loss / coeff, self.layer_idx, self.config.num_layers)
        return logits

    def sinkhorn_load_balancing(self, logits: torch.Tensor, z_coeff=None):
        """Sinkhorn routing (router.py:140-171).  Training: the experts are the top-k of the
        sinkhorn-normalised costs (one iteration kernel, no gradient), the gates the activation of
        the logits at those experts; evaluation: plain top-k of the activation.  Activation: sigmoid
        for top-1, else fp32 softmax over all experts cast back."""
        assert self.config.moe_aux_loss_coeff == 0, "Sinkhorn routing does not support aux loss."
        selection = ops.sinkhorn(logits.detach().contiguous()) if self.training else None
        scores, routing_map, _ = self._route(
            logits, 0.0, z_coeff, selection=selection, plain=True,
            score_function="sigmoid" if self.topk == 1 else "softmax", pre_softmax=self.topk > 1)
        return scores, routing_map

    def seq_aux_loss_load_balancing(self, logits, bsz: int, seq_length: int, z_coeff=None):
        """router.py:233-276: routing by the fused kernel; the per-sequence loss and its gradient by
        the sequence-statistics kernels, on the logits and the final routing map."""
        probs, routing_map, _ = self._route(logits, 0.0, z_coeff)
        coeff = self.config.moe_aux_loss_coeff
        if self.training and torch.is_grad_enabled() and coeff != 0:
            aux_loss = _SeqAuxLoss.apply(logits, routing_map, bsz, seq_length, self.topk, coeff,
                                         self.score_function)
            self.last_aux_loss = aux_loss.detach()
            save_to_aux_losses_tracker("load_balancing_loss", self.last_aux_loss / coeff,
                                       self.layer_idx, self.config.num_layers)
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
            scores, routing_map = self.sinkhorn_load_balancing(logits, z_coeff)
        elif self.routing_type == "aux_loss":
            scores, routing_map, _ = self._route(logits, self.config.moe_aux_loss_coeff, z_coeff)
        elif self.routing_type == "seq_aux_loss":
            scores, routing_map = self.seq_aux_loss_load_balancing(logits, bsz, seq_length, z_coeff)
        elif self.routing_type == "none":
            scores, routing_map, _ = self._route(logits, 0.0, z_coeff)
        else:
            raise ValueError(f"Unsupported MoE routing type: {self.routing_type}")
        return scores, routing_map

    def forward(self, input: torch.Tensor):
        """router.py:423-438."""
        self._maintain_float32_expert_bias()
        input = self.apply_input_jitter(input)
        logits = self.gating(input)
        if logits.dim() == 2:  # [T,H] input: treat as S=T, B=1
            logits = logits.unsqueeze(1)
        return self.routing(logits)
