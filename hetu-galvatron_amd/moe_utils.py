"""Reference-named MoE utilities running on the HIP kernels.

Same names, arguments and error behaviour as galvatron/core/runtime/moe/moe_utils.py so that the
reference's call sites (moe/router.py, moe/token_dispatcher.py) work unchanged:

    permute / unpermute / sort_chunks_by_idxs      moe_utils.py:219-369
    topk_softmax_with_capacity                      moe_utils.py:430-544
    switch_load_balancing_loss_func, z_loss_func,
    sequence_load_balancing_loss_func, sinkhorn     moe_utils.py:14-144
    get_capacity, MoEAuxLossAutoScaler              moe_utils.py:147-216

Differences that callers can observe, all inside the reference's documented contract:
  * `fused=True` is honoured (the reference raises because its TE gate is hard-wired off); both
    values of `fused` run the same HIP kernels.
  * top-k ties go to the lowest expert index (torch.topk leaves ties unspecified).
  * unpermute accumulates the k expert rows of a token in fp32 whatever the probs dtype.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

from . import ops

HAVE_TE = True  # the fused path is always available here


# ---------------------------------------------------------------------------------------------
# Losses (tiny tensors; plain torch, device-agnostic, same formulae as the reference)
# ---------------------------------------------------------------------------------------------

def switch_load_balancing_loss_func(probs, tokens_per_expert, topk, moe_aux_loss_coeff,
                                    sequence_partition_group=None):
    """moe_utils.py:14-59."""
    if sequence_partition_group is not None:
        raise NotImplementedError("sequence-partitioned aux loss needs collectives (single GPU build)")
    num_tokens, num_experts = probs.shape
    aggregated_probs_per_expert = probs.sum(dim=0)
    return torch.sum(aggregated_probs_per_expert * tokens_per_expert) * (
        num_experts * moe_aux_loss_coeff / (num_tokens * num_tokens * topk))


def sequence_load_balancing_loss_func(probs, routing_map, batch_size, seq_length, topk,
                                      moe_aux_loss_coeff, sequence_partition_group=None):
    """moe_utils.py:62-112."""
    if sequence_partition_group is not None:
        raise NotImplementedError("sequence-partitioned aux loss needs collectives (single GPU build)")
    num_experts = probs.shape[1]
    probs_for_aux_loss = probs.view(seq_length, batch_size, -1)
    routing_map = routing_map.view(seq_length, batch_size, -1)
    cost_coeff = routing_map.sum(dim=0, dtype=torch.float).div_(seq_length * topk / num_experts)
    seq_aux_loss = (cost_coeff * probs_for_aux_loss.mean(dim=0)).sum(dim=1).mean()
    return seq_aux_loss * moe_aux_loss_coeff


def z_loss_func(logits, z_loss_coeff):
    """moe_utils.py:115-127."""
    return torch.mean(torch.square(torch.logsumexp(logits, dim=-1))) * z_loss_coeff


def sinkhorn(cost: torch.Tensor, tol: float = 0.0001):
    """moe_utils.py:130-144."""
    cost = torch.exp(cost)
    d0 = torch.ones(cost.size(0), device=cost.device, dtype=cost.dtype)
    d1 = torch.ones(cost.size(1), device=cost.device, dtype=cost.dtype)
    eps = 0.00000001
    error = 1e9
    d1_old = d1
    while error > tol:
        d0 = (1 / d0.size(0)) * 1 / (torch.sum(d1 * cost, 1) + eps)
        d1 = (1 / d1.size(0)) * 1 / (torch.sum(d0.unsqueeze(1) * cost, 0) + eps)
        error = torch.mean(torch.abs(d1_old - d1))
        d1_old = d1
    return d1 * cost * d0.unsqueeze(1)


def get_capacity(num_tokens: int, num_experts: int, capacity_factor: float, min_capacity=None):
    """moe_utils.py:147-163."""
    capacity = math.ceil((num_tokens / num_experts) * capacity_factor)
    if min_capacity is not None and capacity < min_capacity:
        capacity = min_capacity
    return capacity


class MoEAuxLossAutoScaler(torch.autograd.Function):
    """Identity on `output` whose backward injects d(aux_loss) = main_loss_backward_scale
    (moe_utils.py:166-216)."""

    main_loss_backward_scale: torch.Tensor = None

    @staticmethod
    def forward(ctx, output: torch.Tensor, aux_loss: torch.Tensor):
        ctx.save_for_backward(aux_loss)
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (aux_loss,) = ctx.saved_tensors
        if MoEAuxLossAutoScaler.main_loss_backward_scale is None:
            MoEAuxLossAutoScaler.main_loss_backward_scale = torch.tensor(1.0, device=aux_loss.device)
        scale = MoEAuxLossAutoScaler.main_loss_backward_scale
        return grad_output, torch.ones_like(aux_loss) * scale

    @staticmethod
    def set_loss_scale(scale: torch.Tensor):
        if MoEAuxLossAutoScaler.main_loss_backward_scale is None:
            MoEAuxLossAutoScaler.main_loss_backward_scale = scale
        else:
            MoEAuxLossAutoScaler.main_loss_backward_scale.copy_(scale)


# ---------------------------------------------------------------------------------------------
# Permute / unpermute
# ---------------------------------------------------------------------------------------------

class _PermuteRows(torch.autograd.Function):
    """permuted[dst_map[t,e]] = tokens[t]; backward sums the k gradients of a token in fp32."""

    @staticmethod
    def forward(ctx, tokens, dst_map, n_out, padded):
        out, _ = ops.permute_rows(tokens, dst_map, n_out, zero_fill=padded)
        ctx.save_for_backward(dst_map)
        ctx.num_tokens = tokens.shape[0]
        return out

    @staticmethod
    def backward(ctx, grad_permuted):
        (dst_map,) = ctx.saved_tensors
        grad, _ = ops.unpermute_rows(grad_permuted.contiguous(), dst_map, ctx.num_tokens)
        return grad, None, None, None


class _UnpermuteRows(torch.autograd.Function):
    """out[t] = sum_e permuted[dst_map[t,e]] * probs[t,e]  (+ residual[t])."""

    @staticmethod
    def forward(ctx, permuted, dst_map, probs, num_tokens, padded, residual=None):
        out, _ = ops.unpermute_rows(permuted, dst_map, num_tokens, merging_probs=probs,
                                    residual=residual)
        ctx.with_residual = residual is not None
        ctx.with_probs = probs is not None
        ctx.padded = padded
        ctx.n_out = permuted.shape[0]
        if ctx.with_probs:
            ctx.save_for_backward(permuted, dst_map, probs)
        else:
            ctx.save_for_backward(dst_map)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = grad_out.contiguous()
        if ctx.with_probs:
            permuted, dst_map, probs = ctx.saved_tensors
            gp, gprobs = ops.unpermute_rows_bwd(grad_out, permuted, dst_map, probs,
                                                zero_fill=ctx.padded)
            return gp, None, gprobs, None, None, (grad_out if ctx.with_residual else None)
        (dst_map,) = ctx.saved_tensors
        gp, _ = ops.permute_rows(grad_out, dst_map, ctx.n_out, zero_fill=ctx.padded)
        return gp, None, None, None, None, (grad_out if ctx.with_residual else None)


def _as_int(n) -> int:
    return int(n.item()) if torch.is_tensor(n) else int(n)


def _plan_for(routing_map, num_out_tokens, drop_and_pad):
    num_tokens, num_experts = routing_map.shape
    if drop_and_pad and num_out_tokens is not None:
        n_out = _as_int(num_out_tokens)
        capacity = n_out // num_experts
        assert not routing_map.requires_grad
        return ops.permute_plan(routing_map, n_out, capacity=capacity)
    if num_out_tokens is None:
        # the output size depends on the data: one host read, as masked_select does in the reference
        n_out = int(routing_map.sum().item())
    else:
        n_out = _as_int(num_out_tokens)
    return ops.permute_plan(routing_map, n_out)


def permute(tokens, routing_map, num_out_tokens: Optional[int] = None, fused: bool = False,
            drop_and_pad: bool = False):
    """Group the tokens by expert (moe_utils.py:219-277).

    Returns (permuted [N,H], mapping).  With fused=False the mapping is `sorted_indices` (int64
    [N], bit-identical to the reference); with fused=True it is the token-major destination table
    (int32 [T,E]).  Either is only meant to be handed back to `unpermute`.
    """
    assert tokens.dim() == 2 and routing_map.dim() == 2
    plan = _plan_for(routing_map, num_out_tokens, drop_and_pad)
    permuted = _PermuteRows.apply(tokens.contiguous(), plan.dst_map, plan.n_out, plan.padded)
    if fused:
        return permuted, plan.dst_map
    mapping = plan.sorted_indices
    # remember the plan on the index tensor (without a back-reference) so that unpermute can
    # reuse it instead of rebuilding it from routing_map
    mapping._gmoe_plan = dataclasses.replace(plan, sorted_indices=None)
    return permuted, mapping


def unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, restore_shape: torch.Size,
              probs: torch.Tensor = None, routing_map: torch.Tensor = None, fused: bool = False,
              drop_and_pad: bool = False, residual: torch.Tensor = None):
    """Restore the token order, optionally weighting by probs (moe_utils.py:280-353).  `residual`
    (not in the reference's signature) is added to the restored rows in the same pass."""
    num_tokens, hidden = restore_shape
    if probs is not None:
        assert routing_map is not None, "Mask must be provided to permute the probs."
    plan = getattr(sorted_indices, "_gmoe_plan", None)
    if plan is None and sorted_indices.dtype == torch.int32 and sorted_indices.dim() == 2:
        plan = ops.PermutePlan(sorted_indices, None, None, None, None, sorted_indices.shape[0],
                               sorted_indices.shape[1], permuted_tokens.shape[0], padded=drop_and_pad)
    if plan is None and routing_map is not None:
        n_out = permuted_tokens.shape[0]
        cap = n_out // routing_map.shape[1] if drop_and_pad else 0
        plan = ops.permute_plan(routing_map, n_out, capacity=cap, want_sorted=False)
    if plan is None:
        # only the index list is known: scatter-add with fp32 atomics (not differentiable)
        assert not permuted_tokens.requires_grad, \
            "unpermute without routing_map is forward-only; pass routing_map"
        out = ops.scatter_add_rows(permuted_tokens.contiguous(), sorted_indices.contiguous(),
                                   num_tokens)
        return out if residual is None else out + residual
    assert plan.num_tokens == num_tokens
    if probs is not None:
        probs = probs.contiguous()
    if residual is not None:
        residual = residual.reshape(num_tokens, hidden).contiguous()
    return _UnpermuteRows.apply(permuted_tokens.contiguous(), plan.dst_map, probs, num_tokens,
                                plan.padded, residual)


class _SortChunks(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, split_sizes, sorted_idxs):
        out, row_map = ops.sort_chunks(inp, split_sizes, sorted_idxs)
        ctx.save_for_backward(row_map)
        return out

    @staticmethod
    def backward(ctx, grad):
        (row_map,) = ctx.saved_tensors
        return ops.scatter_rows_by_map(grad.contiguous(), row_map), None, None


def sort_chunks_by_idxs(input: torch.Tensor, split_sizes: torch.Tensor, sorted_idxs: torch.Tensor,
                        fused: bool = False):
    """Split `input` into chunks and concatenate them in `sorted_idxs` order (moe_utils.py:356-369).
    The split tables may live on the host or the device; no host synchronisation either way."""
    if input.numel() == 0:
        return input
    return _SortChunks.apply(input.contiguous(), split_sizes, sorted_idxs)


# ---------------------------------------------------------------------------------------------
# Router
# ---------------------------------------------------------------------------------------------

class _RouteTopK(torch.autograd.Function):
    """probs, routing_map, tokens_per_expert = route(logits); differentiable in logits."""

    @staticmethod
    def forward(ctx, logits, k, score_fn, pre_softmax, scaling, expert_bias, num_groups, group_topk,
                aux_scale=0.0, z_scale=0.0, want_stats=False):
        """aux_scale / z_scale: factors of the load-balancing and z-loss gradients that the backward
        adds to dlogits (times MoEAuxLossAutoScaler.main_loss_backward_scale), fused into the same
        kernel instead of separate softmax / logsumexp graphs.  stats = [sum_t scores | sum_t lse^2]."""
        probs, rmap, counts, stats, _ = ops.route_topk(
            logits, k, score_fn, pre_softmax, scaling, expert_bias, num_groups, group_topk,
            want_stats=want_stats)
        ctx.save_for_backward(logits, rmap, counts)
        ctx.cfg = (k, score_fn, pre_softmax, scaling, float(aux_scale), float(z_scale))
        if stats is None:
            stats = logits.new_zeros((0,), dtype=torch.float32)
        ctx.mark_non_differentiable(rmap, counts, stats)
        return probs, rmap, counts, stats

    @staticmethod
    def backward(ctx, dprobs, _dmap, _dcounts, _dstats):
        logits, rmap, counts = ctx.saved_tensors
        k, score_fn, pre_softmax, scaling, aux_scale, z_scale = ctx.cfg
        loss_scale = None
        if aux_scale != 0.0 or z_scale != 0.0:
            loss_scale = MoEAuxLossAutoScaler.main_loss_backward_scale
            if loss_scale is not None:
                loss_scale = loss_scale.detach().to(device=logits.device, dtype=torch.float32)
                loss_scale = loss_scale.reshape(-1)[:1].contiguous()
        dlogits = ops.route_topk_bwd(logits, k, score_fn, pre_softmax, scaling, rmap,
                                     dprobs.contiguous(), counts, aux_scale, z_scale, loss_scale)
        return (dlogits,) + (None,) * 10


def group_limited_topk(scores, topk, num_tokens, num_experts, num_groups, group_topk):
    """moe_utils.py:372-427: top-k restricted to the `group_topk` best expert groups, a group being
    scored by the sum of its top-(topk/group_topk) entries.  Returns (values, indices)."""
    assert scores.shape == (num_tokens, num_experts)
    _, _, _, _, idx = ops.route_topk(scores.contiguous(), topk, "softmax", False, None, None,
                                     num_groups, group_topk, want_topk_idx=True)
    idx = idx.long()
    return torch.gather(scores, 1, idx), idx


def topk_softmax_with_capacity(
    logits: torch.Tensor,
    topk: int,
    capacity_factor: Optional[float] = None,
    pad_to_capacity: bool = False,
    drop_policy: str = "probs",
    use_pre_softmax: bool = False,
    num_groups: Optional[int] = None,
    group_topk: Optional[int] = None,
    scaling_factor: Optional[float] = None,
    deterministic_mode: bool = False,
    score_function: str = "softmax",
    expert_bias: Optional[torch.Tensor] = None,
):
    """Top-k routing with optional capacity (moe_utils.py:430-544).

    Returns (probs [T,E], routing_map [T,E] bool, tokens_per_expert [E] int64 before dropping).
    """
    assert logits.dim() == 2, f"Expected 2D logits [num_tokens, num_experts], got {logits.dim()}."
    num_tokens, num_experts = logits.shape
    if score_function not in ("softmax", "sigmoid"):
        raise ValueError(f"Invalid score_function: {score_function}")
    if capacity_factor is not None and drop_policy not in ("probs", "position"):
        raise ValueError(f"Invalid drop_policy: {drop_policy}")
    if expert_bias is not None:
        expert_bias = expert_bias.detach().to(torch.float32).contiguous()
    probs, routing_map, tokens_per_expert, _ = _RouteTopK.apply(
        logits.contiguous(), topk, score_function, use_pre_softmax, scaling_factor, expert_bias,
        num_groups, group_topk)
    if capacity_factor is None:
        return probs, routing_map, tokens_per_expert
    final_probs, final_map = apply_expert_capacity(probs, routing_map, topk, capacity_factor,
                                                   pad_to_capacity, drop_policy)
    return final_probs, final_map, tokens_per_expert


class _CapacitySelect(torch.autograd.Function):
    """probs * kept with kept chosen by the HIP selection kernel; d probs = grad * kept."""

    @staticmethod
    def forward(ctx, probs, routing_map, capacity, by_position, pad):
        out_probs, kept = ops.capacity_select(probs.contiguous(), routing_map.contiguous(), capacity,
                                              by_position, pad)
        ctx.save_for_backward(kept)
        ctx.mark_non_differentiable(kept)
        return out_probs, kept

    @staticmethod
    def backward(ctx, grad_probs, _grad_kept):
        (kept,) = ctx.saved_tensors
        return grad_probs * kept, None, None, None, None


def apply_expert_capacity(probs, routing_map, topk, capacity_factor, pad_to_capacity=False,
                          drop_policy="probs"):
    """Keep at most `expert_capacity` tokens per expert (moe_utils.py:519-544): a per-column
    top-C along the token axis on the device, lowest token index first among equal keys."""
    num_tokens, num_experts = probs.shape
    if drop_policy not in ("probs", "position"):
        raise ValueError(f"Invalid drop_policy: {drop_policy}")
    expert_capacity = get_capacity(num_tokens * topk, num_experts, capacity_factor)
    expert_capacity = max(1, min(expert_capacity, num_tokens))
    return _CapacitySelect.apply(probs, routing_map, expert_capacity, drop_policy == "position",
                                 pad_to_capacity)


# ---------------------------------------------------------------------------------------------
# Bookkeeping (moe_utils.py:547-662); single process, so no reductions across ranks
# ---------------------------------------------------------------------------------------------

_MOE_LAYER_WISE_LOGGING_TRACKER = {}


def get_moe_layer_wise_logging_tracker():
    return _MOE_LAYER_WISE_LOGGING_TRACKER


def save_to_aux_losses_tracker(name: str, loss: torch.Tensor, layer_idx: int, num_layers: int,
                               reduce_group=None, avg_group=None):
    """moe_utils.py:547-574."""
    if layer_idx is None:
        return
    tracker = get_moe_layer_wise_logging_tracker()
    if name not in tracker:
        tracker[name] = {"values": torch.zeros(num_layers, device=loss.device)}
    tracker[name]["values"][layer_idx - 1] += loss.detach()
    tracker[name]["reduce_group"] = reduce_group
    tracker[name]["avg_group"] = avg_group


def clear_aux_losses_tracker():
    """moe_utils.py:577-583."""
    tracker = get_moe_layer_wise_logging_tracker()
    for name in tracker:
        tracker[name]["values"].zero_()
        tracker[name]["reduce_group"] = None
        tracker[name]["avg_group"] = None


def get_updated_expert_bias(tokens_per_expert, expert_bias, expert_bias_update_rate):
    """moe_utils.py:645-662 without the all-reduce over data-parallel ranks."""
    with torch.no_grad():
        average_tokens = tokens_per_expert.sum(dim=-1, keepdim=True) / tokens_per_expert.shape[-1]
        offset = average_tokens - tokens_per_expert
        return expert_bias + torch.sign(offset) * expert_bias_update_rate


def reduce_aux_losses_tracker_across_ranks():
    """moe_utils.py:586-601.  One process owns the whole layer here, so there is nothing to reduce;
    kept so that callers of the reference's name keep working."""
    return None


def track_moe_metrics(loss_scale, iteration, writer, wandb_writer=None, total_loss_dict=None,
                      per_layer_logging=False):
    """Log the tracked auxiliary losses and clear the tracker (moe_utils.py:604-642)."""
    reduce_aux_losses_tracker_across_ranks()
    tracker = get_moe_layer_wise_logging_tracker()
    if writer is not None:
        aux_losses = {k: v["values"].float() * loss_scale for k, v in tracker.items()}
        for name, loss_list in aux_losses.items():
            if total_loss_dict is not None:
                if name not in total_loss_dict:
                    total_loss_dict[name] = loss_list.mean()
                else:
                    total_loss_dict[name] += loss_list.mean()
            writer.add_scalar(name, loss_list.mean(), iteration)
            if per_layer_logging:
                for i, loss in enumerate(loss_list.tolist()):
                    writer.add_scalar(f"moe/{name}_layer_{i}", loss, iteration)
            if wandb_writer:
                wandb_writer.log({f"{name}": loss_list.mean()}, iteration)
                if per_layer_logging:
                    wandb_writer.log({f"moe/{name}_layer_{i}": loss
                                      for i, loss in enumerate(loss_list.tolist())}, iteration)
    clear_aux_losses_tracker()


def maybe_move_tensor_to_cpu(tensor, as_numpy=False, record_stream=False):
    """moe_utils.py:665-680."""
    if torch.is_tensor(tensor) and tensor.is_cuda:
        cpu_tensor = tensor.to(torch.device("cpu"), non_blocking=True)
        if as_numpy:
            cpu_tensor = cpu_tensor.numpy()
        if record_stream:
            tensor.record_stream(torch.cuda.current_stream())
        tensor = cpu_tensor
    return tensor
