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
# Losses.  The router's own loss terms never pass through here: TopKRouter takes their statistics
# and gradients from the routing kernels.  These are the reference's free functions for other
# callers, on the same device kernels.
# ---------------------------------------------------------------------------------------------

def _no_sequence_partition(group):
    if group is not None:
        raise NotImplementedError("sequence-partitioned aux loss needs collectives (single GPU build)")


class _SwitchLoss(torch.autograd.Function):
    """factor * sum_e tokens_per_expert[e] * sum_t probs[t,e]: one statistics launch, their
    fixed-order reduction and the bookkeeping launch forward, one broadcast launch backward; fp32
    sums whatever the dtype of `probs`."""

    @staticmethod
    def forward(ctx, probs, tokens_per_expert, factor):
        probs = probs.contiguous()
        T, E = probs.shape
        counts = tokens_per_expert.to(torch.int64).contiguous()
        stats = ops.score_stats(probs, 1, "identity")
        loss, _ = ops.router_bookkeeping(stats, counts, E, aux_factor=factor, want_aux=True)
        ctx.save_for_backward(probs, tokens_per_expert.to(torch.float32).contiguous())
        ctx.factor = factor
        return loss.to(probs.dtype)

    @staticmethod
    def backward(ctx, grad_loss):
        probs, weights = ctx.saved_tensors
        g = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        return ops.score_stats_bwd(probs, 1, "identity", weights, aux_scale=ctx.factor, grad_loss=g), None, None


def switch_load_balancing_loss_func(probs, tokens_per_expert, topk, moe_aux_loss_coeff,
                                    sequence_partition_group=None):
    """Switch-transformer load-balancing loss (moe_utils.py:14-59):
    E * coeff / (T^2 * topk) * <sum_t probs[t, :], tokens_per_expert>.  Differentiable in `probs`."""
    _no_sequence_partition(sequence_partition_group)
    T, E = probs.shape
    return _SwitchLoss.apply(probs, tokens_per_expert, E * moe_aux_loss_coeff / (T * T * topk))


class _ZLoss(torch.autograd.Function):
    """coeff / T * sum_t logsumexp(logits[t,:])^2 from the same statistics kernels."""

    @staticmethod
    def forward(ctx, logits, factor):
        logits = logits.contiguous()
        E = logits.shape[1]
        stats = ops.score_stats(logits, 1, "softmax")
        _, loss = ops.router_bookkeeping(stats, None, E, z_factor=factor, want_z=True)
        ctx.save_for_backward(logits)
        ctx.factor = factor
        return loss.to(logits.dtype)

    @staticmethod
    def backward(ctx, grad_loss):
        (logits,) = ctx.saved_tensors
        g = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        return ops.score_stats_bwd(logits, 1, "softmax", z_scale=ctx.factor, grad_loss=g), None


class _SeqAuxLoss(torch.autograd.Function):
    """coeff * mean_b sum_e (count[b,e] * E / (S k)) * mean_s score[s,b,e] of `x` [S*B, E], where
    the scores are x itself (score_fn "identity") or computed from x as logits inside the kernel.
    One statistics launch forward, one gradient launch backward."""

    @staticmethod
    def forward(ctx, x, routing_map, batch_size, seq_length, topk, coeff, score_fn):
        x = x.contiguous()
        loss, counts, _ = ops.seq_aux_loss(x, routing_map.contiguous(), batch_size, seq_length, topk,
                                           coeff, score_fn)
        ctx.save_for_backward(x, counts)
        ctx.cfg = (batch_size, seq_length, topk, coeff, score_fn)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        x, counts = ctx.saved_tensors
        batch_size, seq_length, topk, coeff, score_fn = ctx.cfg
        grad_loss = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        dx = ops.seq_aux_loss_bwd(x, counts, batch_size, seq_length, topk, coeff, score_fn, grad_loss)
        return dx, None, None, None, None, None, None


def sequence_load_balancing_loss_func(probs, routing_map, batch_size, seq_length, topk,
                                      moe_aux_loss_coeff, sequence_partition_group=None):
    """Per-sequence load-balancing loss (moe_utils.py:62-112); `probs` [S*B, E] are the routing
    scores, token (s, b) in row s*B + b.  Differentiable in `probs`."""
    _no_sequence_partition(sequence_partition_group)
    return _SeqAuxLoss.apply(probs, routing_map.bool(), batch_size, seq_length, topk,
                             moe_aux_loss_coeff, "identity")


def z_loss_func(logits, z_loss_coeff):
    """coeff * mean_t logsumexp(logits[t, :])^2 (moe_utils.py:115-127).  Differentiable in `logits`."""
    assert logits.dim() == 2
    return _ZLoss.apply(logits, z_loss_coeff / max(logits.shape[0], 1))


def sinkhorn(cost: torch.Tensor, tol: float = 0.0001):
    """Sinkhorn-normalised exp(cost) (moe_utils.py:130-144) in the dtype of `cost`: the whole
    iteration is one device kernel computing in fp32, so no convergence test ever reaches the host.
    The reference loops until the error is below `tol` however long that takes; here the loop ends
    after `ops.SINKHORN_MAX_ITERS` iterations at the latest (`ops.sinkhorn(..., want_iters=True)`
    returns the count)."""
    assert cost.dim() == 2
    return ops.sinkhorn(cost.contiguous(), tol).to(cost.dtype)


def get_capacity(num_tokens: int, num_experts: int, capacity_factor: float, min_capacity=None):
    """Rows an expert may take: ceil(tokens / experts * factor), at least min_capacity
    (moe_utils.py:147-163)."""
    capacity = math.ceil(num_tokens / num_experts * capacity_factor)
    return capacity if min_capacity is None else max(capacity, min_capacity)


class MoEAuxLossAutoScaler(torch.autograd.Function):
    """Attaches an auxiliary loss to an activation (moe_utils.py:166-216): the forward returns the
    activation untouched; the backward hands the activation's gradient through and gives the loss
    the gradient `main_loss_backward_scale` (1 until set_loss_scale is called), so the loss trains
    the router without being added to the main loss.  TopKRouter's own load-balancing and z losses
    do not go through here: their gradients come out of the routing backward kernel, which reads the
    same scale from the device."""

    main_loss_backward_scale: torch.Tensor = None

    @staticmethod
    def _scale_on(device) -> torch.Tensor:
        cls = MoEAuxLossAutoScaler
        if cls.main_loss_backward_scale is None:
            cls.main_loss_backward_scale = torch.ones((), device=device)
        return cls.main_loss_backward_scale

    @staticmethod
    def forward(ctx, output: torch.Tensor, aux_loss: torch.Tensor):
        ctx.aux_meta = (aux_loss.shape, aux_loss.dtype, aux_loss.device)
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        shape, dtype, device = ctx.aux_meta
        scale = MoEAuxLossAutoScaler._scale_on(device)
        return grad_output, scale.to(device=device, dtype=dtype).expand(shape)

    @staticmethod
    def set_loss_scale(scale: torch.Tensor):
        cls = MoEAuxLossAutoScaler
        if cls.main_loss_backward_scale is None:
            cls.main_loss_backward_scale = scale
        else:
            cls.main_loss_backward_scale.copy_(scale)


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
    """out[t] = sum_e permuted[dst_map[t,e]] * probs[t,e]  (+ addend[t]) (+ residual[t])."""

    @staticmethod
    def forward(ctx, permuted, dst_map, probs, num_tokens, padded, residual=None, addend=None):
        out, _ = ops.unpermute_rows(permuted, dst_map, num_tokens, merging_probs=probs,
                                    residual=residual, addend=addend)
        ctx.with_residual = residual is not None
        ctx.with_addend = addend is not None
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
            return (gp, None, gprobs, None, None, (grad_out if ctx.with_residual else None),
                    (grad_out if ctx.with_addend else None))
        (dst_map,) = ctx.saved_tensors
        gp, _ = ops.permute_rows(grad_out, dst_map, ctx.n_out, zero_fill=ctx.padded)
        return (gp, None, None, None, None, (grad_out if ctx.with_residual else None),
                (grad_out if ctx.with_addend else None))


def scale_rows(x: torch.Tensor, row_scale: torch.Tensor) -> torch.Tensor:
    """x [T,H] * row_scale [T] (or [T,1]) with one rounding, differentiable in both: the combine
    kernels with the identity map (their backward yields the per-row dot products the scale's
    gradient needs)."""
    T = x.shape[0]
    return _UnpermuteRows.apply(x.contiguous(), ops.identity_map(T, x.device),
                                row_scale.reshape(T, 1).contiguous(), T, False)


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
                aux_scale=0.0, z_scale=0.0, want_stats=False, selection_scores=None):
        """aux_scale / z_scale: factors of the load-balancing and z-loss gradients that the backward
        adds to dlogits (times MoEAuxLossAutoScaler.main_loss_backward_scale), fused into the same
        kernel instead of separate softmax / logsumexp graphs.  stats = [sum_t scores | sum_t lse^2].
        selection_scores [T,E] fp32 (no gradient): ranked by the top-k instead of the scores."""
        probs, rmap, counts, stats, _ = ops.route_topk(
            logits, k, score_fn, pre_softmax, scaling, expert_bias, num_groups, group_topk,
            want_stats=want_stats, selection_scores=selection_scores)
        ctx.save_for_backward(logits, rmap, counts)
        ctx.cfg = (k, score_fn, pre_softmax, scaling, float(aux_scale), float(z_scale))
        if stats is None:
            stats = logits.new_zeros((0,), dtype=torch.float32)
        ctx.mark_non_differentiable(rmap, counts, stats)
        # without this autograd fills a zero gradient for each of the three (three fill launches)
        ctx.set_materialize_grads(False)
        return probs, rmap, counts, stats

    @staticmethod
    def backward(ctx, dprobs, _dmap, _dcounts, _dstats):
        logits, rmap, counts = ctx.saved_tensors
        k, score_fn, pre_softmax, scaling, aux_scale, z_scale = ctx.cfg
        if dprobs is None:
            if aux_scale == 0.0 and z_scale == 0.0:
                return (None,) * 12
            dprobs = torch.zeros_like(logits)
        loss_scale = None
        if aux_scale != 0.0 or z_scale != 0.0:
            loss_scale = MoEAuxLossAutoScaler.main_loss_backward_scale
            if loss_scale is not None:
                loss_scale = loss_scale.detach().to(device=logits.device, dtype=torch.float32)
                loss_scale = loss_scale.reshape(-1)[:1].contiguous()
        dlogits = ops.route_topk_bwd(logits, k, score_fn, pre_softmax, scaling, rmap,
                                     dprobs.contiguous(), counts, aux_scale, z_scale, loss_scale)
        return (dlogits,) + (None,) * 11


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
        ctx.set_materialize_grads(False)
        return out_probs, kept

    @staticmethod
    def backward(ctx, grad_probs, _grad_kept):
        (kept,) = ctx.saved_tensors
        return (None if grad_probs is None else grad_probs * kept), None, None, None, None


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
# Bookkeeping (moe_utils.py:547-680); one process owns the whole layer, so nothing is reduced
# across ranks
# ---------------------------------------------------------------------------------------------

_MOE_LAYER_WISE_LOGGING_TRACKER = {}


def get_moe_layer_wise_logging_tracker():
    return _MOE_LAYER_WISE_LOGGING_TRACKER


def aux_losses_tracker_slot(name: str, layer_idx: int, num_layers: int, device):
    """One-element fp32 view of `tracker[name]["values"][layer_idx - 1]` (created on first use), for
    kernels that add a loss value to it on the device; None when layer_idx is None."""
    if layer_idx is None:
        return None
    tracker = get_moe_layer_wise_logging_tracker()
    entry = tracker.setdefault(name, {})
    if "values" not in entry:
        entry["values"] = torch.zeros(num_layers, device=device)
    entry.setdefault("reduce_group", None)
    entry.setdefault("avg_group", None)
    return entry["values"].narrow(0, layer_idx - 1, 1)


def save_to_aux_losses_tracker(name: str, loss: torch.Tensor, layer_idx: int, num_layers: int,
                               reduce_group=None, avg_group=None):
    """Add `loss` to the per-layer logging tracker (moe_utils.py:547-574)."""
    slot = aux_losses_tracker_slot(name, layer_idx, num_layers, loss.device)
    if slot is None:
        return
    slot.add_(loss.detach().to(slot.dtype).reshape(1))
    entry = get_moe_layer_wise_logging_tracker()[name]
    entry["reduce_group"], entry["avg_group"] = reduce_group, avg_group


def clear_aux_losses_tracker():
    """Zero every tracked value (moe_utils.py:577-583)."""
    for entry in get_moe_layer_wise_logging_tracker().values():
        entry["values"].zero_()
        entry["reduce_group"] = entry["avg_group"] = None


def get_updated_expert_bias(tokens_per_expert, expert_bias, expert_bias_update_rate):
    """Aux-loss-free balancing step (moe_utils.py:645-662, without its all-reduce over
    data-parallel ranks): experts below the mean load gain `rate`, experts above lose it.  One
    kernel over all [layers, E] rows."""
    with torch.no_grad():
        return ops.expert_bias_update(tokens_per_expert, expert_bias, expert_bias_update_rate)


def reduce_aux_losses_tracker_across_ranks():
    """moe_utils.py:586-601.  One process owns the whole layer here, so there is nothing to reduce;
    kept so that callers of the reference's name keep working."""
    return None


def track_moe_metrics(loss_scale, iteration, writer, wandb_writer=None, total_loss_dict=None,
                      per_layer_logging=False):
    """Log the tracked auxiliary losses and clear the tracker (moe_utils.py:604-642).  All values
    of all losses come to the host in one transfer."""
    reduce_aux_losses_tracker_across_ranks()
    tracker = get_moe_layer_wise_logging_tracker()
    if writer is not None and tracker:
        names = list(tracker)
        scaled = torch.stack([tracker[n]["values"].float() for n in names]) * loss_scale
        if total_loss_dict is not None:
            means_dev = scaled.mean(dim=1)
            for i, n in enumerate(names):
                total_loss_dict[n] = means_dev[i] if n not in total_loss_dict \
                    else total_loss_dict[n] + means_dev[i]
        host = scaled.cpu()
        for n, row in zip(names, host):
            mean = row.mean()
            writer.add_scalar(n, mean, iteration)
            per_layer = {f"moe/{n}_layer_{i}": v for i, v in enumerate(row.tolist())} \
                if per_layer_logging else {}
            for key, v in per_layer.items():
                writer.add_scalar(key, v, iteration)
            if wandb_writer:
                wandb_writer.log({f"{n}": mean}, iteration)
                if per_layer:
                    wandb_writer.log(per_layer, iteration)
    clear_aux_losses_tracker()


def maybe_move_tensor_to_cpu(tensor, as_numpy=False, record_stream=False):
    """Device tensor -> host copy started on the current stream (moe_utils.py:665-680); anything else
    is returned as it is.  The copy lands in pinned memory, so it really is asynchronous: the
    caller synchronises the stream before reading."""
    if not (torch.is_tensor(tensor) and tensor.is_cuda):
        return tensor
    host = torch.empty(tensor.shape, dtype=tensor.dtype, device="cpu", pin_memory=True)
    host.copy_(tensor, non_blocking=True)
    if record_stream:
        tensor.record_stream(torch.cuda.current_stream(tensor.device))
    return host.numpy() if as_numpy else host
