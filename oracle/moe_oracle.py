"""CPU restatement (torch, fp32/fp64) of the reference's MoE expert-layer path.

TEST INFRASTRUCTURE ONLY: used by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py as the checker / timed CPU baseline.  The product
package never imports it.

Every function cites the reference file:line it follows (paths relative to the
reference tree, `galvatron/core/runtime/...`).  The reference composes torch
library calls; this file composes the same calls on the CPU, with two
deliberate, documented differences (the code is device-agnostic torch: the tests run it on the
CPU, and on GPU tensors, where torch's own kernels evaluate it, for the full benchmark sizes):

* top-k ties.  The reference calls `torch.topk`, whose tie-break is an
  implementation detail.  The oracle fixes the rule "among equal scores the
  lowest expert index wins" (a stable descending sort).  On tie-free inputs the
  two agree (checked in tests/test_oracle.py).
* `grouped_gemm.ops.gmm` is a third-party CUDA extension
  (fanshiqing/grouped_gemm v1.1.4) that is not in the reference tree.  Its
  published contract -- out[rows of group e] = a[rows of group e] @ b[e] -- is
  restated as a per-expert matmul loop, which is also what the reference's own
  SequentialMLP does (moe/mlp.py:188-211).  PARITY UNPINNED against the
  extension's own bf16 accumulation order; pinned against the mathematics
  (dense matmul special cases, fp64 closed form).

Pinning status of each function (see tests/test_oracle.py):
  topk_tie_low_index ............ brute force + torch.topk on tie-free rows
  topk_softmax_with_capacity .... brute force, invariants, HF-Mixtral identity
  switch_load_balancing_loss .... uniform-routing closed form (== coeff)
  sequence_load_balancing_loss .. per-sequence pure-Python loop over (s, b, e) with explicit token
                                  index s*B+b, uniform-routing closed form (== coeff), equality with
                                  the switch loss when the batch is one sequence
  sinkhorn / sinkhorn_routing ... float64 numpy loop, column sums == 1/E and row sums ~ 1/T at
                                  convergence, at least one iteration; routing: k True per row,
                                  gates == activation on the selected experts
  get_updated_expert_bias ....... hand-computed example, sign(0) == 0, mean load unchanged by shift
  z_loss ........................ closed form on constant rows (log(E)^2)
  permute / sorted_indices ...... np.nonzero(map.T) closed form, invariants
  unpermute ..................... index_add_, round-trip identity, linearity
  row_id_map_te ................. inverse-permutation invariant
  unpermute_bwd_with_probs ...... torch autograd of the forward
  gmm ........................... E=1 dense matmul, fp64 closed form, empty groups
  swiglu / swiglu_back .......... autograd of F.silu(y1)*y2
  swiglu_fp8_input_store ........ the cast is the reference's own call (torch's float8_e4m3fn
                                  conversion); checked on every bf16 bit pattern against a numpy
                                  restatement of round-to-nearest-even on 3 mantissa bits with the
                                  NaN code beyond the range; backward == swiglu_back on the cast
  sequential_mlp ................ without bias == grouped_mlp on the transposed weights; with bias:
                                  token-by-token fp64 loop, torch.nn.functional.linear with bias
                                  (E = 1), a zero bias changes nothing, the returned bias rows are
                                  fc2_b[expert of the row]
  allgather_combine ............. per-token fp64 loop over the selected experts; a bias that is the
                                  same row b everywhere combines to b * sum of the token's gates
  shared_expert_mlp ............. token-by-token fp64 loop, transformers' LlamaMLP (SiLU-gated MLP)
  grouped_mlp / moe_layer ....... transformers' MixtralSparseMoeBlock (the model the reference's
                                  own correctness test compares with): forward and the gradients
                                  of x, gate weight, w1, w2, both dispatcher forms; Mixtral expert
                                  formula from Hugging Face keys (tests/test_checkpoint.py)
  rms_norm ...................... torch.nn.functional.rms_norm, transformers' MixtralRMSNorm on
                                  fp32 input, closed form on constant-magnitude rows, scale
                                  invariance (flash-attn is not importable here: restated
                                  from its published formula)
  quantize_fp8_block ............ not in the reference at all (defined here); round trip within
                                  half an fp8 step of the tile maximum
  quantize_fp8_rows ............. not in the reference at all (defined here); brute force over the
                                  exponents (the chosen one is the smallest that keeps the block
                                  within +-448), powers of two and exactly representable blocks
                                  round-trip without error, round trip within half an fp8 step
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------
# Pre-router normalisation
# ----------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """models/moe_modules.py:24-30 applies `GalvatronNorm` = flash_attn.ops.rms_norm.RMSNorm
    (transformer/norm.py:20-26; third-party flash-attn >= 2.0.8, requirements.txt:5) before the
    router.  Its published formula: y = x / sqrt(mean(x^2, -1) + eps) * weight, evaluated in fp32
    and rounded once to the dtype of x; the residual handed to the MLP is x itself."""
    xf = x.float()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * rstd * weight.float()).to(x.dtype)


# ----------------------------------------------------------------------------
# Router
# ----------------------------------------------------------------------------

def gate_logits(x: torch.Tensor, w_r: torch.Tensor, router_dtype: Optional[str] = None) -> torch.Tensor:
    """moe/router.py:49-68 (`Router.gating`): logits = linear(x.to(rd), W_r.to(rd))."""
    rd = x.dtype
    if router_dtype == "fp32":
        rd = torch.float32
    elif router_dtype == "fp64":
        rd = torch.float64
    return F.linear(x.to(rd), w_r.to(rd))


def topk_tie_low_index(scores: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """`torch.topk(scores, k, dim=1)` (moe/moe_utils.py:485) with the tie rule fixed:
    values descending, equal values ordered by ascending expert index; NaN sorts first
    (as in torch)."""
    vals, idx = torch.sort(scores, dim=1, descending=True, stable=True)
    return vals[:, :k].contiguous(), idx[:, :k].contiguous()


def get_capacity(num_tokens: int, num_experts: int, capacity_factor: float, min_capacity=None) -> int:
    """moe/moe_utils.py:147-163."""
    capacity = math.ceil((num_tokens / num_experts) * capacity_factor)
    if min_capacity is not None and capacity < min_capacity:
        capacity = min_capacity
    return capacity


def group_limited_topk(scores, topk, num_tokens, num_experts, num_groups, group_topk):
    """moe/moe_utils.py:372-427.  Group score = sum of the top-(topk/group_topk) scores in the
    group; the best `group_topk` groups survive (ties: lowest group index); others -> -inf."""
    group_scores = (
        topk_tie_low_index(scores.view(num_tokens * num_groups, -1), topk // group_topk)[0]
        .view(num_tokens, num_groups, -1)
        .sum(dim=-1)
    )
    group_idx = topk_tie_low_index(group_scores, group_topk)[1]
    group_mask = torch.zeros_like(group_scores)
    group_mask.scatter_(1, group_idx, 1)
    score_mask = (
        group_mask.unsqueeze(-1)
        .expand(num_tokens, num_groups, num_experts // num_groups)
        .reshape(num_tokens, -1)
    )
    masked_scores = scores.masked_fill(~score_mask.bool(), float("-inf"))
    return topk_tie_low_index(masked_scores, topk)


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
    return_topk: bool = False,
):
    """moe/moe_utils.py:430-544.  Returns (probs[T,E], routing_map[T,E] bool, tokens_per_expert[E])."""
    assert logits.dim() == 2
    num_tokens, num_experts = logits.shape

    def compute_topk(scores, topk, num_groups=None, group_topk=None):
        if group_topk:
            return group_limited_topk(scores, topk, num_tokens, num_experts, num_groups, group_topk)
        return topk_tie_low_index(scores, topk)

    if score_function == "softmax":
        if use_pre_softmax:
            scores = torch.softmax(logits, dim=-1, dtype=torch.float32).type_as(logits)
            probs, top_indices = compute_topk(scores, topk, num_groups, group_topk)
        else:
            scores, top_indices = compute_topk(logits, topk, num_groups, group_topk)
            probs = torch.softmax(scores, dim=-1, dtype=torch.float32).type_as(logits)
    elif score_function == "sigmoid":
        scores = torch.sigmoid(logits)
        if expert_bias is not None:
            scores_for_routing = scores + expert_bias
            _, top_indices = compute_topk(scores_for_routing, topk, num_groups, group_topk)
            scores = torch.gather(scores, dim=1, index=top_indices).type_as(logits)
        else:
            scores, top_indices = compute_topk(scores, topk, num_groups, group_topk)
        probs = scores / (scores.sum(dim=-1, keepdim=True) + 1e-20) if topk > 1 else scores
    else:
        raise ValueError(f"Invalid score_function: {score_function}")

    if scaling_factor:
        probs = probs * scaling_factor

    topk_masked_gates = torch.zeros_like(logits).scatter(1, top_indices, probs)
    topk_map = torch.zeros_like(logits).int().scatter(1, top_indices, 1).bool()
    tokens_per_expert = topk_map.sum(dim=0)

    if capacity_factor is None:
        out = (topk_masked_gates, topk_map, tokens_per_expert)
    else:
        expert_capacity = get_capacity(num_tokens * topk, num_experts, capacity_factor)
        if drop_policy == "probs":
            # torch.topk(..., dim=0, sorted=False) restated with the fixed tie rule
            # (lowest token index wins among equal gate values).
            _, capacity_indices = topk_tie_low_index(topk_masked_gates.T.contiguous(), expert_capacity)
            capacity_indices = capacity_indices.T
        elif drop_policy == "position":
            _, capacity_indices = topk_tie_low_index(topk_map.int().T.contiguous(), expert_capacity)
            capacity_indices = capacity_indices.T
        else:
            raise ValueError(f"Invalid drop_policy: {drop_policy}")
        capacity_mask = torch.zeros_like(logits).scatter(0, capacity_indices, 1).bool()
        if pad_to_capacity:
            final_map = capacity_mask
            final_probs = topk_masked_gates * final_map
        else:
            final_map = torch.logical_and(topk_map, capacity_mask)
            final_probs = topk_masked_gates * final_map
        out = (final_probs, final_map, tokens_per_expert)
    if return_topk:
        return out + (top_indices,)
    return out


def probs_from_map(logits: torch.Tensor, routing_map: torch.Tensor) -> torch.Tensor:
    """Gates of the default branch for a GIVEN selection: fp32 softmax over the selected logits,
    cast to logits.dtype, zero elsewhere.  Equals moe/moe_utils.py:494-495 + 512 whenever
    `routing_map` is the top-k set (softmax is permutation invariant).  Differentiable in logits;
    used to compare floating-point results while holding the integer routing fixed."""
    masked = logits.float().masked_fill(~routing_map, float("-inf"))
    return torch.softmax(masked, dim=-1).to(logits.dtype)


def switch_load_balancing_loss(probs, tokens_per_expert, topk, coeff):
    """moe/moe_utils.py:14-59 (no sequence partition group)."""
    num_tokens, num_experts = probs.shape
    aggregated = probs.sum(dim=0)
    return torch.sum(aggregated * tokens_per_expert) * (
        num_experts * coeff / (num_tokens * num_tokens * topk)
    )


def sequence_load_balancing_loss(probs, routing_map, batch_size, seq_length, topk, coeff):
    """moe/moe_utils.py:62-112 (no sequence partition group)."""
    num_experts = probs.shape[1]
    p = probs.view(seq_length, batch_size, -1)
    m = routing_map.view(seq_length, batch_size, -1)
    cost_coeff = m.sum(dim=0, dtype=torch.float).div_(seq_length * topk / num_experts)
    return (cost_coeff * p.mean(dim=0)).sum(dim=1).mean() * coeff


def z_loss(logits, coeff):
    """moe/moe_utils.py:115-127."""
    return torch.mean(torch.square(torch.logsumexp(logits, dim=-1))) * coeff


def sinkhorn(cost: torch.Tensor, tol: float = 0.0001):
    """moe/moe_utils.py:130-144."""
    cost = torch.exp(cost)
    d0 = torch.ones(cost.size(0), dtype=cost.dtype, device=cost.device)
    d1 = torch.ones(cost.size(1), dtype=cost.dtype, device=cost.device)
    eps = 0.00000001
    error = 1e9
    d1_old = d1
    while error > tol:
        d0 = (1 / d0.size(0)) * 1 / (torch.sum(d1 * cost, 1) + eps)
        d1 = (1 / d1.size(0)) * 1 / (torch.sum(d0.unsqueeze(1) * cost, 0) + eps)
        error = torch.mean(torch.abs(d1_old - d1))
        d1_old = d1
    return d1 * cost * d0.unsqueeze(1)


def sinkhorn_routing(logits: torch.Tensor, topk: int, training: bool = True):
    """`TopKRouter.sinkhorn_load_balancing` (moe/router.py:140-171): in training the experts are the
    top-k of sinkhorn(float(logits)) (no gradient), otherwise of the activated logits; the scores
    are activation(logits) * map with activation = sigmoid (k == 1) or fp32 softmax cast back.
    Ties go to the lowest expert index.  Returns (scores [T,E], routing_map [T,E] bool)."""
    def activation(lg):
        if topk == 1:
            return torch.sigmoid(lg)
        return torch.softmax(lg, dim=-1, dtype=torch.float32).type_as(lg)

    if training:
        with torch.no_grad():
            norm_logits = sinkhorn(logits.to(dtype=torch.float32))
            _, indices = topk_tie_low_index(norm_logits, topk)
        act = activation(logits)
    else:
        act = activation(logits)
        _, indices = topk_tie_low_index(act.detach(), topk)
    rmap = torch.zeros_like(act).int().scatter(1, indices, 1).bool()
    return act * rmap, rmap


def get_updated_expert_bias(tokens_per_expert, expert_bias, expert_bias_update_rate):
    """moe/moe_utils.py:645-662 without the all-reduce over data-parallel ranks."""
    average_tokens = tokens_per_expert.sum(dim=-1, keepdim=True) / tokens_per_expert.shape[-1]
    offset = average_tokens - tokens_per_expert
    return expert_bias + torch.sign(offset) * expert_bias_update_rate


def router_forward(
    x: torch.Tensor,
    w_r: torch.Tensor,
    topk: int,
    router_dtype: Optional[str] = None,
    load_balancing_type: str = "none",
    aux_loss_coeff: float = 0.0,
    z_loss_coeff: Optional[float] = None,
    seq_shape: Optional[Tuple[int, int]] = None,
    **topk_kwargs,
):
    """moe/router.py:371-438 (`TopKRouter.forward` = gating + routing), training mode.
    `seq_shape` = (seq_length, batch_size) for the sequence-level loss.

    Returns (probs, routing_map, aux_total) where aux_total is the sum of the
    auxiliary losses whose gradient the reference injects through
    MoEAuxLossAutoScaler (moe/moe_utils.py:166-216) with backward scale 1.0;
    adding `aux_total` to the main loss reproduces those gradients exactly.
    """
    logits = gate_logits(x, w_r, router_dtype)
    logits = logits.view(-1, w_r.shape[0])
    aux_total = logits.new_zeros((), dtype=torch.float32)
    if z_loss_coeff is not None:
        aux_total = aux_total + z_loss(logits, z_loss_coeff).float()
    probs, routing_map, tokens_per_expert = topk_softmax_with_capacity(logits, topk, **topk_kwargs)
    if load_balancing_type == "aux_loss" and aux_loss_coeff != 0:
        score_function = topk_kwargs.get("score_function", "softmax")
        if score_function == "softmax":
            scores = torch.softmax(logits, dim=-1, dtype=torch.float32)  # router.py:182-183
        else:
            scores = torch.sigmoid(logits)
            scores = scores / (scores.sum(dim=-1, keepdim=True) + 1e-20) if topk > 1 else scores
        aux_total = aux_total + switch_load_balancing_loss(
            scores, tokens_per_expert, topk, aux_loss_coeff
        ).float()
    elif load_balancing_type == "seq_aux_loss" and aux_loss_coeff != 0:
        # moe/router.py:233-276: scores as above, the FINAL routing map, token (s, b) in row s*B+b
        score_function = topk_kwargs.get("score_function", "softmax")
        if score_function == "softmax":
            scores = torch.softmax(logits, dim=-1, dtype=torch.float32)
        else:
            scores = torch.sigmoid(logits)
            scores = scores / (scores.sum(dim=-1, keepdim=True) + 1e-20) if topk > 1 else scores
        assert seq_shape is not None, "seq_aux_loss needs (seq_length, batch_size)"
        seq_length, batch_size = seq_shape
        aux_total = aux_total + sequence_load_balancing_loss(
            scores, routing_map, batch_size, seq_length, topk, aux_loss_coeff).float()
    elif load_balancing_type not in ("none", "aux_loss", "seq_aux_loss"):
        raise ValueError(load_balancing_type)
    return probs, routing_map, aux_total


# ----------------------------------------------------------------------------
# Permute / unpermute
# ----------------------------------------------------------------------------

def permute(tokens, routing_map, num_out_tokens=None, drop_and_pad: bool = False):
    """moe/moe_utils.py:219-277, unfused branch.  Returns (permuted[N,H], sorted_indices[N] int64)."""
    num_tokens, hidden = tokens.shape
    num_experts = routing_map.shape[1]
    if drop_and_pad and num_out_tokens is not None:
        capacity = num_out_tokens // num_experts
        rm = routing_map.to(dtype=torch.int8).T.contiguous()
        sorted_indices = rm.argsort(dim=-1, descending=True, stable=True)[:, :capacity].contiguous()
        sorted_indices = sorted_indices.view(-1)
    else:
        rm = routing_map.bool().T.contiguous()
        token_indices = torch.arange(num_tokens, device=routing_map.device).unsqueeze(0).expand(num_experts, -1)
        sorted_indices = token_indices.masked_select(rm)
    return tokens.index_select(0, sorted_indices), sorted_indices


def permuted_probs(probs, routing_map):
    """moe/token_dispatcher.py:233-235 / moe_utils.py:339."""
    return probs.T.contiguous().masked_select(routing_map.T.contiguous())


def unpermute(permuted_tokens, sorted_indices, restore_shape, probs=None, routing_map=None,
              drop_and_pad: bool = False, accumulate_dtype=None):
    """moe/moe_utils.py:280-353, unfused branch.

    `accumulate_dtype=torch.float32` gives the fp32-accumulated variant (the semantics of the
    reference's fused kernel, moe/fused_kernels.py:226-249); None follows the unfused code
    literally (product and scatter_add_ in the promoted dtype).
    """
    _, hidden = restore_shape
    input_dtype = permuted_tokens.dtype
    if accumulate_dtype is not None:
        permuted_tokens = permuted_tokens.to(accumulate_dtype)
    if probs is not None:
        assert routing_map is not None
        if drop_and_pad:
            num_experts = routing_map.size(1)
            capacity = sorted_indices.size(0) // num_experts
            num_unpermuted = probs.size(0)
            probs_T_1D = probs.T.contiguous().view(-1)
            indices_dim0 = torch.arange(num_experts, device=routing_map.device).unsqueeze(-1)
            indices_dim1 = sorted_indices.view(num_experts, capacity)
            indices_1D = (indices_dim0 * num_unpermuted + indices_dim1).view(-1)
            pp = probs_T_1D.index_select(0, indices_1D)
        else:
            pp = permuted_probs(probs, routing_map)
        if accumulate_dtype is not None:
            pp = pp.to(accumulate_dtype)
        permuted_tokens = permuted_tokens * pp.unsqueeze(-1)
    out = torch.zeros(restore_shape, dtype=permuted_tokens.dtype, device=permuted_tokens.device)
    out.scatter_add_(0, sorted_indices.unsqueeze(1).expand(-1, hidden), permuted_tokens)
    return out.to(dtype=input_dtype)


def sort_chunks_by_idxs(inp, split_sizes, sorted_idxs):
    """moe/moe_utils.py:356-369, unfused branch."""
    chunks = torch.split(inp, split_sizes.tolist(), dim=0)
    return torch.cat([chunks[i] for i in sorted_idxs.tolist()], dim=0)


def row_id_map_te(routing_map: torch.Tensor) -> torch.Tensor:
    """Semantics of `triton_make_row_id_map` (moe/fused_kernels.py:514-605): an int64 [E,T]
    table whose entry (e,t) is the destination row of token t in expert e's block of the
    expert-major permuted tensor, or -1 when token t is not routed to e."""
    rm = routing_map.bool().T.contiguous()  # [E,T]
    flat = rm.reshape(-1)
    ranks = torch.cumsum(flat.to(torch.int64), 0) - 1
    out = torch.where(flat, ranks, torch.full_like(ranks, -1))
    return out.view(rm.shape)


def unpermute_fused(inp, row_id_map, merging_probs=None):
    """`_unpermute_kernel` (moe/fused_kernels.py:199-264): per token, fp32 accumulation over the
    experts (ascending) of inp[row_id_map[e,t]] * merging_probs[t,e]; result cast to inp.dtype."""
    E, T = row_id_map.shape
    acc = torch.zeros(T, inp.shape[1], dtype=torch.float32, device=inp.device)
    for e in range(E):
        rows = row_id_map[e]
        sel = rows >= 0
        v = inp[rows[sel]].float()
        if merging_probs is not None:
            v = v * merging_probs[sel, e].float().unsqueeze(-1)
        acc[sel] += v
    return acc.to(inp.dtype)


def unpermute_bwd_with_probs(grad_out, row_id_map, fwd_input, merging_probs):
    """`_unpermute_bwd_with_merging_probs_kernel` (moe/fused_kernels.py:319-396):
    dInp[row] = (dOut[t] * p[t,e]).to(dtype); dProbs[t,e] = sum_h fwd_input[row,h] * dOut[t,h]
    (fp32), zero where the token is not routed to e."""
    E, T = row_id_map.shape
    n_out = fwd_input.shape[0]
    act_grad = torch.zeros(n_out, grad_out.shape[1], dtype=grad_out.dtype, device=grad_out.device)
    probs_grad = torch.zeros(T, E, dtype=merging_probs.dtype, device=grad_out.device)
    for e in range(E):
        rows = row_id_map[e]
        sel = rows >= 0
        g = grad_out[sel].float()
        act_grad[rows[sel]] = (g * merging_probs[sel, e].float().unsqueeze(-1)).to(grad_out.dtype)
        probs_grad[sel, e] = (fwd_input[rows[sel]].float() * g).sum(-1).to(merging_probs.dtype)
    return act_grad, probs_grad


# ----------------------------------------------------------------------------
# Experts
# ----------------------------------------------------------------------------

def gmm(a, b, batch_sizes, trans_b: bool = False, compute_dtype=torch.float32):
    """Contract of `grouped_gemm.ops.gmm` (call sites moe/mlp.py:106-112): rows of `a` are
    partitioned into consecutive groups of batch_sizes[e] rows; group e is multiplied by b[e]
    (or b[e].T if trans_b).  Computed in `compute_dtype`, returned in a.dtype.  Differentiable."""
    outs = []
    start = 0
    for e, n in enumerate(batch_sizes.tolist()):
        be = b[e].to(compute_dtype)
        if trans_b:
            be = be.t()
        outs.append(a[start:start + n].to(compute_dtype) @ be)
        start += n
    assert start == a.shape[0]
    return torch.cat(outs, dim=0).to(a.dtype)


def swiglu(y):
    """transformer/fused_kernels.py:142-145 and the `glu` closure at moe/mlp.py:52-57."""
    y1, y2 = torch.chunk(y, 2, -1)
    return F.silu(y1) * y2


def swiglu_back(g, y):
    """transformer/fused_kernels.py:157-162."""
    y1, y2 = torch.chunk(y, 2, -1)
    s = torch.sigmoid(y1)
    return torch.cat((g * s * (1 + y1 * (1 - s)) * y2, g * F.silu(y1)), -1)


class SwiGLUFp8InputStore(torch.autograd.Function):
    """`SwiGLUFunction` with fp8_input_store=True (transformer/fused_kernels.py:190-204): the
    forward is swiglu(input); the backward sees input.to(float8_e4m3fn).to(input.dtype)."""

    @staticmethod
    def forward(ctx, y):
        ctx.save_for_backward(y.to(torch.float8_e4m3fn))
        ctx.ori_dtype = y.dtype
        return swiglu(y)

    @staticmethod
    def backward(ctx, g):
        (y8,) = ctx.saved_tensors
        return swiglu_back(g, y8.to(ctx.ori_dtype))


def swiglu_fp8_input_store(y):
    return SwiGLUFp8InputStore.apply(y)


def grouped_mlp(x_perm, w1, w2, tokens_per_expert, compute_dtype=torch.float32):
    """`GroupedMLP.forward` (moe/mlp.py:99-126): fc1 = gmm(x, w1[E,H,2F]); act = silu(fc1[:, :F]) *
    fc1[:, F:]; fc2 = gmm(act, w2[E,F,H]).  Intermediates are rounded to x.dtype between the
    ops, as separate kernels would."""
    fc1 = gmm(x_perm, w1, tokens_per_expert, compute_dtype=compute_dtype)
    act = swiglu(fc1.to(compute_dtype)).to(x_perm.dtype)
    return gmm(act, w2, tokens_per_expert, compute_dtype=compute_dtype)


def sequential_mlp(x_perm, fc1_w, fc2_w, tokens_per_expert, fc1_b=None, fc2_b=None,
                   compute_dtype=torch.float32):
    """`SequentialMLP.forward` (moe/mlp.py:176-211) over experts that are the dense `MLP` with
    `is_expert=True` (transformer/mlp.py:104-138): per expert e on its rows,
    t = x @ fc1_w[e].T (+ fc1_b[e], one rounding: `intermediate_parallel + bias_parallel`, which
    bias_swiglu_impl computes the same way), act = silu(t[:, :F]) * t[:, F:], out = act @ fc2_w[e].T;
    the fc2 bias is NOT added (skip_bias_add) but returned as rows, `output_bias.expand_as(output)`.
    fc1_w [E,2F,H], fc2_w [E,H,F], fc1_b [E,2F], fc2_b [E,H].  Returns (out, out_bias or None)."""
    outs, biases = [], []
    start = 0
    for e, n in enumerate(tokens_per_expert.tolist()):
        xe = x_perm[start:start + n]
        t = (xe.to(compute_dtype) @ fc1_w[e].to(compute_dtype).t()).to(x_perm.dtype)
        if fc1_b is not None:
            t = t + fc1_b[e]
        act = swiglu(t.to(compute_dtype)).to(x_perm.dtype)
        outs.append((act.to(compute_dtype) @ fc2_w[e].to(compute_dtype).t()).to(x_perm.dtype))
        if fc2_b is not None:
            biases.append(fc2_b[e].expand_as(outs[-1]))
        start += n
    assert start == x_perm.shape[0]
    return torch.cat(outs, dim=0), (torch.cat(biases, dim=0) if fc2_b is not None else None)


def allgather_combine(expert_out, probs, routing_map, sorted_indices, restore_shape, bias=None):
    """`MoEAllGatherTokenDispatcher.token_unpermutation` at EP = TP = 1 (moe/token_dispatcher.py:
    216-284): rows weighted by their gate and summed per token; the experts' bias rows, when there
    are any, take the same weighting and combine and are returned beside the output, not added."""
    pp = permuted_probs(probs, routing_map)
    out = unpermute(expert_out * pp.unsqueeze(-1), sorted_indices, restore_shape, routing_map=routing_map)
    out_bias = None
    if bias is not None:
        out_bias = unpermute(bias * pp.unsqueeze(-1), sorted_indices, restore_shape,
                             routing_map=routing_map).to(bias.dtype)
    return out.to(expert_out.dtype), out_bias


def shared_expert_mlp(x, w1s, w2s, compute_dtype=torch.float32):
    """`SharedExpertMLP.forward` (moe/mlp.py:271-278) without the optional gate: a dense SwiGLU
    MLP over all tokens, w1s [H, 2Fs], w2s [Fs, H]."""
    fc1 = (x.to(compute_dtype) @ w1s.to(compute_dtype)).to(x.dtype)
    act = swiglu(fc1.to(compute_dtype)).to(x.dtype)
    return (act.to(compute_dtype) @ w2s.to(compute_dtype)).to(x.dtype)


# ----------------------------------------------------------------------------
# Whole layer
# ----------------------------------------------------------------------------

def moe_layer(x, w_r, w1, w2, topk, residual=None, router_dtype=None, dispatcher="allgather",
              load_balancing_type="none", aux_loss_coeff=0.0, z_loss_coeff=None,
              shared_w1=None, shared_w2=None, compute_dtype=torch.float32,
              routing_override=None, **topk_kwargs):
    """router -> dispatch -> experts -> combine (+ residual), i.e. GalvatronMoERouter +
    GalvatronMoEMLP.forward (models/moe_modules.py:50-52, 121-128) at EP=TP=1.

    x: [S,B,H] or [T,H].  Returns (out, aux_total, info).  `routing_override=(probs, map)`
    replaces the router's output (used to hold the integer routing fixed when comparing
    floating-point results).
    """
    shape = x.shape
    H = shape[-1]
    x2d = x.reshape(-1, H)
    if routing_override is None:
        probs, routing_map, aux_total = router_forward(
            x2d, w_r, topk, router_dtype, load_balancing_type, aux_loss_coeff, z_loss_coeff,
            **topk_kwargs)
    else:
        probs, routing_map = routing_override
        aux_total = torch.zeros((), dtype=torch.float32, device=x.device)
    tokens_per_expert = routing_map.sum(dim=0).long()          # token_dispatcher.py:205
    permuted, sorted_indices = permute(x2d, routing_map)       # token_dispatcher.py:207-212
    expert_out = grouped_mlp(permuted, w1, w2, tokens_per_expert, compute_dtype)
    if dispatcher == "allgather":
        pp = permuted_probs(probs, routing_map)                # token_dispatcher.py:233-237
        weighted = expert_out.to(compute_dtype) * pp.to(compute_dtype).unsqueeze(-1)
        out = unpermute(weighted, sorted_indices, x2d.shape, routing_map=routing_map)
        out = out.to(expert_out.dtype)                         # token_dispatcher.py:281
    else:                                                      # alltoall, token_dispatcher.py:672-680
        out = unpermute(expert_out, sorted_indices, x2d.shape, probs=probs,
                        routing_map=routing_map, accumulate_dtype=compute_dtype)
    if shared_w1 is not None:
        out = out + shared_expert_mlp(x2d, shared_w1, shared_w2, compute_dtype)  # token_dispatcher.py:686-688
    out = out.view(shape)
    if residual is not None:
        out = out + residual                                   # moe_modules.py:127
    info = dict(probs=probs, routing_map=routing_map, tokens_per_expert=tokens_per_expert,
                sorted_indices=sorted_indices)
    return out, aux_total, info


# ----------------------------------------------------------------------------
# fp8 block-scaled expert weights (not in the reference: moe/mlp.py:164-184 is commented out)
# ----------------------------------------------------------------------------

FP8_MAX = 448.0  # largest finite float8_e4m3fn


def quantize_fp8_block(w: torch.Tensor, block: int = 128):
    """Quantise the last two dims of w [..., K, M] in `block` x `block` tiles to float8_e4m3fn with
    one scale per tile: scale = bf16(amax / 448) (1.0 for an all-zero tile), q = rne(w / scale).
    Returns (q float8_e4m3fn [..., K, M], scales bf16 [..., ceil(K/block), ceil(M/block)])."""
    *lead, K, M = w.shape
    kb, mb = (K + block - 1) // block, (M + block - 1) // block
    wp = torch.zeros(*lead, kb * block, mb * block, dtype=torch.float32, device=w.device)
    wp[..., :K, :M] = w.float()
    tiles = wp.view(*lead, kb, block, mb, block)
    amax = tiles.abs().amax(dim=(-3, -1))
    scale = (amax / FP8_MAX).to(torch.bfloat16)
    scale = torch.where(scale.float() == 0, torch.ones_like(scale), scale)
    q = (tiles / scale.float().unsqueeze(-1).unsqueeze(-3)).clamp(-FP8_MAX, FP8_MAX)
    q = q.view(*lead, kb * block, mb * block)[..., :K, :M].contiguous().to(torch.float8_e4m3fn)
    return q, scale


def dequantize_fp8_block(q: torch.Tensor, scale: torch.Tensor, block: int = 128) -> torch.Tensor:
    """w = float(q) * scale[block row, block col] in fp32."""
    *lead, K, M = q.shape
    s = scale.float().repeat_interleave(block, dim=-2).repeat_interleave(block, dim=-1)
    return q.float() * s[..., :K, :M]


def quantize_fp8_rows(x: torch.Tensor, block: int = 128):
    """Quantise x [N, K] along K in blocks of `block` elements to float8_e4m3fn with one power-of-two
    scale 2^e per row and block: the smallest e with amax * 2^-e <= 448 (e = -127 for an all-zero
    block, clamped to [-127, 127]), q = rne(x * 2^-e).  Returns (q [N, K], e int32 [ceil(K/block), N]).
    Not in the reference (its fp8 path is commented out, moe/mlp.py:164-184): the format of the
    build's fp8-activation products."""
    N, K = x.shape
    kb = (K + block - 1) // block
    xp = torch.zeros(N, kb * block, dtype=torch.float32, device=x.device)
    xp[:, :K] = x.float()
    tiles = xp.view(N, kb, block)
    amax = tiles.abs().amax(dim=-1)
    m, ex = torch.frexp(amax)  # amax = m * 2^ex, m in [0.5, 1); 448 = 0.875 * 2^9
    e = torch.where(m <= 0.875, ex - 9, ex - 8)
    e = torch.where(amax == 0, torch.full_like(e, -127), e).clamp(-127, 127)
    q = torch.ldexp(tiles, -e.unsqueeze(-1)).view(N, kb * block)[:, :K].contiguous().to(torch.float8_e4m3fn)
    return q, e.t().contiguous().to(torch.int32)


def dequantize_fp8_rows(q: torch.Tensor, e: torch.Tensor, block: int = 128) -> torch.Tensor:
    """x = float(q) * 2^e[block of the column, row] in fp32 (exact)."""
    N, K = q.shape
    ee = e.t().repeat_interleave(block, dim=1)[:, :K]
    return torch.ldexp(q.float(), ee)

