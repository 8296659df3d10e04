"""Tensor-level wrappers over the C ABI: argument checks, output allocation (PyTorch's caching
allocator owns all memory), stream selection.  No autograd here; see moe_utils.py / fused_kernels.py
/ grouped_gemm for the differentiable, reference-named entry points.
"""
from __future__ import annotations

import collections
from dataclasses import dataclass
from typing import Optional

import torch

from . import _C

_DTYPES = {torch.float32: _C.GMOE_F32, torch.bfloat16: _C.GMOE_BF16, torch.float16: _C.GMOE_F16}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32, bfloat16, float16 only)" % t.dtype)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _check_dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        assert t.is_cuda, "MoE HIP kernels need tensors on the GPU (got %s)" % t.device
        assert t.is_contiguous(), "MoE HIP kernels need contiguous tensors"
        if dev is None:
            dev = t.device
        else:
            assert t.device == dev, "tensors on different devices"
    return dev


def _index(dev) -> int:
    return dev.index if dev.index is not None else torch.cuda.current_device()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev) -> int:
    """Raw handle of the current stream of `dev` (no Stream object is built for it)."""
    if _raw_stream is not None:
        return _raw_stream(_index(dev))
    return torch.cuda.current_stream(dev).cuda_stream


class _on:
    """`with _on(dev):` makes `dev` the current device for a library call, like torch.cuda.device,
    at a fraction of its cost: a step with few rows per expert is bound by the time Python takes
    to issue the launches."""
    __slots__ = ("idx", "prev")

    def __init__(self, dev):
        self.idx = _index(dev)

    def __enter__(self):
        self.prev = torch.cuda._exchange_device(self.idx)

    def __exit__(self, *exc):
        torch.cuda._maybe_exchange_device(self.prev)
        return False


if not (hasattr(torch.cuda, "_exchange_device") and hasattr(torch.cuda, "_maybe_exchange_device")):
    _on = torch.cuda.device  # noqa: F811  (a torch without the two calls: the public context manager)


# --------------------------------------------------------------------------------------------
# Router
# --------------------------------------------------------------------------------------------

def route_topk(logits: torch.Tensor, k: int, score_fn: str = "softmax", pre_softmax: bool = False,
               scaling: Optional[float] = None, expert_bias: Optional[torch.Tensor] = None,
               num_groups: Optional[int] = None, group_topk: Optional[int] = None,
               want_stats: bool = False, want_topk_idx: bool = False,
               selection_scores: Optional[torch.Tensor] = None):
    """Returns (probs [T,E], routing_map [T,E] bool, tokens_per_expert [E] int64, stats [E+1] fp32
    or None, topk_idx [T,k] int32 or None).  `selection_scores` [T,E] fp32: what top-k ranks instead
    of the scores (the gates still come from the scores)."""
    assert logits.dim() == 2, f"Expected 2D logits [num_tokens, num_experts], got {logits.dim()}."
    dev = _check_dev(logits, expert_bias, selection_scores)
    if selection_scores is not None:
        assert selection_scores.dtype == torch.float32 and selection_scores.shape == logits.shape
    T, E = logits.shape
    assert 1 <= k <= E, "topk must be in [1, num_experts]"
    if score_fn not in ("softmax", "sigmoid"):
        raise ValueError(f"Invalid score_function: {score_fn}")
    if expert_bias is not None:
        assert expert_bias.dtype == torch.float32 and expert_bias.numel() == E
    probs = torch.empty_like(logits)
    rmap = torch.empty((T, E), dtype=torch.bool, device=dev)
    counts = torch.empty((E,), dtype=torch.int64, device=dev)
    topk_idx = torch.empty((T, k), dtype=torch.int32, device=dev) if want_topk_idx else None
    stats = ws = None
    L = _C.lib()
    if want_stats:
        stats = torch.empty((E + 1,), dtype=torch.float32, device=dev)
        ws = torch.empty((L.gmoe_route_workspace_bytes(T, E),), dtype=torch.uint8, device=dev)
    with _on(dev):
        st = L.gmoe_route_topk(
            _ptr(logits), _dt(logits), T, E, k,
            _C.SCORE_SIGMOID if score_fn == "sigmoid" else _C.SCORE_SOFTMAX,
            1 if pre_softmax else 0, float(scaling) if scaling else 0.0, _ptr(expert_bias),
            _ptr(selection_scores),
            int(num_groups) if group_topk else 0, int(group_topk) if group_topk else 0,
            _ptr(probs), _ptr(rmap), _ptr(topk_idx), _ptr(counts), _ptr(stats), _ptr(ws),
            _stream(dev))
    _C.check(st, "gmoe_route_topk")
    return probs, rmap, counts, stats, topk_idx


def _score_fn(score_fn: str) -> int:
    """softmax | sigmoid | identity (the tensor already holds the scores)."""
    try:
        return {"softmax": _C.SCORE_SOFTMAX, "sigmoid": _C.SCORE_SIGMOID,
                "identity": _C.SCORE_IDENTITY}[score_fn]
    except KeyError:
        raise ValueError(f"Invalid score_function: {score_fn}")


def seq_aux_loss(logits: torch.Tensor, routing_map: torch.Tensor, batch_size: int, seq_length: int,
                 k: int, coeff: float, score_fn: str = "softmax"):
    """Sequence-level load-balancing loss (gmoe_seq_aux_loss).  Returns (loss [] fp32,
    seq_counts [B,E] fp32, seq_scores [B,E] fp32)."""
    dev = _check_dev(logits, routing_map)
    T, E = logits.shape
    assert T == batch_size * seq_length and routing_map.shape == (T, E)
    assert routing_map.dtype == torch.bool
    counts = torch.empty((batch_size, E), dtype=torch.float32, device=dev)
    scores = torch.empty((batch_size, E), dtype=torch.float32, device=dev)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_seq_aux_loss(_ptr(logits), _dt(logits), _ptr(routing_map), seq_length,
                                        batch_size, E, k, _score_fn(score_fn), float(coeff),
                                        _ptr(counts), _ptr(scores), _ptr(loss), _stream(dev))
    _C.check(st, "gmoe_seq_aux_loss")
    return loss, counts, scores


def seq_aux_loss_bwd(logits: torch.Tensor, seq_counts: torch.Tensor, batch_size: int,
                     seq_length: int, k: int, coeff: float, score_fn: str = "softmax",
                     grad_loss: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d loss / d logits of seq_aux_loss, times grad_loss (a device scalar) when given."""
    dev = _check_dev(logits, seq_counts, grad_loss)
    T, E = logits.shape
    assert seq_counts.shape == (batch_size, E) and seq_counts.dtype == torch.float32
    if grad_loss is not None:
        assert grad_loss.dtype == torch.float32 and grad_loss.numel() == 1
    dlogits = torch.empty_like(logits)
    scale = coeff * E / (batch_size * seq_length * seq_length * k)
    with _on(dev):
        st = _C.lib().gmoe_seq_aux_loss_bwd(_ptr(logits), _dt(logits), seq_length, batch_size, E, k,
                                            _score_fn(score_fn), _ptr(seq_counts), float(scale),
                                            _ptr(grad_loss), _ptr(dlogits), _stream(dev))
    _C.check(st, "gmoe_seq_aux_loss_bwd")
    return dlogits


def score_stats(x: torch.Tensor, k: int = 1, score_fn: str = "identity") -> torch.Tensor:
    """stats [E+1] fp32 of a [T,E] matrix: stats[e] = sum_t score(x)[t,e], stats[E] = sum_t
    logsumexp(x[t,:])^2 (gmoe_score_stats), summed in a fixed order."""
    dev = _check_dev(x)
    T, E = x.shape
    L = _C.lib()
    stats = torch.empty((E + 1,), dtype=torch.float32, device=dev)
    ws = torch.empty((L.gmoe_route_workspace_bytes(T, E),), dtype=torch.uint8, device=dev)
    with _on(dev):
        st = L.gmoe_score_stats(_ptr(x), _dt(x), T, E, k, _score_fn(score_fn), _ptr(stats), _ptr(ws),
                                _stream(dev))
    _C.check(st, "gmoe_score_stats")
    return stats


def score_stats_bwd(x: torch.Tensor, k: int = 1, score_fn: str = "identity",
                    weights: Optional[torch.Tensor] = None, aux_scale: float = 0.0,
                    z_scale: float = 0.0, grad_loss: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d/dx of aux_scale * <weights, stats[:E]> + z_scale * stats[E], times grad_loss (a device
    scalar) when given (gmoe_score_stats_bwd)."""
    dev = _check_dev(x, weights, grad_loss)
    T, E = x.shape
    if weights is not None:
        assert weights.dtype == torch.float32 and weights.numel() == E
    if grad_loss is not None:
        assert grad_loss.dtype == torch.float32 and grad_loss.numel() == 1
    dx = torch.empty_like(x)
    with _on(dev):
        st = _C.lib().gmoe_score_stats_bwd(_ptr(x), _dt(x), T, E, k, _score_fn(score_fn), _ptr(weights),
                                           float(aux_scale), float(z_scale), _ptr(grad_loss), _ptr(dx),
                                           _stream(dev))
    _C.check(st, "gmoe_score_stats_bwd")
    return dx


# The iteration is one workgroup's loop on the device: a bound keeps a tolerance that is never met
# (tol = 0) from looking like a hang.  Routing-sized problems converge to 1e-4 in tens of iterations.
SINKHORN_MAX_ITERS = 10000


def sinkhorn(logits: torch.Tensor, tol: float = 0.0001, max_iters: int = SINKHORN_MAX_ITERS,
             want_iters: bool = False):
    """Sinkhorn-normalised routing costs [T,E] fp32 of the logits (gmoe_sinkhorn); the iteration
    runs on the device, at most `max_iters` times (`want_iters`: also the count, a device int32)."""
    dev = _check_dev(logits)
    T, E = logits.shape
    out = torch.empty((T, E), dtype=torch.float32, device=dev)
    iters = torch.zeros((1,), dtype=torch.int32, device=dev) if want_iters else None
    with _on(dev):
        st = _C.lib().gmoe_sinkhorn(_ptr(logits), _dt(logits), T, E, float(tol), int(max_iters),
                                    _ptr(out), _ptr(iters), _stream(dev))
    _C.check(st, "gmoe_sinkhorn")
    return (out, iters) if want_iters else out


def router_bookkeeping(stats: Optional[torch.Tensor], tokens_per_expert: Optional[torch.Tensor],
                       num_experts: int, aux_factor: float = 0.0, z_factor: float = 0.0,
                       want_aux: bool = False, want_z: bool = False,
                       aux_slot: Optional[torch.Tensor] = None, aux_slot_scale: float = 1.0,
                       z_slot: Optional[torch.Tensor] = None, z_slot_scale: float = 1.0,
                       local_tokens: Optional[torch.Tensor] = None):
    """Loss values from the router statistics, tracker slots and the running token counts in one
    launch (gmoe_router_bookkeeping).  `aux_slot` / `z_slot`: one-element fp32 views that receive
    `+= loss * scale`.  Returns (aux_loss or None, z_loss or None) as device scalars."""
    dev = _check_dev(stats, tokens_per_expert, local_tokens)
    for t in (stats, aux_slot, z_slot, local_tokens):
        assert t is None or t.dtype == torch.float32
    for t in (aux_slot, z_slot):
        assert t is None or (t.is_cuda and t.numel() >= 1)
    aux = torch.empty((), dtype=torch.float32, device=dev) if want_aux else None
    z = torch.empty((), dtype=torch.float32, device=dev) if want_z else None
    with _on(dev):
        st = _C.lib().gmoe_router_bookkeeping(_ptr(stats), _ptr(tokens_per_expert), num_experts,
                                              float(aux_factor), float(z_factor), _ptr(aux), _ptr(z),
                                              _ptr(aux_slot), float(aux_slot_scale), _ptr(z_slot),
                                              float(z_slot_scale), _ptr(local_tokens), _stream(dev))
    _C.check(st, "gmoe_router_bookkeeping")
    return aux, z


def expert_bias_update(tokens_per_expert: torch.Tensor, expert_bias: torch.Tensor,
                       update_rate: float) -> torch.Tensor:
    """expert_bias + sign(mean(tokens) - tokens) * rate over the last dimension
    (gmoe_expert_bias_update)."""
    tokens = tokens_per_expert.to(torch.float32).contiguous()
    bias = expert_bias.to(torch.float32).contiguous()
    dev = _check_dev(tokens, bias)
    assert tokens.shape == bias.shape and tokens.dim() >= 1
    E = tokens.shape[-1]
    rows = tokens.numel() // E if E else 0
    out = torch.empty_like(bias)
    with _on(dev):
        st = _C.lib().gmoe_expert_bias_update(_ptr(tokens), _ptr(bias), rows, E, float(update_rate),
                                              _ptr(out), _stream(dev))
    _C.check(st, "gmoe_expert_bias_update")
    return out


def route_topk_bwd(logits, k, score_fn, pre_softmax, scaling, routing_map, dprobs,
                   tokens_per_expert=None, aux_scale: float = 0.0, z_scale: float = 0.0,
                   loss_scale: Optional[torch.Tensor] = None):
    dev = _check_dev(logits, routing_map, dprobs, tokens_per_expert, loss_scale)
    if loss_scale is not None:
        assert loss_scale.dtype == torch.float32 and loss_scale.numel() == 1
    T, E = logits.shape
    assert dprobs.shape == logits.shape and dprobs.dtype == logits.dtype
    assert routing_map.dtype == torch.bool and routing_map.shape == logits.shape
    dlogits = torch.empty_like(logits)
    with _on(dev):
        st = _C.lib().gmoe_route_topk_bwd(
            _ptr(logits), _dt(logits), T, E, k,
            _C.SCORE_SIGMOID if score_fn == "sigmoid" else _C.SCORE_SOFTMAX,
            1 if pre_softmax else 0, float(scaling) if scaling else 0.0, _ptr(routing_map),
            _ptr(dprobs), _ptr(tokens_per_expert), float(aux_scale), float(z_scale),
            _ptr(loss_scale), _ptr(dlogits), _stream(dev))
    _C.check(st, "gmoe_route_topk_bwd")
    return dlogits


# --------------------------------------------------------------------------------------------
# Permutation plan + row movers
# --------------------------------------------------------------------------------------------

@dataclass
class PermutePlan:
    """Device-side description of one expert-major permutation.

    dst_map [T,E] int32: destination row of (token, expert) or -1; sorted_indices [n_out] int64:
    source token of every permuted row (the reference's `sorted_indices`); tokens_per_expert [E]
    and expert_offsets [E+1] int64.
    """
    dst_map: torch.Tensor
    sorted_indices: Optional[torch.Tensor]
    row_id_map: Optional[torch.Tensor]
    tokens_per_expert: torch.Tensor
    expert_offsets: torch.Tensor
    num_tokens: int
    num_experts: int
    n_out: int
    padded: bool = False  # fixed-capacity blocks: some permuted rows may have no source token


def permute_plan(routing_map: torch.Tensor, n_out: int, capacity: int = 0,
                 want_sorted: bool = True, want_row_id_map: bool = False) -> PermutePlan:
    assert routing_map.dim() == 2
    if routing_map.dtype != torch.bool:
        routing_map = routing_map.bool()
    routing_map = routing_map.contiguous()
    dev = _check_dev(routing_map)
    T, E = routing_map.shape
    L = _C.lib()
    dst_map = torch.empty((T, E), dtype=torch.int32, device=dev)
    # rows that stay unwritten (padding of a fixed-capacity block) read as token 0
    sorted_indices = (torch.zeros if capacity > 0 else torch.empty)(
        (n_out,), dtype=torch.int64, device=dev) if want_sorted else None
    row_id_map = torch.empty((E, T), dtype=torch.int64, device=dev) if want_row_id_map else None
    counts = torch.empty((E,), dtype=torch.int64, device=dev)
    offsets = torch.empty((E + 1,), dtype=torch.int64, device=dev)
    ws = torch.empty((max(1, L.gmoe_permute_plan_workspace_bytes(T, E)),), dtype=torch.uint8,
                     device=dev)
    with _on(dev):
        st = L.gmoe_permute_plan(_ptr(routing_map), T, E, int(capacity), _ptr(dst_map),
                                 _ptr(sorted_indices), int(n_out), _ptr(row_id_map), _ptr(counts),
                                 _ptr(offsets), _ptr(ws), _stream(dev))
    _C.check(st, "gmoe_permute_plan")
    return PermutePlan(dst_map, sorted_indices, row_id_map, counts, offsets, T, E, int(n_out),
                       padded=capacity > 0)


def permute_rows(tokens: torch.Tensor, dst_map: torch.Tensor, n_out: int,
                 probs: Optional[torch.Tensor] = None, zero_fill: bool = False):
    """permuted[dst_map[t,e]] = tokens[t]; optionally permuted_probs[dst] = probs[t,e]."""
    dev = _check_dev(tokens, dst_map, probs)
    T, H = tokens.shape
    assert dst_map.dtype == torch.int32 and dst_map.shape[0] == T
    E = dst_map.shape[1]
    alloc = torch.zeros if zero_fill else torch.empty
    out = alloc((n_out, H), dtype=tokens.dtype, device=dev)
    pp = None
    if probs is not None:
        assert probs.shape == (T, E)
        pp = alloc((n_out,), dtype=probs.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_permute_rows(_ptr(tokens), _dt(tokens), T, H, E, _ptr(dst_map), n_out,
                                        _ptr(out), _ptr(probs), _dt(probs) if probs is not None else 0,
                                        _ptr(pp), _stream(dev))
    _C.check(st, "gmoe_permute_rows")
    return out, pp


def unpermute_rows(permuted: torch.Tensor, dst_map: torch.Tensor, num_tokens: int,
                   merging_probs: Optional[torch.Tensor] = None,
                   permuted_probs: Optional[torch.Tensor] = None,
                   residual: Optional[torch.Tensor] = None, addend: Optional[torch.Tensor] = None):
    """out[t] = sum_e permuted[dst_map[t,e]] * merging_probs[t,e] (fp32 accumulation), plus
    `addend[t]` and then `residual[t]`, each added to the rounded value before it, when given."""
    dev = _check_dev(permuted, dst_map, merging_probs, permuted_probs, residual, addend)
    n_out, H = permuted.shape
    T, E = dst_map.shape
    assert T == num_tokens and dst_map.dtype == torch.int32
    for extra in (residual, addend):
        assert extra is None or (extra.shape == (T, H) and extra.dtype == permuted.dtype)
    out = torch.empty((T, H), dtype=permuted.dtype, device=dev)
    pdt = 0
    up = None
    if merging_probs is not None:
        assert merging_probs.shape == (T, E)
        pdt = _dt(merging_probs)
    if permuted_probs is not None:
        assert merging_probs is None or merging_probs.dtype == permuted_probs.dtype
        pdt = _dt(permuted_probs)
        up = torch.empty((T, E), dtype=permuted_probs.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_unpermute_rows(_ptr(permuted), _dt(permuted), T, H, E, _ptr(dst_map),
                                          n_out, _ptr(merging_probs), pdt, _ptr(out),
                                          _ptr(permuted_probs), _ptr(up), _ptr(addend),
                                          _ptr(residual), _stream(dev))
    _C.check(st, "gmoe_unpermute_rows")
    return out, up


def unpermute_rows_bwd(grad_out: torch.Tensor, fwd_input: torch.Tensor, dst_map: torch.Tensor,
                       merging_probs: torch.Tensor, zero_fill: bool = False):
    dev = _check_dev(grad_out, fwd_input, dst_map, merging_probs)
    T, H = grad_out.shape
    n_out = fwd_input.shape[0]
    E = dst_map.shape[1]
    assert fwd_input.dtype == grad_out.dtype and fwd_input.shape[1] == H
    # rows no token maps to (padding of a fixed-capacity block) get a zero gradient
    grad_perm = torch.zeros_like(fwd_input) if zero_fill else torch.empty_like(fwd_input)
    grad_probs = torch.empty_like(merging_probs)
    with _on(dev):
        st = _C.lib().gmoe_unpermute_rows_bwd(_ptr(grad_out), _ptr(fwd_input), _dt(grad_out), T, H,
                                              E, _ptr(dst_map), n_out, _ptr(merging_probs),
                                              _dt(merging_probs), _ptr(grad_perm),
                                              _ptr(grad_probs), _stream(dev))
    _C.check(st, "gmoe_unpermute_rows_bwd")
    return grad_perm, grad_probs


def scatter_add_rows(permuted: torch.Tensor, sorted_indices: torch.Tensor, num_tokens: int,
                     permuted_probs: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[sorted_indices[r]] += permuted[r] (* permuted_probs[r]) for callers without a plan."""
    dev = _check_dev(permuted, sorted_indices, permuted_probs)
    n, H = permuted.shape
    assert sorted_indices.dtype == torch.int64 and sorted_indices.numel() == n
    acc = torch.zeros((num_tokens, H), dtype=torch.float32, device=dev)
    L = _C.lib()
    with _on(dev):
        st = L.gmoe_scatter_add_rows(_ptr(permuted), _dt(permuted), n, H, _ptr(sorted_indices),
                                     _ptr(permuted_probs),
                                     _dt(permuted_probs) if permuted_probs is not None else 0,
                                     num_tokens, _ptr(acc), _stream(dev))
        _C.check(st, "gmoe_scatter_add_rows")
        if permuted.dtype == torch.float32:
            return acc
        out = torch.empty((num_tokens, H), dtype=permuted.dtype, device=dev)
        st = L.gmoe_cast_rows(_ptr(acc), acc.numel(), _dt(out), _ptr(out), _stream(dev))
        _C.check(st, "gmoe_cast_rows")
    return out


def sort_chunks(inp: torch.Tensor, split_sizes: torch.Tensor, sorted_idxs: torch.Tensor):
    """Returns (out, row_map) with out = cat(chunks[sorted_idxs]) and row_map[dst] = src."""
    dev = _check_dev(inp)
    n, H = inp.shape
    if split_sizes.device.type == "cpu":
        # host tables can be checked for free (torch.split in the reference raises on a mismatch)
        assert int(split_sizes.sum()) == n, "split sizes must sum to the number of rows"
        if sorted_idxs.device.type == "cpu" and sorted_idxs.numel():
            assert 0 <= int(sorted_idxs.min()) and int(sorted_idxs.max()) < split_sizes.numel()
    split_sizes = split_sizes.to(device=dev, dtype=torch.int64).contiguous()
    sorted_idxs = sorted_idxs.to(device=dev, dtype=torch.int64).contiguous()
    out = torch.empty_like(inp)
    row_map = torch.empty((n,), dtype=torch.int64, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_sort_chunks(_ptr(inp), _dt(inp), n, H, _ptr(split_sizes),
                                       _ptr(sorted_idxs), split_sizes.numel(), _ptr(out),
                                       _ptr(row_map), _stream(dev))
    _C.check(st, "gmoe_sort_chunks")
    return out, row_map


def scatter_rows_by_map(inp: torch.Tensor, row_map: torch.Tensor) -> torch.Tensor:
    """out[row_map[r]] = inp[r] (inverse of the gather sort_chunks performed)."""
    dev = _check_dev(inp, row_map)
    n, H = inp.shape
    out = torch.empty_like(inp)
    with _on(dev):
        st = _C.lib().gmoe_scatter_rows_by_map(_ptr(inp), _dt(inp), n, H, _ptr(row_map), _ptr(out),
                                               _stream(dev))
    _C.check(st, "gmoe_scatter_rows_by_map")
    return out


# --------------------------------------------------------------------------------------------
# Expert MLP
# --------------------------------------------------------------------------------------------

_ACTS = {"silu": _C.ACT_SILU, "swiglu": _C.ACT_SILU, "gelu": _C.ACT_GELU, "geglu": _C.ACT_GELU}


def glu_fwd(y: torch.Tensor, act: str = "silu") -> torch.Tensor:
    dev = _check_dev(y)
    assert y.dim() == 2 and y.shape[1] % 2 == 0
    N, F2 = y.shape
    out = torch.empty((N, F2 // 2), dtype=y.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_glu_fwd(_ptr(y), _dt(y), N, F2 // 2, _ACTS[act], _ptr(out), _stream(dev))
    _C.check(st, "gmoe_glu_fwd")
    return out


def bias_rows(x: Optional[torch.Tensor], bias: torch.Tensor, num_rows: Optional[int] = None,
              expert_offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = x[r] + bias[expert of row r] (one rounding).  bias [M] with no offset table (every
    row in one group) or [E,M] with expert_offsets [E+1] (device int64); `x` None expands the bias
    alone to `num_rows` rows."""
    dev = _check_dev(x, bias, expert_offsets)
    if expert_offsets is None:
        assert bias.dim() == 1 or bias.shape[0] == 1
        E = 1
    else:
        assert bias.dim() == 2 and expert_offsets.dtype == torch.int64
        E = bias.shape[0]
        assert expert_offsets.numel() == E + 1
    M = bias.shape[-1]
    if x is not None:
        assert x.dim() == 2 and x.shape[1] == M and x.dtype == bias.dtype
        N = x.shape[0]
    else:
        assert num_rows is not None
        N = int(num_rows)
    out = torch.empty((N, M), dtype=bias.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_bias_rows(_ptr(x), _ptr(bias), _dt(bias), N, M, _ptr(expert_offsets), E,
                                     _ptr(out), _stream(dev))
    _C.check(st, "gmoe_bias_rows")
    return out


def bias_rows_bwd(grad: torch.Tensor, expert_offsets: Optional[torch.Tensor] = None,
                  num_experts: int = 1) -> torch.Tensor:
    """Sum of `grad` [N,M] over each expert's rows -> [E,M] ([M] without an offset table), fp32
    sums in a fixed order, rounded once to grad's dtype."""
    dev = _check_dev(grad, expert_offsets)
    N, M = grad.shape
    E = 1 if expert_offsets is None else int(num_experts)
    if expert_offsets is not None:
        assert expert_offsets.dtype == torch.int64 and expert_offsets.numel() == E + 1
    out = torch.empty((E, M) if expert_offsets is not None else (M,), dtype=grad.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_bias_rows_bwd(_ptr(grad), _dt(grad), N, M, _ptr(expert_offsets), E,
                                         _ptr(out), _stream(dev))
    _C.check(st, "gmoe_bias_rows_bwd")
    return out


def glu_bwd(grad_out: torch.Tensor, y: torch.Tensor, act: str = "silu") -> torch.Tensor:
    dev = _check_dev(grad_out, y)
    N, F2 = y.shape
    assert grad_out.shape == (N, F2 // 2) and grad_out.dtype == y.dtype
    dy = torch.empty_like(y)
    with _on(dev):
        st = _C.lib().gmoe_glu_bwd(_ptr(grad_out), _ptr(y), _dt(y), N, F2 // 2, _ACTS[act], _ptr(dy),
                                   _stream(dev))
    _C.check(st, "gmoe_glu_bwd")
    return dy


def glu_fwd_fp8store(y: torch.Tensor, act: str = "silu"):
    """(act(y[:, :F]) * y[:, F:], y.to(float8_e4m3fn)) in one pass over y
    (transformer/fused_kernels.py:190-197 with fp8_input_store)."""
    dev = _check_dev(y)
    assert y.dim() == 2 and y.shape[1] % 2 == 0
    N, F2 = y.shape
    out = torch.empty((N, F2 // 2), dtype=y.dtype, device=dev)
    y8 = torch.empty((N, F2), dtype=torch.float8_e4m3fn, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_glu_fwd_fp8store(_ptr(y), _dt(y), N, F2 // 2, _ACTS[act], _ptr(out), _ptr(y8),
                                            _stream(dev))
    _C.check(st, "gmoe_glu_fwd_fp8store")
    return out, y8


def glu_bwd_fp8in(grad_out: torch.Tensor, y_fp8: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """The activation backward on y_fp8 widened to grad_out's dtype
    (transformer/fused_kernels.py:199-204 with fp8_input_store)."""
    dev = _check_dev(grad_out, y_fp8)
    N, F2 = y_fp8.shape
    assert y_fp8.dtype == torch.float8_e4m3fn and grad_out.shape == (N, F2 // 2)
    dy = torch.empty((N, F2), dtype=grad_out.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_glu_bwd_fp8in(_ptr(grad_out), _ptr(y_fp8), _dt(grad_out), N, F2 // 2,
                                         _ACTS[act], _ptr(dy), _stream(dev))
    _C.check(st, "gmoe_glu_bwd_fp8in")
    return dy


def expert_offsets_from_batch_sizes(batch_sizes: torch.Tensor, device) -> torch.Tensor:
    """Exclusive prefix [E+1] int64 on `device`.  A tensor produced by this package's dispatchers
    carries its device-side offsets (attribute `_gmoe_offsets`), which avoids any copy."""
    cached = getattr(batch_sizes, "_gmoe_offsets", None)
    if cached is not None and cached.device == torch.device(device):
        return cached
    bs = batch_sizes.to(torch.int64)
    off = torch.zeros(bs.numel() + 1, dtype=torch.int64, device=bs.device)
    torch.cumsum(bs, 0, out=off[1:])
    return off.to(device)


class _DeviceTableCache:
    """Small constant device tensors built once per key and shared by every stream afterwards.

    A table is written on the device's default stream and that stream is synchronised once, so any
    stream may read it later without an event.  Nothing is built while a stream is capturing a HIP
    graph (the host-to-device copy would be recorded into the graph, or fail): the caller warms the
    shape up first.  At the limit the least recently used entry goes, after a device
    synchronisation, because a kernel on some stream may still be reading it."""

    def __init__(self, limit: int):
        self.limit = limit
        self.entries = collections.OrderedDict()

    def get(self, key, device, build):
        t = self.entries.get(key)
        if t is not None:
            self.entries.move_to_end(key)
            return t
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("a device-side table for %r is missing while a HIP graph is being "
                               "captured: run the step once before the capture" % (key,))
        if len(self.entries) >= self.limit:
            torch.cuda.synchronize(device)
            self.entries.popitem(last=False)
        default = torch.cuda.default_stream(device)
        with torch.cuda.stream(default):
            t = build()
        default.synchronize()
        self.entries[key] = t
        return t


_ONE_GROUP = _DeviceTableCache(1024)
_IDENTITY_MAPS = _DeviceTableCache(32)


def one_group(n: int, device) -> torch.Tensor:
    """`batch_sizes` of a single group holding n rows: a device int64 [1] tensor that carries its
    offset table [0, n], built once per (n, device), so dense products on the grouped kernels cost
    no host-to-device copy per call."""
    device = torch.device(device)

    def build():
        t = torch.tensor([n], dtype=torch.int64, device=device)
        t._gmoe_offsets = torch.tensor([0, n], dtype=torch.int64, device=device)
        return t

    return _ONE_GROUP.get((int(n), device), device, build)


def identity_map(n: int, device) -> torch.Tensor:
    """dst_map [n,1] int32 = arange(n): the combine kernels as a per-row scaling."""
    device = torch.device(device)
    return _IDENTITY_MAPS.get((int(n), device), device,
                              lambda: torch.arange(n, dtype=torch.int32, device=device).view(n, 1))


def gmm(a: torch.Tensor, b: torch.Tensor, expert_offsets: torch.Tensor, trans_a: bool = False,
        trans_b: bool = False, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Grouped GEMM on device offsets (see gmoe_gmm in include/galvatron_moe.h)."""
    dev = _check_dev(a, b, expert_offsets)
    assert a.dim() == 2 and a.dtype == b.dtype
    assert expert_offsets.dtype == torch.int64
    E = expert_offsets.numel() - 1
    out_dtype = out_dtype or a.dtype
    N, K = a.shape
    if trans_a:
        assert not trans_b and b.dim() == 2 and b.shape[0] == N
        M = b.shape[1]
        c = torch.empty((E, K, M), dtype=out_dtype, device=dev)
    else:
        assert b.dim() == 3 and b.shape[0] == E
        if trans_b:
            assert b.shape[2] == K
            M = b.shape[1]
        else:
            assert b.shape[1] == K
            M = b.shape[2]
        c = torch.empty((N, M), dtype=out_dtype, device=dev)
    L = _C.lib()
    ws_bytes = L.gmoe_gmm_workspace_bytes(E, N, K, M, 1 if trans_a else 0, 1 if trans_b else 0, _dt(a))
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
    with _on(dev):
        st = L.gmoe_gmm(_ptr(a), _ptr(b), _ptr(c), _ptr(expert_offsets), E, N, K, M,
                        1 if trans_a else 0, 1 if trans_b else 0, _dt(a), _DTYPES[out_dtype],
                        _ptr(ws), ws_bytes, _stream(dev))
    _C.check(st, "gmoe_gmm")
    return c


def gmm_glu(a: torch.Tensor, w1: torch.Tensor, expert_offsets: torch.Tensor, act: str = "silu"):
    """fc1 = gmm(a, w1 [E,K,2F]); act_out = act(fc1[:, :F]) * fc1[:, F:], one launch for large
    16-bit groups.  Returns (fc1 [N,2F], act_out [N,F])."""
    dev = _check_dev(a, w1, expert_offsets)
    assert a.dim() == 2 and w1.dim() == 3 and a.dtype == w1.dtype and w1.shape[1] == a.shape[1]
    assert expert_offsets.dtype == torch.int64 and w1.shape[2] % 2 == 0
    E = expert_offsets.numel() - 1
    assert w1.shape[0] == E
    N, K = a.shape
    F = w1.shape[2] // 2
    fc1 = torch.empty((N, 2 * F), dtype=a.dtype, device=dev)
    out = torch.empty((N, F), dtype=a.dtype, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_gmm_glu(_ptr(a), _ptr(w1), _ptr(fc1), _ptr(out), _ptr(expert_offsets), E,
                                   N, K, F, _ACTS[act], _dt(a), _stream(dev))
    _C.check(st, "gmoe_gmm_glu")
    return fc1, out


def gmm_glu_bwd(grad_out: torch.Tensor, w2: torch.Tensor, fc1: torch.Tensor,
                expert_offsets: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """grad_fc1 [N,2F] from grad_out [N,K] and w2 [E,F,K]: d(act) = gmm(grad_out, w2, trans_b) fused
    with the backward of the gated activation (fc1 read back, d(act) never stored)."""
    dev = _check_dev(grad_out, w2, fc1, expert_offsets)
    assert grad_out.dim() == 2 and w2.dim() == 3 and grad_out.dtype == w2.dtype == fc1.dtype
    E = expert_offsets.numel() - 1
    N, K = grad_out.shape
    F = w2.shape[1]
    assert w2.shape == (E, F, K) and fc1.shape == (N, 2 * F)
    dfc1 = torch.empty_like(fc1)
    with _on(dev):
        st = _C.lib().gmoe_gmm_glu_bwd(_ptr(grad_out), _ptr(w2), _ptr(fc1), _ptr(dfc1),
                                       _ptr(expert_offsets), E, N, K, F, _ACTS[act], _dt(grad_out),
                                       _stream(dev))
    _C.check(st, "gmoe_gmm_glu_bwd")
    return dfc1


def quantize_fp8_block(w: torch.Tensor):
    """w [..., K, M] -> (q [..., K, M] float8_e4m3fn, scale [..., ceil(K/128), ceil(M/128)] bf16),
    one scale per 128x128 tile (see gmoe_quantize_fp8_block in include/galvatron_moe.h)."""
    assert w.dim() >= 2
    w = w.contiguous()
    dev = _check_dev(w)
    *lead, K, M = w.shape
    batch = 1
    for d in lead:
        batch *= d
    q = torch.empty(w.shape, dtype=torch.float8_e4m3fn, device=dev)
    scale = torch.empty((*lead, (K + 127) // 128, (M + 127) // 128), dtype=torch.bfloat16, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_quantize_fp8_block(_ptr(w), _dt(w), batch, K, M, _ptr(q), _ptr(scale),
                                              _stream(dev))
    _C.check(st, "gmoe_quantize_fp8_block")
    return q, scale


def gmm_fp8w(a: torch.Tensor, b_q: torch.Tensor, b_scale: torch.Tensor, expert_offsets: torch.Tensor,
             trans_b: bool = False) -> torch.Tensor:
    """Grouped GEMM of bf16 rows with block-scaled fp8 weights: c[rows_e] = a[rows_e] @ w[e]
    (or @ w[e]^T with trans_b), w[e] = float(b_q[e]) * scale per 128x128 tile."""
    dev = _check_dev(a, b_q, b_scale, expert_offsets)
    assert a.dim() == 2 and a.dtype == torch.bfloat16 and b_q.dtype == torch.float8_e4m3fn
    assert b_scale.dtype == torch.bfloat16 and expert_offsets.dtype == torch.int64
    assert b_q.is_contiguous() and b_scale.is_contiguous() and a.is_contiguous()
    E = expert_offsets.numel() - 1
    N, K = a.shape
    assert b_q.dim() == 3 and b_q.shape[0] == E
    M = b_q.shape[1] if trans_b else b_q.shape[2]
    assert (b_q.shape[2] if trans_b else b_q.shape[1]) == K
    assert tuple(b_scale.shape) == (E, (b_q.shape[1] + 127) // 128, (b_q.shape[2] + 127) // 128)
    c = torch.empty((N, M), dtype=torch.bfloat16, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_gmm_fp8w(_ptr(a), _ptr(b_q), _ptr(b_scale), _ptr(c), _ptr(expert_offsets),
                                    E, N, K, M, 1 if trans_b else 0, _stream(dev))
    _C.check(st, "gmoe_gmm_fp8w")
    return c


def quantize_fp8_rows(x: torch.Tensor):
    """x [N,K] -> (q [N,K] float8_e4m3fn, scales [ceil(K/128), N] int32): one power-of-two scale per row
    and 128 reduction elements, the dword holding its E8M0 byte in all four bytes (see
    gmoe_quantize_fp8_rows in include/galvatron_moe.h).  `row_scale_exponents` decodes the table."""
    assert x.dim() == 2
    x = x.contiguous()
    dev = _check_dev(x)
    N, K = x.shape
    q = torch.empty((N, K), dtype=torch.float8_e4m3fn, device=dev)
    scales = torch.empty(((K + 127) // 128, N), dtype=torch.int32, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_quantize_fp8_rows(_ptr(x), _dt(x), N, K, _ptr(q), _ptr(scales), _stream(dev))
    _C.check(st, "gmoe_quantize_fp8_rows")
    return q, scales


def glu_fwd_quantize_fp8_rows(y: torch.Tensor, act: str = "silu"):
    """quantize_fp8_rows(glu_fwd(y, act)) in one pass, bit for bit; the activation itself is not stored."""
    dev = _check_dev(y)
    assert y.dim() == 2 and y.shape[1] % 16 == 0
    N, F = y.shape[0], y.shape[1] // 2
    q = torch.empty((N, F), dtype=torch.float8_e4m3fn, device=dev)
    scales = torch.empty(((F + 127) // 128, N), dtype=torch.int32, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_glu_fwd_quantize_fp8_rows(_ptr(y), _dt(y), N, F, _ACTS[act], _ptr(q),
                                                     _ptr(scales), _stream(dev))
    _C.check(st, "gmoe_glu_fwd_quantize_fp8_rows")
    return q, scales


def glu_bwd_quantize_fp8_rows(grad_out: torch.Tensor, y: torch.Tensor, act: str = "silu"):
    """quantize_fp8_rows(glu_bwd(grad_out, y, act)) in one pass, bit for bit; F a multiple of 128."""
    dev = _check_dev(grad_out, y)
    N, F2 = y.shape
    assert grad_out.shape == (N, F2 // 2) and grad_out.dtype == y.dtype and (F2 // 2) % 128 == 0
    q = torch.empty((N, F2), dtype=torch.float8_e4m3fn, device=dev)
    scales = torch.empty((F2 // 128, N), dtype=torch.int32, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_glu_bwd_quantize_fp8_rows(_ptr(grad_out), _ptr(y), _dt(y), N, F2 // 2,
                                                     _ACTS[act], _ptr(q), _ptr(scales), _stream(dev))
    _C.check(st, "gmoe_glu_bwd_quantize_fp8_rows")
    return q, scales


def row_scale_exponents(scales: torch.Tensor) -> torch.Tensor:
    """The exponents e (scale = 2^e) of a table from quantize_fp8_rows, as int32 [ceil(K/128), N]."""
    return (scales & 0xFF) - 127


def gmm_fp8a(a_q: torch.Tensor, a_scale: torch.Tensor, b_q: torch.Tensor, b_scale: torch.Tensor,
             expert_offsets: torch.Tensor, trans_b: bool = False) -> torch.Tensor:
    """Grouped GEMM with fp8 on both sides on the block-scaled fp8 MFMA: c[rows_e] (bf16) =
    deq(a_q)[rows_e] @ w[e] (or @ w[e]^T with trans_b); (a_q, a_scale) from quantize_fp8_rows,
    (b_q, b_scale) from quantize_fp8_block.  Any row count; fastest with few rows per expert, where an
    expert's weights are streamed once (see gmoe_gmm_fp8a)."""
    dev = _check_dev(a_q, a_scale, b_q, b_scale, expert_offsets)
    assert a_q.dim() == 2 and a_q.dtype == torch.float8_e4m3fn and b_q.dtype == torch.float8_e4m3fn
    assert a_scale.dtype == torch.int32 and b_scale.dtype == torch.bfloat16
    assert expert_offsets.dtype == torch.int64
    E = expert_offsets.numel() - 1
    N, K = a_q.shape
    assert tuple(a_scale.shape) == ((K + 127) // 128, N)
    assert b_q.dim() == 3 and b_q.shape[0] == E
    M = b_q.shape[1] if trans_b else b_q.shape[2]
    assert (b_q.shape[2] if trans_b else b_q.shape[1]) == K
    assert tuple(b_scale.shape) == (E, (b_q.shape[1] + 127) // 128, (b_q.shape[2] + 127) // 128)
    c = torch.empty((N, M), dtype=torch.bfloat16, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_gmm_fp8a(_ptr(a_q), _ptr(a_scale), _ptr(b_q), _ptr(b_scale), _ptr(c),
                                    _ptr(expert_offsets), E, N, K, M, 1 if trans_b else 0, _stream(dev))
    _C.check(st, "gmoe_gmm_fp8a")
    return c


def capacity_select(probs: torch.Tensor, routing_map: torch.Tensor, capacity: int,
                    by_position: bool = False, pad: bool = False):
    """At most `capacity` tokens per expert (see gmoe_capacity_select in include/galvatron_moe.h).
    Returns (probs * kept [T,E], kept [T,E] bool)."""
    dev = _check_dev(probs, routing_map)
    T, E = probs.shape
    assert routing_map.shape == (T, E) and routing_map.dtype in (torch.bool, torch.uint8)
    assert capacity >= 1
    out_probs = torch.empty_like(probs)
    out_map = torch.empty((T, E), dtype=torch.bool, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_capacity_select(_ptr(probs), _dt(probs), _ptr(routing_map), T, E,
                                           int(capacity), 1 if by_position else 0, 1 if pad else 0,
                                           _ptr(out_probs), _ptr(out_map), _stream(dev))
    _C.check(st, "gmoe_capacity_select")
    return out_probs, out_map


def rmsnorm_fwd(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """y = x * rstd * weight over the last dimension (gmoe_rmsnorm_fwd).  Returns (y, rstd[T] fp32)."""
    dev = _check_dev(x, weight)
    H = x.shape[-1]
    assert weight.shape == (H,) and weight.dtype == x.dtype
    x2 = x.reshape(-1, H)
    T = x2.shape[0]
    y = torch.empty_like(x2)
    rstd = torch.empty((T,), dtype=torch.float32, device=dev)
    with _on(dev):
        st = _C.lib().gmoe_rmsnorm_fwd(_ptr(x2), _ptr(weight), T, H, float(eps), _dt(x2), _ptr(y),
                                       _ptr(rstd), _stream(dev))
    _C.check(st, "gmoe_rmsnorm_fwd")
    return y.view(x.shape), rstd


def rmsnorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor,
                dresidual: Optional[torch.Tensor] = None):
    """(dx, dweight) of rmsnorm_fwd (gmoe_rmsnorm_bwd); `dresidual` [T,H], the gradient arriving at
    x along the residual branch, is added to dx inside the kernel."""
    dev = _check_dev(dy, x, weight, rstd, dresidual)
    if dresidual is not None:
        assert dresidual.dtype == x.dtype and dresidual.numel() == x.numel()
    H = x.shape[-1]
    x2, dy2 = x.reshape(-1, H), dy.reshape(-1, H)
    T = x2.shape[0]
    assert dy2.shape == x2.shape and dy2.dtype == x2.dtype and rstd.shape == (T,)
    assert rstd.dtype == torch.float32
    L = _C.lib()
    rows = L.gmoe_rmsnorm_bwd_workspace_rows(T, H, _dt(x2))
    if rows < 0:
        raise RuntimeError("gmoe_rmsnorm_bwd: unsupported shape T=%d H=%d %s" % (T, H, x.dtype))
    ws = torch.empty((max(rows, 1), H), dtype=torch.float32, device=dev)
    dx = torch.empty_like(x2)
    dw = torch.empty_like(weight)
    with _on(dev):
        st = L.gmoe_rmsnorm_bwd(_ptr(dy2), _ptr(x2), _ptr(weight), _ptr(rstd), _ptr(dresidual), T, H,
                                _dt(x2), _ptr(dx),
                                _ptr(dw), _ptr(ws), rows, _stream(dev))
    _C.check(st, "gmoe_rmsnorm_bwd")
    return dx.view(x.shape), dw


def gate_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the HIP gate projection covers this shape: any expert count up to 4096 (beyond 16
    experts the table is padded to a multiple of 8 rows for the dense products), operands of one
    16- or 32-bit float type, rows of x that are multiples of 16 bytes."""
    H = x.shape[-1]
    E = weight.shape[0]
    return (x.is_cuda and x.dtype == weight.dtype and x.dtype in _DTYPES
            and H % (4 if x.dtype == torch.float32 else 8) == 0
            and (E <= 16 or (H % 8 == 0 and E <= 4096)))


def _gate_padded_experts(E: int) -> int:
    """Beyond 16 experts the projection runs as dense products whose rows are 16-byte multiples:
    the expert count is padded to a multiple of 8 with zero rows of the weight."""
    return E if E <= 16 else (E + 7) // 8 * 8


def _pad_rows(t: torch.Tensor, rows: int) -> torch.Tensor:
    out = t.new_zeros((rows,) + tuple(t.shape[1:]))
    out[: t.shape[0]].copy_(t)
    return out


def _pad_cols(t: torch.Tensor, cols: int) -> torch.Tensor:
    out = t.new_zeros((t.shape[0], cols))
    out[:, : t.shape[1]].copy_(t)
    return out


def gate_fwd(x: torch.Tensor, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None):
    """logits [.., E] = x [.., H] @ weight[E, H]^T (gmoe_gate_fwd); out_dtype = x.dtype or float32."""
    dev = _check_dev(x, weight)
    E, H = weight.shape
    assert x.shape[-1] == H and x.dtype == weight.dtype
    out_dtype = out_dtype or x.dtype
    x2 = x.reshape(-1, H)
    T = x2.shape[0]
    E_real = E
    E = _gate_padded_experts(E)
    if E != E_real:
        weight = _pad_rows(weight, E)
    logits = torch.empty((T, E), dtype=out_dtype, device=dev)
    with _on(dev):
        nbytes = _C.lib().gmoe_gate_fwd_workspace_bytes(T, H, E, _dt(x2))
        if nbytes < 0:
            raise RuntimeError("gmoe_gate_fwd: unsupported shape T=%d H=%d E=%d" % (T, H, E))
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev) if nbytes else None
        st = _C.lib().gmoe_gate_fwd(_ptr(x2), _ptr(weight), T, H, E, _dt(x2), _ptr(logits), _dt(logits),
                                    _ptr(ws), nbytes, _stream(dev))
    _C.check(st, "gmoe_gate_fwd")
    if E != E_real:
        logits = logits[:, :E_real].contiguous()
    return logits.view(*x.shape[:-1], E_real)


def gate_bwd(dlogits: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, need_dx=True, need_dw=True):
    """(dx, dweight) of gate_fwd (gmoe_gate_bwd_input, gmoe_gate_bwd_weight)."""
    dev = _check_dev(dlogits, x, weight)
    E, H = weight.shape
    x2, dl = x.reshape(-1, H), dlogits.reshape(-1, E)
    T = x2.shape[0]
    assert dl.shape[0] == T
    E_real = E
    E = _gate_padded_experts(E)
    if E != E_real:
        # zero weight rows and zero gradient columns for the padding experts: dx is unchanged and the
        # padding rows of dw are dropped
        weight, dl = _pad_rows(weight, E), _pad_cols(dl, E)
    L = _C.lib()
    dx = dw = None
    with _on(dev):
        if need_dx:
            dx = torch.empty_like(x2)
            nbytes = L.gmoe_gate_bwd_input_workspace_bytes(T, H, E, _dt(x2), _dt(dl))
            if nbytes < 0:
                raise RuntimeError("gmoe_gate_bwd_input: unsupported shape T=%d H=%d E=%d" % (T, H, E))
            ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev) if nbytes else None
            st = L.gmoe_gate_bwd_input(_ptr(dl), _dt(dl), _ptr(weight), T, H, E, _dt(x2), _ptr(dx),
                                       _ptr(ws), nbytes, _stream(dev))
            _C.check(st, "gmoe_gate_bwd_input")
            dx = dx.view(x.shape)
        if need_dw:
            rows = L.gmoe_gate_bwd_workspace_rows(T, H, E, _dt(x2))
            if rows < 0:
                raise RuntimeError("gmoe_gate_bwd_weight: unsupported shape T=%d H=%d E=%d" % (T, H, E))
            ws = torch.empty((max(rows, 1), E * H), dtype=torch.float32, device=dev)
            dw = torch.empty_like(weight)
            st = L.gmoe_gate_bwd_weight(_ptr(dl), _dt(dl), _ptr(x2), T, H, E, _dt(x2), _ptr(dw), _ptr(ws),
                                        rows, _stream(dev))
            _C.check(st, "gmoe_gate_bwd_weight")
            if E != E_real:
                dw = dw[:E_real].contiguous()
    return dx, dw
