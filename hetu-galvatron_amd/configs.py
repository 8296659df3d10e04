"""The benchmark / parity workloads and their seeded synthetic inputs.

Inputs are drawn from a CPU generator in fp32 in a fixed order (x, w_r, w1, w2, dy, extras) and then
cast, so a CPU checker and the GPU path see identical bits.  Activations ~ N(0,1), every weight ~
N(0, 0.02) (`init_method_std`, args_schema.py:243).  Token index = s*B + b for x [S,B,H].
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    tokens: int
    hidden: int
    ffn: int
    experts: int
    topk: int
    dtype: torch.dtype
    batch: int = 1
    shared_ffn: Optional[int] = None   # total width of the shared experts
    zipf: Optional[float] = None       # per-expert logit bias giving Zipf(s) loads
    empty_experts: int = 0             # experts forced to receive no token
    global_experts: Optional[int] = None  # C5: experts in the whole EP group
    fp8_weights: bool = False

    @property
    def routed_rows(self) -> int:
        return self.tokens * self.topk

    def gemm_flops(self, fwd_only: bool = False, dx_only: bool = False) -> float:
        """Grouped-GEMM FLOPs: forward 6*N*H*F, backward twice that (dX + dW per GEMM)."""
        n = self.routed_rows
        fwd = 6.0 * n * self.hidden * self.ffn
        if self.shared_ffn:
            fwd += 6.0 * self.tokens * self.hidden * self.shared_ffn
        if fwd_only:
            return fwd
        if dx_only:
            return 2.0 * fwd
        return 3.0 * fwd

    def permute_bytes(self) -> float:
        """(T + N) * H * sizeof + 8 * N: read each token row once, write N rows and the indices."""
        es = torch.finfo(self.dtype).bits // 8
        return (self.tokens + self.routed_rows) * self.hidden * es + 8.0 * self.routed_rows

    def unpermute_bytes(self) -> float:
        es = torch.finfo(self.dtype).bits // 8
        return (self.tokens + self.routed_rows) * self.hidden * es + 12.0 * self.routed_rows


WORKLOADS = {
    # the five benchmark configurations: CPU-runnable, Mixtral 8x7B, fine-grained, skewed, DeepSeek-V3 shard
    "tiny": Workload("tiny", 2048, 512, 1024, 8, 2, torch.float32, batch=2),
    "mixtral": Workload("mixtral", 16384, 4096, 14336, 8, 2, torch.bfloat16, batch=4),
    "finegrained": Workload("finegrained", 8192, 2048, 1408, 64, 8, torch.bfloat16, batch=1,
                            shared_ffn=4 * 1408),
    "mixtral_skew": Workload("mixtral_skew", 16384, 4096, 14336, 8, 2, torch.bfloat16, batch=4,
                             zipf=1.2, empty_experts=1),
    "dsv3_shard": Workload("dsv3_shard", 4096, 7168, 2048, 32, 8, torch.bfloat16, batch=1,
                           global_experts=256, fp8_weights=True),
    # the reference's own test model (tests/utils/model_configs/mixtral-test.yaml:3-27)
    "mixtral_test": Workload("mixtral_test", 64, 128, 256, 4, 2, torch.bfloat16, batch=2),
}


def scaled(w: Workload, tokens: int = None, ffn: int = None, hidden: int = None) -> Workload:
    """The same workload at a reduced size (for checkers that must finish in seconds)."""
    return replace(w, tokens=tokens or w.tokens, ffn=ffn or w.ffn, hidden=hidden or w.hidden)


def zipf_logit_bias(experts: int, s: float, empty: int, tau: float = 1.0) -> torch.Tensor:
    """b_e = tau * ln p_e with p_e ~ rank^-s; the last `empty` experts get -1e4 (never selected)."""
    ranks = torch.arange(1, experts + 1, dtype=torch.float32)
    p = ranks.pow(-s)
    p = p / p.sum()
    b = tau * p.log()
    if empty:
        b[experts - empty:] = -1e4
    return b


def make_inputs(w: Workload, seed: int = 1234, device="cpu", with_weights: bool = True):
    """Returns a dict of tensors in w.dtype on `device`:
    x [S,B,H], w_r [E,H], w1 [E,H,2F], w2 [E,F,H], dy [S,B,H] (+ logit_bias [E], shared_w1/2)."""
    g = torch.Generator().manual_seed(seed)
    S = w.tokens // w.batch
    out = {}
    out["x"] = torch.randn(S, w.batch, w.hidden, generator=g)
    out["w_r"] = 0.02 * torch.randn(w.experts, w.hidden, generator=g)
    if with_weights:
        out["w1"] = 0.02 * torch.randn(w.experts, w.hidden, 2 * w.ffn, generator=g)
        out["w2"] = 0.02 * torch.randn(w.experts, w.ffn, w.hidden, generator=g)
    out["dy"] = torch.randn(S, w.batch, w.hidden, generator=g)
    if w.shared_ffn and with_weights:
        out["shared_w1"] = 0.02 * torch.randn(w.hidden, 2 * w.shared_ffn, generator=g)
        out["shared_w2"] = 0.02 * torch.randn(w.shared_ffn, w.hidden, generator=g)
    out = {k: v.to(w.dtype).to(device) for k, v in out.items()}
    if w.zipf:
        # logits = x @ w_r^T have std 0.02 * sqrt(H); the bias is scaled to that spread.  0.85 is
        # the factor for which the realised top-2 loads of the Mixtral shape are closest to
        # Zipf(1.2) (mean |log ratio| 0.13; a token picks two distinct experts, so no load can
        # exceed half of the routed rows)
        tau = 0.02 * math.sqrt(w.hidden) * 0.85
        out["logit_bias"] = zipf_logit_bias(w.experts, w.zipf, w.empty_experts, tau).to(device)
    return out


def multinomial_counts(total_rows: int, experts: int, seed: int = 1234, empty: int = 2) -> torch.Tensor:
    """tokens_per_expert for a one-GPU share of a larger expert-parallel group: `total_rows` rows
    spread multinomially over the local experts, `empty` of which are forced to zero."""
    g = torch.Generator().manual_seed(seed)
    p = torch.ones(experts)
    if empty:
        p[torch.randperm(experts, generator=g)[:empty]] = 0
    idx = torch.multinomial(p / p.sum(), total_rows, replacement=True, generator=g)
    return torch.bincount(idx, minlength=experts).to(torch.int64)
