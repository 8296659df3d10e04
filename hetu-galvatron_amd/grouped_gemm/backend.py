"""`grouped_gemm.backend.gmm`: the non-differentiable grouped GEMM."""
import torch

from .. import ops as _ops


def gmm(a, b, batch_sizes, trans_a=False, trans_b=False, c=None):
    """a [N,K] @ b per group.  trans_a: returns [E,K,M] = a_e^T @ b_e with b [N,M]; otherwise b is
    [E,K,M] ([E,M,K] if trans_b) and the result is [N,M].  batch_sizes: int64 [E], host or device."""
    offsets = _ops.expert_offsets_from_batch_sizes(batch_sizes, a.device)
    out = _ops.gmm(a.contiguous(), b.contiguous(), offsets, trans_a=trans_a, trans_b=trans_b)
    if c is not None:
        c.copy_(out)
        return c
    return out
