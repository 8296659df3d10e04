"""`grouped_gemm.ops.gmm`: differentiable grouped GEMM (call sites moe/mlp.py:106-112)."""
import torch

from .. import ops as _ops


class GroupedGemm(torch.autograd.Function):
    """out[rows_e] = a[rows_e] @ op(b[e]); dA is the same product against the transposed weights,
    dB[e] = a[rows_e]^T @ grad[rows_e] (zeros for an expert without rows)."""

    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b):
        offsets = _ops.expert_offsets_from_batch_sizes(batch_sizes, a.device)
        a = a.contiguous()
        b = b.contiguous()
        ctx.save_for_backward(a, b, offsets)
        ctx.trans_b = trans_b
        return _ops.gmm(a, b, offsets, trans_a=False, trans_b=trans_b)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, offsets = ctx.saved_tensors
        trans_b = ctx.trans_b
        agrad = bgrad = None
        if ctx.needs_input_grad[0]:
            agrad = _ops.gmm(grad, b, offsets, trans_a=False, trans_b=not trans_b)
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if trans_b else (a, grad)
            bgrad = _ops.gmm(lhs, rhs, offsets, trans_a=True, trans_b=False)
        return agrad, bgrad, None, None


def gmm(a, b, batch_sizes, trans_b=False):
    return GroupedGemm.apply(a, b, batch_sizes, trans_b)
