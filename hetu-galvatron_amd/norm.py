"""RMS normalisation in front of the router, on the HIP kernels.

The reference builds its norms through `GalvatronNorm(config, hidden_size, eps)`
(galvatron/core/runtime/transformer/norm.py:6-30), which for `normalization == "RMSNorm"` returns
`flash_attn.ops.rms_norm.RMSNorm(hidden_size, eps, device, dtype)`; `GalvatronMoEAttention`
applies one as `pre_router_norm` right before the router and hands the un-normalised tensor on
as the MLP residual (galvatron/core/runtime/models/moe_modules.py:24-30).  This module has the
same constructor arguments, parameter name (`weight`, initialised to ones, no bias) and forward
value: y = x * rsqrt(mean(x^2) + eps) * weight in fp32, rounded once to the input dtype.
"""
import torch

from . import ops


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        x = x.contiguous()
        y, rstd = ops.rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, rstd = ctx.saved_tensors
        dx, dw = ops.rmsnorm_bwd(dy.contiguous(), x, weight, rstd)
        return dx, dw, None


class _RMSNormWithResidual(torch.autograd.Function):
    """(norm(x), x): the fork at models/moe_modules.py:27-29.  One backward kernel takes the gradient
    of the normalised branch and adds the gradient of the residual branch, with the roundings of the
    separate add autograd would run."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        x = x.contiguous()
        y, rstd = ops.rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, weight, rstd)
        ctx.set_materialize_grads(False)
        return y, x.view_as(x)

    @staticmethod
    def backward(ctx, dy, dres):
        x, weight, rstd = ctx.saved_tensors
        if dy is None:
            return dres, None, None
        dx, dw = ops.rmsnorm_bwd(dy.contiguous(), x, weight, rstd,
                                 None if dres is None else dres.contiguous())
        return dx, dw, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor, epsilon: float) -> torch.Tensor:
    """`flash_attn.ops.rms_norm.rms_norm(x, weight, epsilon)`: normalise the last dimension."""
    assert x.shape[-1] == weight.shape[0], "weight must have the size of the last dimension"
    return _RMSNorm.apply(x, weight, epsilon)


class RMSNorm(torch.nn.Module):
    """Constructor and attributes of `flash_attn.ops.rms_norm.RMSNorm`."""

    def __init__(self, hidden_size, eps=1e-5, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(hidden_size, device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, x):
        return rms_norm(x, self.weight, self.eps)


class GalvatronNorm:
    """transformer/norm.py:6-30: a factory keyed by `config.normalization`.  Only the RMSNorm
    branch lies on the MoE path; "LayerNorm" (flash-attn's DropoutAddLayerNorm there) is refused."""

    def __new__(cls, config, hidden_size: int, eps: float = 1e-5):
        kind = getattr(config, "normalization", "RMSNorm")
        if kind == "RMSNorm":
            device = torch.cuda.current_device() if torch.cuda.is_available() else None
            return RMSNorm(hidden_size=hidden_size, eps=eps, device=device,
                           dtype=getattr(config, "params_dtype", None))
        if kind == "LayerNorm":
            raise NotImplementedError("LayerNorm is outside the MoE path built here; use RMSNorm")
        raise Exception("Only LayerNorm and RMSNorm are curently supported")


class PreRouterNorm(torch.nn.Module):
    """The tail of `GalvatronMoEAttention.forward` (models/moe_modules.py:26-30): returns
    (pre_router_norm(hidden_states), hidden_states) = (router / expert input, MLP residual)."""

    def __init__(self, config, device=None):
        super().__init__()
        self.pre_router_norm = RMSNorm(config.hidden_size, getattr(config, "norm_epsilon", 1e-5),
                                       device=device, dtype=getattr(config, "params_dtype", None))

    def forward(self, hidden_states):
        n = self.pre_router_norm
        return _RMSNormWithResidual.apply(hidden_states, n.weight, n.eps)
