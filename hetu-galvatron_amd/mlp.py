"""Expert MLPs with the reference's interface (galvatron/core/runtime/moe/mlp.py).

`GroupedMLP` (mlp.py:26-126): weight1 [H, E*2F] viewed [E,H,2F] (gate half first), weight2 [E*F, H]
viewed [E,F,H]; forward(permuted [N,H], tokens_per_expert [E]) -> (out [N,H], None) computed as
grouped GEMM -> gated activation -> grouped GEMM on the HIP kernels.
`SharedExpertMLP` (mlp.py:215-400): a dense gated MLP over all tokens with the reference's
parameters (`linear_fc1.weight [2Fs,H]`, `linear_fc2.weight [H,Fs]`, optional `gate_weight [1,H]`),
run as one group on the grouped kernels, optionally on its own stream beside the routed experts.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch.nn.parameter import Parameter

from . import ops
from .config import MoEConfig
from .grouped_gemm import ops as gg_ops


class _GLU(torch.autograd.Function):
    """act(y[:, :F]) * y[:, F:]  (mlp.py:52-57; backward transformer/fused_kernels.py:157-162)."""

    @staticmethod
    def forward(ctx, y, act):
        ctx.save_for_backward(y)
        ctx.act = act
        return ops.glu_fwd(y, act)

    @staticmethod
    def backward(ctx, grad_out):
        (y,) = ctx.saved_tensors
        return ops.glu_bwd(grad_out.contiguous(), y, ctx.act), None


class _GLUFp8Store(torch.autograd.Function):
    """The same activation with its input kept as float8_e4m3fn for the backward
    (SwiGLUFunction with fp8_input_store, transformer/fused_kernels.py:190-204): a quarter (fp32)
    or half (16-bit) of the saved bytes, the gradient computed on the rounded input."""

    @staticmethod
    def forward(ctx, y, act):
        out, y8 = ops.glu_fwd_fp8store(y, act)
        ctx.save_for_backward(y8)
        ctx.act = act
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (y8,) = ctx.saved_tensors
        return ops.glu_bwd_fp8in(grad_out.contiguous(), y8, ctx.act), None


def glu(y: torch.Tensor, act: str = "silu", fp8_input_store: bool = False) -> torch.Tensor:
    shape = y.shape
    fn = _GLUFp8Store if fp8_input_store else _GLU
    out = fn.apply(y.reshape(-1, shape[-1]).contiguous(), act)
    return out.view(*shape[:-1], shape[-1] // 2)


def swiglu(y: torch.Tensor) -> torch.Tensor:
    """transformer/fused_kernels.py:142-145."""
    return glu(y, "silu")


class _BiasRows(torch.autograd.Function):
    """x [N,M] + bias [M] row by row (x None: the bias alone as `num_rows` rows); the bias gradient
    is the column sum of the incoming gradient."""

    @staticmethod
    def forward(ctx, x, bias, num_rows):
        ctx.has_x = x is not None
        ctx.bias_shape = bias.shape
        return ops.bias_rows(None if x is None else x.contiguous(), bias.contiguous(), num_rows)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        grad_bias = ops.bias_rows_bwd(grad).view(ctx.bias_shape) if ctx.needs_input_grad[1] else None
        return (grad if ctx.has_x else None), grad_bias, None


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """`intermediate_parallel + bias_parallel` (transformer/mlp.py:132-133) on rows [..., M]."""
    shape = x.shape
    return _BiasRows.apply(x.reshape(-1, shape[-1]), bias, None).view(shape)


def expand_bias(bias: torch.Tensor, num_rows: int) -> torch.Tensor:
    """`output_bias.expand_as(output)` (moe/mlp.py:203) as rows of their own, [num_rows, M]."""
    return _BiasRows.apply(None, bias, num_rows)


def bias_swiglu_impl(input, bias, fp8_input_store=False):
    """transformer/fused_kernels.py:207-216: swiglu(input + bias), the sum rounded to the input's
    dtype as the reference's `y + bias` is."""
    if bias is not None:
        input = add_bias(input, bias)
    return glu(input, "silu", fp8_input_store)


class _FusedGatedExperts(torch.autograd.Function):
    """out = gmm(act(gmm(x, w1)[:, :F]) * gmm(x, w1)[:, F:], w2) with the activation fused into the
    first GEMM's epilogue and its backward into the epilogue of the d(act) GEMM
    (same math, op by op, as moe/mlp.py:106-112 and its autograd)."""

    # The fused d(act) GEMM + activation backward gives the same bits as the two launches.  Its
    # epilogue reads fc1 and writes d(fc1) (4 bytes of HBM traffic per accumulator) while the matrix
    # cores of that workgroup's CU idle, which the separate activation-backward kernel at HBM speed
    # nearly makes up for: measured in the same run the fused form is 0.06 ms per step faster on the
    # Mixtral shape (3.55 ms against 2.85 + 0.86 ms in isolation), 0.03 ms slower on the fine-grained
    # one and equal on the DeepSeek-V3-shape shard; it never materialises d(act) (0.94 GB at the
    # Mixtral shape), which decides it.
    fuse_backward = True

    @staticmethod
    def forward(ctx, x, w1, w2, batch_sizes, act):
        offsets = ops.expert_offsets_from_batch_sizes(batch_sizes, x.device)
        x = x.contiguous()
        w1 = w1.contiguous()
        w2 = w2.contiguous()
        fc1, h = ops.gmm_glu(x, w1, offsets, act)
        out = ops.gmm(h, w2, offsets)
        ctx.save_for_backward(x, w1, w2, fc1, h, offsets)
        ctx.act = act
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w1, w2, fc1, h, offsets = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        dx = dw1 = dw2 = None
        if _FusedGatedExperts.fuse_backward:
            dfc1 = ops.gmm_glu_bwd(grad_out, w2, fc1, offsets, ctx.act)
        else:
            dfc1 = ops.glu_bwd(ops.gmm(grad_out, w2, offsets, trans_b=True), fc1, ctx.act)
        if ctx.needs_input_grad[2]:
            dw2 = ops.gmm(h, grad_out, offsets, trans_a=True)
        if ctx.needs_input_grad[0]:
            dx = ops.gmm(dfc1, w1, offsets, trans_b=True)
        if ctx.needs_input_grad[1]:
            dw1 = ops.gmm(x, dfc1, offsets, trans_a=True)
        return dx, dw1, dw2, None, None


def fused_gated_experts(x, w1, w2, batch_sizes, act: str = "silu"):
    """x [N,H], w1 [E,H,2F], w2 [E,F,H], batch_sizes [E] -> [N,H]."""
    return _FusedGatedExperts.apply(x, w1, w2, batch_sizes, act)


class _Fp8GatedExperts(torch.autograd.Function):
    """The gated expert MLP on block-scaled fp8 weights (frozen): forward and the gradient of the
    input only.  Weight layouts are those of GroupedMLP, [E,H,2F] and [E,F,H]; the dX GEMMs read the
    same fp8 tensors with the transposed-operand flag."""

    @staticmethod
    def _gemm(a, w_q, w_scale, offsets, fp8_activations, trans_b=False):
        if fp8_activations:
            # the rows are quantised too (a power-of-two scale per row and 128 elements) and the
            # product runs on the block-scaled fp8 MFMA
            a_q, a_scale = ops.quantize_fp8_rows(a)
            return ops.gmm_fp8a(a_q, a_scale, w_q, w_scale, offsets, trans_b=trans_b)
        return ops.gmm_fp8w(a, w_q, w_scale, offsets, trans_b=trans_b)

    @staticmethod
    def forward(ctx, x, w1_q, w1_scale, w2_q, w2_scale, batch_sizes, act, fp8_activations):
        offsets = ops.expert_offsets_from_batch_sizes(batch_sizes, x.device)
        gemm = _Fp8GatedExperts._gemm
        x = x.contiguous()
        fc1 = gemm(x, w1_q, w1_scale, offsets, fp8_activations)
        if fp8_activations:
            # activation and row quantiser in one pass: the activation is needed as fp8 rows only
            h_q, h_scale = ops.glu_fwd_quantize_fp8_rows(fc1, act)
            out = ops.gmm_fp8a(h_q, h_scale, w2_q, w2_scale, offsets)
        else:
            out = gemm(ops.glu_fwd(fc1, act), w2_q, w2_scale, offsets, False)
        ctx.save_for_backward(w1_q, w1_scale, w2_q, w2_scale, fc1, offsets)
        ctx.act = act
        ctx.fp8_activations = fp8_activations
        return out

    @staticmethod
    def backward(ctx, grad_out):
        w1_q, w1_scale, w2_q, w2_scale, fc1, offsets = ctx.saved_tensors
        gemm = _Fp8GatedExperts._gemm
        dact = gemm(grad_out.contiguous(), w2_q, w2_scale, offsets, ctx.fp8_activations, trans_b=True)
        if ctx.fp8_activations and (fc1.shape[1] // 2) % 128 == 0:
            d_q, d_scale = ops.glu_bwd_quantize_fp8_rows(dact, fc1, ctx.act)
            dx = ops.gmm_fp8a(d_q, d_scale, w1_q, w1_scale, offsets, trans_b=True)
        else:
            dx = gemm(ops.glu_bwd(dact, fc1, ctx.act), w1_q, w1_scale, offsets, ctx.fp8_activations,
                      trans_b=True)
        return dx, None, None, None, None, None, None, None


def fp8_gated_experts(x, w1_q, w1_scale, w2_q, w2_scale, batch_sizes, act: str = "silu",
                      fp8_activations: bool = False):
    """x [N,H] bf16; (w1_q [E,H,2F], w1_scale) and (w2_q [E,F,H], w2_scale) from
    ops.quantize_fp8_block; batch_sizes [E] -> [N,H] bf16.  `fp8_activations`: the rows entering each
    of the four products are quantised to fp8 as well (ops.quantize_fp8_rows) and the products run on
    the fp8 MFMA; off by default, where the bf16 rows are multiplied with the exactly widened weights."""
    return _Fp8GatedExperts.apply(x, w1_q, w1_scale, w2_q, w2_scale, batch_sizes, act, fp8_activations)


def _act_name(config: MoEConfig) -> str:
    if config.activation_func in (F.silu, "silu", "swiglu"):
        return "silu"
    if config.activation_func in (F.gelu, "gelu", "geglu"):
        return "gelu"
    raise ValueError("Activation function must be silu or gelu when using GroupedMLP.")


class GroupedMLP(torch.nn.Module):
    """All local experts in two grouped GEMMs."""

    def __init__(self, num_local_experts: int, config: MoEConfig, tp_of_ep_group=None,
                 layer_idx: int = None, device=None):
        super().__init__()
        self.config = config
        self.num_local_experts = num_local_experts
        assert config.add_bias_linear is False, \
            "bias not supported in Grouped GEMM yet, please set '--disable-bias-linear' instead."
        assert tp_of_ep_group is None, "expert tensor parallelism needs collectives (single GPU build)"
        assert config.gated_linear_unit, "GroupedMLP here implements the gated (SwiGLU / GeGLU) MLP"
        self.act = _act_name(config)
        device = torch.cuda.current_device() if device is None else device
        fc1_out = config.moe_ffn_hidden_size * num_local_experts * 2
        fc2_in = config.moe_ffn_hidden_size * num_local_experts
        self.weight1 = Parameter(torch.empty(config.hidden_size, fc1_out, device=device,
                                             dtype=config.params_dtype))
        self.weight2 = Parameter(torch.empty(fc2_in, config.hidden_size, device=device,
                                             dtype=config.params_dtype))
        self.layer_idx = layer_idx
        # True: activation fused into the GEMM epilogues; False: the reference's three-op sequence
        self.fuse_activation = True
        self.reset_parameters()

    def reset_parameters(self):
        std = self.config.init_method_std
        torch.nn.init.normal_(self.weight1, mean=0.0, std=std)
        torch.nn.init.normal_(self.weight2, mean=0.0, std=std)

    def forward(self, permuted_local_hidden_states: torch.Tensor, tokens_per_expert: torch.Tensor):
        E, H = self.num_local_experts, self.config.hidden_size
        w1 = self.weight1.view(E, H, -1)
        w2 = self.weight2.view(E, -1, H)
        if permuted_local_hidden_states.nelement() != 0 and self.fuse_activation:
            fc2_output = fused_gated_experts(permuted_local_hidden_states, w1, w2, tokens_per_expert,
                                             self.act)
        elif permuted_local_hidden_states.nelement() != 0:
            fc1_output = gg_ops.gmm(permuted_local_hidden_states, w1, tokens_per_expert, trans_b=False)
            intermediate = glu(fc1_output, self.act)
            fc2_output = gg_ops.gmm(intermediate, w2, tokens_per_expert, trans_b=False)
        else:
            # no token for the local experts: keep the parameters in the graph (mlp.py:113-124)
            h = torch.matmul(permuted_local_hidden_states, self.weight1.view(H, -1))
            half = h.shape[-1] // 2
            h = F.silu(h[:, :half]) * h[:, half:]
            fc2_output = torch.matmul(h, self.weight2.view(-1, H))
        return fc2_output, None


class Fp8GroupedMLP(torch.nn.Module):
    """GroupedMLP with frozen, block-scaled fp8 (e4m3) expert weights: same forward signature,
    gradients flow to the input only.  The reference has the fp8 expert path commented out
    (mlp.py:164-184); the weight format is the one of ops.quantize_fp8_block."""

    def __init__(self, mlp: GroupedMLP, fp8_activations: bool = False):
        super().__init__()
        self.config = mlp.config
        self.num_local_experts = mlp.num_local_experts
        self.act = mlp.act
        # also quantise the rows entering each product and run them on the fp8 MFMA (see ops.gmm_fp8a)
        self.fp8_activations = fp8_activations
        E, H = mlp.num_local_experts, mlp.config.hidden_size
        with torch.no_grad():
            w1_q, w1_s = ops.quantize_fp8_block(mlp.weight1.detach().view(E, H, -1))
            w2_q, w2_s = ops.quantize_fp8_block(mlp.weight2.detach().view(E, -1, H))
        for name, t in (("weight1_q", w1_q), ("weight1_scale", w1_s), ("weight2_q", w2_q),
                        ("weight2_scale", w2_s)):
            self.register_buffer(name, t)

    def forward(self, permuted_local_hidden_states: torch.Tensor, tokens_per_expert: torch.Tensor):
        if permuted_local_hidden_states.nelement() == 0:
            return permuted_local_hidden_states.new_zeros(permuted_local_hidden_states.shape), None
        out = fp8_gated_experts(permuted_local_hidden_states, self.weight1_q, self.weight1_scale,
                                self.weight2_q, self.weight2_scale, tokens_per_expert, self.act,
                                self.fp8_activations)
        return out, None


class _Linear(torch.nn.Module):
    """`weight [out, in]`, y = x @ weight^T, the layout of the reference's expert
    Column/RowParallelLinear (tensor_parallel/layers.py:547-988) at tensor-parallel size 1.  With
    `config.add_bias_linear` it carries `bias [out]` (zero-initialised, as there) and, like those
    layers under `skip_bias_add=True` (transformer/mlp.py:71, 87), does not add it: the caller does."""

    def __init__(self, in_features: int, out_features: int, config: MoEConfig, device):
        super().__init__()
        self.weight = Parameter(torch.empty(out_features, in_features, device=device,
                                            dtype=config.params_dtype))
        torch.nn.init.normal_(self.weight, mean=0.0, std=config.init_method_std)
        if config.add_bias_linear:
            self.bias = Parameter(torch.zeros(out_features, device=device, dtype=config.params_dtype))
        else:
            self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # one group holding every row: the grouped GEMM with the transposed-operand flag; the
        # one-entry offset table lives on the device and is built once per row count
        return gg_ops.gmm(x, self.weight.unsqueeze(0), ops.one_group(x.shape[0], x.device), trans_b=True)


class ExpertMLP(torch.nn.Module):
    """One expert of SequentialMLP: linear_fc1 [2F, H] (gate rows first, then up rows), gated
    activation, linear_fc2 [H, F]  (transformer/mlp.py:23-134 with is_expert=True)."""

    def __init__(self, config: MoEConfig, device=None):
        super().__init__()
        assert config.gated_linear_unit
        self.act = _act_name(config)
        H, Fe = config.hidden_size, config.moe_ffn_hidden_size
        self.linear_fc1 = _Linear(H, 2 * Fe, config, device)
        self.linear_fc2 = _Linear(Fe, H, config, device)

    def forward(self, hidden_states: torch.Tensor):
        """Returns (output, output_bias): with `add_bias_linear` the fc1 bias is added in front of the
        activation and the fc2 bias is handed back un-added, [H] (transformer/mlp.py:104-138)."""
        fc2_bias = self.linear_fc2.bias
        if hidden_states.shape[0] == 0:
            keep = self.linear_fc1.weight.sum() + self.linear_fc2.weight.sum()
            if self.linear_fc1.bias is not None:
                keep = keep + self.linear_fc1.bias.sum()
            return hidden_states.new_zeros(hidden_states.shape) + 0.0 * keep, fc2_bias
        fc1 = self.linear_fc1(hidden_states)
        if self.linear_fc1.bias is not None:
            fc1 = add_bias(fc1, self.linear_fc1.bias)
        return self.linear_fc2(glu(fc1, self.act)), fc2_bias


class SequentialMLP(torch.nn.Module):
    """The experts one after the other, each on its slice of the permuted rows (mlp.py:128-211):
    `local_experts[i].linear_fc1.weight [2F,H]`, `.linear_fc2.weight [H,F]`."""

    def __init__(self, num_local_experts: int, config: MoEConfig, tp_of_ep_group=None,
                 tp_and_ep_group=None, layer_idx: int = None, device=None):
        super().__init__()
        assert tp_of_ep_group is None and tp_and_ep_group is None, \
            "expert tensor parallelism needs collectives (single GPU build)"
        self.config = config
        self.add_bias = config.add_bias_linear
        self.num_local_experts = num_local_experts
        device = torch.cuda.current_device() if device is None else device
        self.local_experts = torch.nn.ModuleList(
            [ExpertMLP(config, device=device) for _ in range(num_local_experts)])
        self.layer_idx = layer_idx

    def forward(self, permuted_local_hidden_states: torch.Tensor, tokens_per_expert: torch.Tensor):
        """Returns (output, output_bias); with `add_bias_linear` output_bias holds, row by row, the
        fc2 bias of the row's expert (mlp.py:200-207), which the dispatcher weights and combines
        like the output; with a single local expert it is that expert's [H] bias (mlp.py:184-186)."""
        if self.num_local_experts == 1:
            return self.local_experts[0](permuted_local_hidden_states)
        counts = tokens_per_expert.tolist()  # one host read, as in the reference (mlp.py:188)
        rows, total = permuted_local_hidden_states.shape[0], sum(counts)
        tokens_list = torch.split(permuted_local_hidden_states[:total], counts)
        outs, biases = [], []
        for expert, tokens in zip(self.local_experts, tokens_list):
            out, out_bias = expert(tokens)
            outs.append(out)
            if self.add_bias:
                biases.append(expand_bias(out_bias, tokens.shape[0]))
        if total < rows:  # the dispatcher sized the buffer by an upper bound: unused rows stay zero
            pad = permuted_local_hidden_states.new_zeros(rows - total, outs[0].shape[1])
            outs.append(pad)
            if self.add_bias:
                biases.append(pad)
        return torch.cat(outs, dim=0), (torch.cat(biases, dim=0) if self.add_bias else None)


class SharedExpertMLP(torch.nn.Module):
    """Dense gated MLP applied to every token (mlp.py:215-400), width
    `moe_shared_expert_intermediate_size`, with the reference's parameter names and layouts:
    `linear_fc1.weight [2Fs, H]` (gate rows first, then up rows), `linear_fc2.weight [H, Fs]`,
    `gate_weight [1, H]` when `gate` (output * sigmoid(x . gate_weight), mlp.py:271-278).

    With `config.moe_shared_expert_overlap` the reference's staged interface is available
    (pre_forward_comm, linear_fc1_forward_and_act, linear_fc2_forward, post_forward_comm,
    get_output): the stages enqueue on a stream of the class, so the dense products run beside
    the dispatch and the routed experts, and get_output makes the current stream wait for them."""

    stream = None  # shared by all instances, default priority

    def __init__(self, config: MoEConfig, gate: bool = False, device=None):
        super().__init__()
        self.config = config
        assert config.add_bias_linear is False, "bias is not supported in the shared experts"
        assert config.gated_linear_unit, "the shared experts here are a gated (SwiGLU / GeGLU) MLP"
        self.act = _act_name(config)
        Fs = config.moe_shared_expert_intermediate_size
        assert Fs is not None
        device = torch.cuda.current_device() if device is None else device
        H = config.hidden_size
        self.linear_fc1 = _Linear(H, 2 * Fs, config, device)
        self.linear_fc2 = _Linear(Fs, H, config, device)
        self.use_shared_expert_gate = gate
        self.gate_weight = None
        if gate:
            self.gate_weight = Parameter(torch.empty(1, H, device=device, dtype=config.params_dtype))
            torch.nn.init.normal_(self.gate_weight, mean=0.0, std=config.init_method_std)
        self.overlap = bool(getattr(config, "moe_shared_expert_overlap", False))
        self._staged = {}
        if self.overlap and SharedExpertMLP.stream is None:
            SharedExpertMLP.stream = torch.cuda.Stream(device=device)

    # -- the three pieces of the forward ----------------------------------------------------------
    def _gate_score(self, x2d):
        from .router import _GateProjection  # the one-expert case of the gate projection kernels

        w = self.gate_weight if self.gate_weight.dtype == x2d.dtype else self.gate_weight.to(x2d.dtype)
        if not ops.gate_supported(x2d, w):
            raise ValueError("shared-expert gate: unsupported operands (dtype %s, hidden size %d)"
                             % (x2d.dtype, x2d.shape[-1]))
        logits = _GateProjection.apply(x2d, w, x2d.dtype)
        return torch.sigmoid(logits)

    def _fc1_act(self, x2d):
        # the SwiGLU input goes to the backward as fp8 where the reference's fused branch would
        # store it so (mlp.py:316-330: bias_activation_fusion, SiLU, activation_func_fp8_input_store)
        cfg = self.config
        fp8 = (getattr(cfg, "bias_activation_fusion", False) and self.act == "silu"
               and getattr(cfg, "activation_func_fp8_input_store", False))
        return glu(self.linear_fc1(x2d), self.act, fp8)

    def _finish(self, fc2_out, gate_score):
        if gate_score is None:
            return fc2_out
        from .moe_utils import scale_rows

        return scale_rows(fc2_out, gate_score)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        shape = hidden_states.shape
        x = hidden_states.reshape(-1, shape[-1]).contiguous()
        score = self._gate_score(x) if self.use_shared_expert_gate else None
        out = self._finish(self.linear_fc2(self._fc1_act(x)), score)
        return out.view(shape)

    # -- staged interface (mlp.py:280-400) ----------------------------------------------------------
    def pre_forward_comm(self, input):
        assert self.overlap, "stages out of order"
        # a forward that raised between two stages leaves its pieces behind: start afresh
        self._staged = {}
        side = SharedExpertMLP.stream
        side.wait_stream(torch.cuda.current_stream())
        self._staged = {"shape": input.shape}
        with torch.cuda.stream(side):
            x = input.reshape(-1, input.shape[-1]).contiguous()
            x.record_stream(side)
            self._staged["x"] = x
            self._staged["score"] = self._gate_score(x) if self.use_shared_expert_gate else None

    def linear_fc1_forward_and_act(self, overlapped_comm_output=None):
        assert self.overlap and "x" in self._staged, "stages out of order"
        with torch.cuda.stream(SharedExpertMLP.stream):
            self._staged["act"] = self._fc1_act(self._staged.pop("x"))

    def linear_fc2_forward(self, overlapped_comm_output=None):
        assert self.overlap and "act" in self._staged, "stages out of order"
        with torch.cuda.stream(SharedExpertMLP.stream):
            self._staged["fc2"] = self.linear_fc2(self._staged.pop("act"))

    def post_forward_comm(self):
        assert self.overlap and "fc2" in self._staged, "stages out of order"  # no collective at TP 1

    def get_output(self):
        assert self.overlap and "fc2" in self._staged, "stages out of order"
        st = self._staged
        self._staged = {}
        with torch.cuda.stream(SharedExpertMLP.stream):
            out = self._finish(st["fc2"], st["score"]).view(st["shape"])
        cur = torch.cuda.current_stream()
        cur.wait_stream(SharedExpertMLP.stream)
        out.record_stream(cur)
        return out
