"""The gated activation with its input kept as float8_e4m3fn for the backward
(SwiGLUFunction with fp8_input_store, transformer/fused_kernels.py:190-204; used by the shared
experts at moe/mlp.py:316-330) on the GPU through the C ABI: the stored bytes against torch's own
cast on the CPU (the reference's call), the backward against the plain kernel on the widened input."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def fp8_bytes(t):
    return t.view(torch.uint8)


def test_stored_bytes_equal_the_cast_on_every_bf16_value(pkg, dev):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    y = bits.view(torch.bfloat16).view(256, 256).contiguous()
    out, y8 = pkg.ops.glu_fwd_fp8store(y.to(dev), "silu")
    want = y.to(torch.float8_e4m3fn)
    assert y8.dtype == torch.float8_e4m3fn and y8.shape == (256, 256)
    assert torch.equal(fp8_bytes(y8.cpu()), fp8_bytes(want))
    # the forward value does not see the cast
    ref = pkg.ops.glu_fwd(y.to(dev), "silu")
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,F", [(300, 128), (7, 12), (64, 1032)])   # (7, 12): rows without 16-byte pieces
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_cast_and_backward_on_random_values(pkg, orc, dev, dtype, N, F, act):
    g = torch.Generator().manual_seed(N + F)
    y = torch.randn(N, 2 * F, generator=g) * 4
    # ties of the fp8 grid, the range limit and beyond, subnormals, signed zeros, NaN
    special = torch.tensor([17.0, 19.0, -17.0, 448.0, 464.0, 465.0, -470.0, 1e4, 2.0 ** -9, 2.0 ** -10,
                            3 * 2.0 ** -10, -0.0, 0.0, float("nan"), 0.0703125, -0.0732421875])
    y.view(-1)[: special.numel()] = special
    y = y.to(dtype)
    go = torch.randn(N, F, generator=g).to(dtype)
    out, y8 = pkg.ops.glu_fwd_fp8store(y.to(dev), act)
    assert torch.equal(fp8_bytes(y8.cpu()), fp8_bytes(y.to(torch.float8_e4m3fn)))
    ref = pkg.ops.glu_fwd(y.to(dev), act)
    assert torch.equal(out.view(torch.uint8), ref.view(torch.uint8))   # NaN == NaN bytewise
    # backward: the plain kernel on the widened bytes gives the same bits
    dy = pkg.ops.glu_bwd_fp8in(go.to(dev), y8, act)
    wide = y8.to(dtype)
    assert torch.equal(wide.cpu().view(torch.uint8), y.to(torch.float8_e4m3fn).to(dtype).view(torch.uint8))
    dy_ref = pkg.ops.glu_bwd(go.to(dev), wide, act)
    # (NaN inputs give NaN gradients on both sides, whatever their payload bits)
    assert dy.dtype == dtype and torch.equal(torch.isnan(dy), torch.isnan(dy_ref))
    assert torch.equal(torch.nan_to_num(dy, nan=0.0), torch.nan_to_num(dy_ref, nan=0.0))
    if act == "silu":
        # and the oracle's autograd of the reference's function, away from the NaN inputs
        yo = y.clone().float()
        yo[torch.isnan(yo) | (yo.abs() > 464)] = 1.0
        yo = yo.to(dtype).requires_grad_(True)
        orc.swiglu_fp8_input_store(yo).backward(go)
        mine = pkg.ops.glu_bwd_fp8in(go.to(dev), pkg.ops.glu_fwd_fp8store(yo.detach().to(dev), act)[1], act)
        tol = dict(rtol=2e-2, atol=1e-2) if dtype != torch.float32 else dict(rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(mine.cpu().float(), yo.grad.float(), **tol)


def test_autograd_function_and_shared_experts(pkg, orc, dev):
    """glu(..., fp8_input_store=True) saves one byte per element; the shared experts take that path
    under the reference's conditions and their gradients follow the oracle's."""
    g = torch.Generator().manual_seed(9)
    y = (torch.randn(4, 50, 64, generator=g) * 2).bfloat16().to(dev).requires_grad_(True)
    out = pkg.mlp.bias_swiglu_impl(y, None, True)
    assert out.shape == (4, 50, 32)
    saved = out.grad_fn.saved_tensors if hasattr(out.grad_fn, "saved_tensors") else None
    go = torch.randn(4, 50, 32, generator=g).bfloat16().to(dev)
    out.backward(go)
    yo = y.detach().cpu().view(-1, 64).requires_grad_(True)
    orc.swiglu_fp8_input_store(yo).backward(go.cpu().view(-1, 32))
    torch.testing.assert_close(y.grad.cpu().view(-1, 64).float(), yo.grad.float(), rtol=2e-2, atol=1e-2)
    assert saved is None or all(t.dtype == torch.float8_e4m3fn for t in saved)

    H, Fs, T = 128, 192, 320
    cfg = pkg.MoEConfig(hidden_size=H, moe_shared_expert_intermediate_size=Fs, params_dtype=torch.bfloat16,
                        bias_activation_fusion=True, activation_func_fp8_input_store=True)
    m = pkg.SharedExpertMLP(cfg, device=dev)
    with torch.no_grad():
        m.linear_fc1.weight.copy_((torch.randn(2 * Fs, H, generator=g) / H ** 0.5).to(dev))
        m.linear_fc2.weight.copy_((torch.randn(H, Fs, generator=g) / Fs ** 0.5).to(dev))
    x = torch.randn(T, H, generator=g).bfloat16()
    gy = torch.randn(T, H, generator=g).bfloat16()
    xg = x.to(dev).requires_grad_(True)
    o = m(xg)
    o.backward(gy.to(dev))
    # oracle: the same MLP with the reference's function in the middle; fp32 math on values rounded
    # to bf16 where the kernels store them (fc1, the activation), so the fp8 bytes are the same
    def stored(t):
        return t + (t.bfloat16().float() - t).detach()

    xo = x.float().requires_grad_(True)
    w1 = m.linear_fc1.weight.detach().cpu().float().requires_grad_(True)
    w2 = m.linear_fc2.weight.detach().cpu().float().requires_grad_(True)
    fc1 = stored(torch.nn.functional.linear(xo, w1))
    ref = torch.nn.functional.linear(stored(orc.swiglu_fp8_input_store(fc1)), w2)
    ref.backward(gy.float())
    tol = dict(rtol=2e-2, atol=1e-2)
    torch.testing.assert_close(o.detach().cpu().float(), ref.detach().float(), **tol)
    torch.testing.assert_close(xg.grad.cpu().float(), xo.grad.float(), **tol)
    for mine, want in ((m.linear_fc1.weight.grad, w1.grad), (m.linear_fc2.weight.grad, w2.grad)):
        torch.testing.assert_close(mine.cpu().float(), want.float(), rtol=2e-2,
                                   atol=2e-2 * want.float().abs().max().item())
