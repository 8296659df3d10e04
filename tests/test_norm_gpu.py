"""Pre-router RMS normalisation on the GPU through the C ABI, against the oracle (fp32 formula,
one rounding) and torch autograd of it."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
       torch.float16: dict(rtol=2e-3, atol=2e-3)}

SHAPES = [  # T, H
    (64, 128),       # the reference's test model
    (1, 8),          # one row, one vector
    (37, 2056),      # ragged: rows not a multiple of the row group, H not a multiple of 256 vectors
    (1000, 4096),    # Mixtral hidden size
    (300, 7168),     # DeepSeek-V3 hidden size
    (5000, 2048),    # more row groups than the backward grid
    (19, 8192),
]


def reference(orc, x, w, dy, eps):
    xo = x.float().requires_grad_(True)
    wo = w.float().requires_grad_(True)
    y = orc.rms_norm(xo, wo, eps)
    y.backward(dy.float())
    return y.detach(), xo.grad, wo.grad


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("T,H", SHAPES)
def test_rms_norm_forward_backward(pkg, orc, dev, dtype, T, H):
    g = torch.Generator().manual_seed(T + H)
    x = (2.0 * torch.randn(T, H, generator=g) + 0.25).to(dtype)
    w = (1.0 + 0.2 * torch.randn(H, generator=g)).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    eps = 1e-5
    print("case", dtype, T, H, flush=True)
    xg = x.to(dev).requires_grad_(True)
    wg = w.to(dev).requires_grad_(True)
    y = pkg.norm.rms_norm(xg, wg, eps)
    assert y.dtype == dtype and y.shape == (T, H)
    y.backward(dy.to(dev))
    ry, rdx, rdw = reference(orc, x, w, dy, eps)
    torch.testing.assert_close(y.detach().cpu().float(), ry, **TOL[dtype])
    if dtype != torch.float32:
        # one rounding of the fp32 value: only a last-bit difference of rstd can move a result
        # across a rounding boundary, so nearly all elements carry the oracle's bits
        differ = (y.detach().cpu() != orc.rms_norm(x, w, eps)).float().mean().item()
        assert differ < 1e-3, differ
    torch.testing.assert_close(xg.grad.cpu().float(), rdx, **TOL[dtype])
    # the weight gradient sums T terms in fp32 and is rounded once
    tol = dict(rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * max(1.0, T ** 0.5))
    torch.testing.assert_close(wg.grad.cpu().float(), rdw, **tol)


def test_rms_norm_saved_rstd_and_determinism(pkg, dev):
    g = torch.Generator().manual_seed(11)
    x = torch.randn(777, 4096, generator=g).bfloat16().to(dev)
    w = torch.ones(4096, dtype=torch.bfloat16, device=dev)
    dy = torch.randn(777, 4096, generator=g).bfloat16().to(dev)
    y, rstd = pkg.ops.rmsnorm_fwd(x, w, 1e-5)
    want = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    torch.testing.assert_close(rstd, want, rtol=1e-5, atol=0)
    a = pkg.ops.rmsnorm_bwd(dy, x, w, rstd)
    b = pkg.ops.rmsnorm_bwd(dy, x, w, rstd)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_rms_norm_module_and_pre_router_wiring(pkg, orc, dev):
    """RMSNorm has flash-attn's constructor and parameters; PreRouterNorm returns (normed, residual)
    like the tail of GalvatronMoEAttention.forward; 3-d [S, B, H] input keeps its shape."""
    cfg = pkg.MoEConfig(hidden_size=256, num_moe_experts=4, moe_ffn_hidden_size=128,
                        params_dtype=torch.bfloat16)
    with torch.cuda.device(dev):
        m = pkg.norm.GalvatronNorm(cfg, 256, eps=cfg.norm_epsilon)
    assert isinstance(m, pkg.norm.RMSNorm) and m.bias is None
    assert m.weight.dtype == torch.bfloat16 and torch.all(m.weight == 1) and m.weight.is_cuda
    assert [n for n, _ in m.named_parameters()] == ["weight"]
    pre = pkg.norm.PreRouterNorm(cfg, device=dev)
    h = torch.randn(16, 2, 256, device=dev).bfloat16()
    normed, residual = pre(h)
    assert residual.data_ptr() == h.data_ptr() and torch.equal(residual, h) and normed.shape == h.shape
    torch.testing.assert_close(normed.cpu().float(),
                               orc.rms_norm(h.cpu(), pre.pre_router_norm.weight.detach().cpu(), 1e-5).float(),
                               rtol=2e-2, atol=1e-2)
    cfg.normalization = "LayerNorm"
    with pytest.raises(NotImplementedError):
        pkg.norm.GalvatronNorm(cfg, 256)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_pre_router_norm_adds_the_residual_gradient_in_the_kernel(pkg, dev, dtype):
    """The fork (norm(x), x): its single backward kernel gives the bits of rms_norm's backward
    followed by autograd's add of the residual branch's gradient; unused branches are handled."""
    cfg = pkg.MoEConfig(hidden_size=1024, num_moe_experts=4, moe_ffn_hidden_size=128, params_dtype=dtype)
    pre = pkg.norm.PreRouterNorm(cfg, device=dev)
    g = torch.Generator().manual_seed(5)
    with torch.no_grad():
        pre.pre_router_norm.weight.copy_((1 + 0.2 * torch.randn(1024, generator=g)).to(dev))
    x = torch.randn(333, 1024, generator=g).to(dtype).to(dev)
    dy = torch.randn(333, 1024, generator=g).to(dtype).to(dev)
    dres = torch.randn(333, 1024, generator=g).to(dtype).to(dev)
    xa = x.clone().requires_grad_(True)
    normed, residual = pre(xa)
    torch.autograd.backward([normed, residual], [dy, dres])
    wgrad = pre.pre_router_norm.weight.grad.clone()
    pre.pre_router_norm.weight.grad = None
    xb = x.clone().requires_grad_(True)
    y = pkg.norm.rms_norm(xb, pre.pre_router_norm.weight, cfg.norm_epsilon)
    torch.autograd.backward([y, xb * 1.0], [dy, dres])   # separate add by autograd
    assert torch.equal(normed, y)
    assert torch.equal(xa.grad, xb.grad)
    assert torch.equal(wgrad, pre.pre_router_norm.weight.grad)
    # only one branch used
    xc = x.clone().requires_grad_(True)
    pre(xc)[1].backward(dres)
    assert torch.equal(xc.grad, dres)
    xd = x.clone().requires_grad_(True)
    pre(xd)[0].backward(dy)
    xe = x.clone().requires_grad_(True)
    pkg.norm.rms_norm(xe, pre.pre_router_norm.weight, cfg.norm_epsilon).backward(dy)
    assert torch.equal(xd.grad, xe.grad)


def test_rms_norm_empty_and_bad_shapes(pkg, dev):
    w = torch.ones(64, dtype=torch.bfloat16, device=dev, requires_grad=True)
    x = torch.empty(0, 64, dtype=torch.bfloat16, device=dev, requires_grad=True)
    y = pkg.norm.rms_norm(x, w, 1e-5)
    assert y.shape == (0, 64)
    y.sum().backward()
    assert torch.count_nonzero(w.grad) == 0
    with pytest.raises(RuntimeError):   # H not a multiple of the 16-byte vector
        pkg.ops.rmsnorm_fwd(torch.zeros(4, 12, dtype=torch.bfloat16, device=dev),
                            torch.ones(12, dtype=torch.bfloat16, device=dev), 1e-5)
    with pytest.raises(RuntimeError):   # beyond the widest kernel
        pkg.ops.rmsnorm_fwd(torch.zeros(2, 32768, dtype=torch.bfloat16, device=dev),
                            torch.ones(32768, dtype=torch.bfloat16, device=dev), 1e-5)


def test_full_size_norm_and_gate_against_torch_on_the_gpu(pkg, dev):
    """Benchmark size (T 16384, H 4096, E 8), too large for the CPU oracle in a quick test: torch's
    own fp32 rms_norm / linear with autograd on the GPU as the independent implementation, and the
    invariant mean(y^2 / w^2) = 1 per row that fixes the scale."""
    T, H, E = 16384, 4096, 8
    g = torch.Generator(device=dev).manual_seed(17)
    x = (torch.randn(T, H, generator=g, device=dev) * 3).bfloat16().requires_grad_(True)
    wn = (1 + 0.1 * torch.randn(H, generator=g, device=dev)).bfloat16().requires_grad_(True)
    wg = (torch.randn(E, H, generator=g, device=dev) * 0.02).bfloat16().requires_grad_(True)
    dl = torch.randn(T, E, generator=g, device=dev).bfloat16()
    dy = torch.randn(T, H, generator=g, device=dev).bfloat16()
    y = pkg.norm.rms_norm(x, wn, 1e-5)
    logits = pkg.router._GateProjection.apply(y, wg, torch.bfloat16)
    torch.autograd.backward([y, logits], [dy, dl])
    xr = x.detach().float().requires_grad_(True)
    wnr = wn.detach().float().requires_grad_(True)
    wgr = wg.detach().float().requires_grad_(True)
    yr = torch.nn.functional.rms_norm(xr, (H,), wnr, 1e-5)
    yb = yr.detach().bfloat16().float()
    lr = torch.nn.functional.linear(yb + (yr - yr.detach()), wgr)   # the gate sees the rounded y
    torch.autograd.backward([yr, lr], [dy.float(), dl.float()])
    tol = dict(rtol=2e-2, atol=1e-2)
    torch.testing.assert_close(y.detach().float(), yr.detach(), **tol)
    torch.testing.assert_close(logits.detach().float(), lr.detach(), **tol)
    torch.testing.assert_close(x.grad.float(), xr.grad, **tol)
    torch.testing.assert_close(wg.grad.float(), wgr.grad, rtol=2e-2, atol=1e-2 * T ** 0.5)
    torch.testing.assert_close(wn.grad.float(), wnr.grad, rtol=2e-2, atol=1e-2 * T ** 0.5)
    ms = (y.detach().float() / wn.detach().float()).pow(2).mean(-1)
    torch.testing.assert_close(ms, torch.ones_like(ms), rtol=5e-3, atol=0)
