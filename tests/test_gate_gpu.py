"""The router's gate projection (Router.gating) on the GPU through the C ABI, against the oracle's
fp32 matmul of the same rounded operands and torch autograd of it."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=1e-4, atol=1e-4), torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
       torch.float16: dict(rtol=2e-3, atol=2e-3)}

SHAPES = [  # T, H, E
    (128, 128, 4),      # the reference's test model
    (1, 8, 1),
    (45, 2056, 8),      # ragged rows, H not a multiple of the per-wavefront split
    (1000, 4096, 8),    # Mixtral
    (3000, 4096, 8),    # more row groups than workgroups in the weight-gradient kernel
    (257, 7168, 16),    # two column slabs in the backward kernels
    (300, 512, 12),     # E not a multiple of 4
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("T,H,E", SHAPES)
@pytest.mark.parametrize("fp32_logits", [False, True])
def test_gate_projection_forward_backward(pkg, orc, dev, dtype, T, H, E, fp32_logits):
    if fp32_logits and dtype == torch.float32:
        pytest.skip("same as the plain fp32 case")
    g = torch.Generator().manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    w = (torch.randn(E, H, generator=g) / H ** 0.5).to(dtype)
    ldt = torch.float32 if fp32_logits else dtype
    dl = torch.randn(T, E, generator=g).to(ldt)
    print("case", dtype, T, H, E, fp32_logits, flush=True)
    xd, wd = x.to(dev), w.to(dev)
    logits = pkg.ops.gate_fwd(xd, wd, out_dtype=ldt)
    assert logits.shape == (T, E) and logits.dtype == ldt
    want = orc.gate_logits(x, w, "fp32" if fp32_logits else None)
    assert want.dtype == ldt
    torch.testing.assert_close(logits.cpu().float(), want.float(), **TOL[dtype if not fp32_logits else torch.float32])
    dx, dw = pkg.ops.gate_bwd(dl.to(dev), xd, wd)
    assert dx.dtype == dtype and dw.dtype == dtype
    torch.testing.assert_close(dx.cpu().float(), dl.float() @ w.float(), **TOL[dtype])
    tol = dict(rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * max(1.0, T ** 0.5))
    torch.testing.assert_close(dw.cpu().float(), dl.float().t() @ x.float(), **tol)
    # deterministic
    dx2, dw2 = pkg.ops.gate_bwd(dl.to(dev), xd, wd)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)
    assert torch.equal(logits, pkg.ops.gate_fwd(xd, wd, out_dtype=ldt))


@pytest.mark.parametrize("router_dtype", [None, "fp32"])
def test_router_gating_uses_the_hip_projection_and_matches_f_linear(pkg, dev, router_dtype):
    """TopKRouter.gating on [S,B,H] input: same values and gradients as F.linear on the casts
    (router.py:49-68), within bf16 tolerance; larger expert counts fall back to the BLAS library."""
    cfg = pkg.MoEConfig(hidden_size=512, num_moe_experts=8, moe_ffn_hidden_size=64,
                        moe_router_dtype=router_dtype, params_dtype=torch.bfloat16)
    router = pkg.TopKRouter(cfg).to(dev)
    with torch.no_grad():
        router.weight.copy_(torch.randn(8, 512, device=dev) * 0.05)
    x = torch.randn(24, 2, 512, device=dev).bfloat16().requires_grad_(True)
    calls = []
    orig = pkg.ops.gate_fwd
    pkg.ops.gate_fwd = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        logits = router.gating(x)
    finally:
        pkg.ops.gate_fwd = orig
    assert calls, "the HIP gate projection was not used"
    rd = torch.float32 if router_dtype == "fp32" else torch.bfloat16
    assert logits.shape == (24, 2, 8) and logits.dtype == rd
    go = torch.randn(24, 2, 8, device=dev).to(rd)
    logits.backward(go)
    x2 = x.detach().clone().requires_grad_(True)
    w2 = router.weight.detach().clone().requires_grad_(True)
    ref = torch.nn.functional.linear(x2.to(rd), w2.to(rd))
    ref.backward(go)
    tol = dict(rtol=2e-2, atol=1e-2)
    torch.testing.assert_close(logits.float(), ref.float(), **tol)
    torch.testing.assert_close(x.grad.float(), x2.grad.float(), **tol)
    torch.testing.assert_close(router.weight.grad.float(), w2.grad.float(), rtol=2e-2, atol=7e-2)
    assert x.grad.dtype == torch.bfloat16 and router.weight.grad.dtype == torch.bfloat16
    # 64 experts: outside the small-E kernels
    cfg64 = pkg.MoEConfig(hidden_size=512, num_moe_experts=64, moe_ffn_hidden_size=64,
                          params_dtype=torch.bfloat16)
    r64 = pkg.TopKRouter(cfg64).to(dev)
    assert r64.gating(x.detach()).shape == (24, 2, 64)


def test_gate_projection_without_rows_and_bad_shapes(pkg, dev):
    w = torch.randn(8, 64, device=dev).bfloat16()
    x = torch.empty(0, 64, device=dev, dtype=torch.bfloat16)
    assert pkg.ops.gate_fwd(x, w).shape == (0, 8)
    dx, dw = pkg.ops.gate_bwd(torch.empty(0, 8, device=dev, dtype=torch.bfloat16), x, w)
    assert dx.shape == (0, 64) and torch.count_nonzero(dw) == 0
    with pytest.raises(RuntimeError):   # H not a multiple of the 16-byte piece
        pkg.ops.gate_fwd(torch.zeros(4, 12, device=dev, dtype=torch.bfloat16),
                         torch.zeros(8, 12, device=dev, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):   # too many experts for the register-resident backward
        pkg.ops.gate_bwd(torch.zeros(4, 24, device=dev, dtype=torch.bfloat16),
                         torch.zeros(4, 64, device=dev, dtype=torch.bfloat16),
                         torch.zeros(24, 64, device=dev, dtype=torch.bfloat16))
