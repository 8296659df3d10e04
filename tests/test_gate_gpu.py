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
    (8192, 2048, 64),   # the fine-grained configuration: two expert blocks in the forward kernel,
                        # gradients as dense products, the weight gradient in 32 row ranges
    (300, 512, 40),     # a partial second expert block
    (45, 2056, 48),     # ... with ragged rows and a reduction that does not fill the last stage
    (257, 4104, 64),    # rows that do not start on a cache line
    (700, 1024, 128),   # forward as a dense product with its reduction split over the workspace
    (4096, 7168, 256),  # the DeepSeek-V3-shape router
    (300, 512, 24),     # few rows, ragged
    (1000, 1024, 32),   # forward on the one-pass kernel, gradients on the dense products
    (300, 512, 20),     # beyond 16 experts and not a multiple of 8: zero rows pad the table to 24
    (1000, 1024, 60),   # ... to 64
    (257, 4104, 17),    # ... 17 -> 24 with ragged rows
    (512, 1024, 100),   # ... 100 -> 104, forward as a dense product
]


# fp32 operands with fp32 logits is the plain fp32 case: not generated twice
@pytest.mark.parametrize("dtype,fp32_logits", [(torch.bfloat16, False), (torch.float32, False),
                                               (torch.float16, False), (torch.bfloat16, True),
                                               (torch.float16, True)])
@pytest.mark.parametrize("T,H,E", SHAPES)
def test_gate_projection_forward_backward(pkg, orc, dev, dtype, T, H, E, fp32_logits):
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
    # one product on the same operands: the output's own rounding (16-bit), or the rounding of T
    # fp32 additions in another order (fp32: 6e-8 * |terms| * sqrt(T))
    tol = dict(TOL[dtype])
    if dtype == torch.float32:
        tol["atol"] = max(tol["atol"], 1e-5 * T ** 0.5)
    torch.testing.assert_close(dw.cpu().float(), dl.float().t() @ x.float(), **tol)
    if fp32_logits and dtype != torch.float32 and E > 16:
        # the fp32 gradient enters as hi + lo: far closer to the fp32 product than one 16-bit
        # rounding of the gradient would be (relative error 2^-9 per term)
        ref = dl.double() @ w.double()
        err = (dx.cpu().double() - ref).abs().max().item()
        one_rounding = (dl.to(dtype).double() @ w.double() - ref).abs().max().item()
        assert err <= ref.abs().max().item() * 2.0 ** -8 and one_rounding > 0
    # deterministic
    dx2, dw2 = pkg.ops.gate_bwd(dl.to(dev), xd, wd)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)
    assert torch.equal(logits, pkg.ops.gate_fwd(xd, wd, out_dtype=ldt))


@pytest.mark.parametrize("router_dtype", [None, "fp32"])
def test_router_gating_uses_the_hip_projection_and_matches_f_linear(pkg, dev, router_dtype):
    """TopKRouter.gating on [S,B,H] input: same values and gradients as F.linear on the casts
    (router.py:49-68), within bf16 tolerance; 64 experts stay on the HIP path too."""
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
    # 64 experts: dense products on the grouped-GEMM kernels, still through ops.gate_fwd
    cfg64 = pkg.MoEConfig(hidden_size=512, num_moe_experts=64, moe_ffn_hidden_size=64,
                          moe_router_dtype=router_dtype, params_dtype=torch.bfloat16)
    r64 = pkg.TopKRouter(cfg64).to(dev)
    with torch.no_grad():
        r64.weight.copy_(torch.randn(64, 512, device=dev) * 0.05)
    calls.clear()
    pkg.ops.gate_fwd = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        x3 = x.detach().clone().requires_grad_(True)
        l64 = r64.gating(x3)
    finally:
        pkg.ops.gate_fwd = orig
    assert calls and l64.shape == (24, 2, 64) and l64.dtype == rd
    go64 = torch.randn(24, 2, 64, device=dev).to(rd)
    l64.backward(go64)
    x4 = x.detach().clone().requires_grad_(True)
    w4 = r64.weight.detach().clone().requires_grad_(True)
    ref64 = torch.nn.functional.linear(x4.to(rd), w4.to(rd))
    ref64.backward(go64)
    torch.testing.assert_close(l64.float(), ref64.float(), **tol)
    torch.testing.assert_close(x3.grad.float(), x4.grad.float(), **tol)
    torch.testing.assert_close(r64.weight.grad.float(), w4.grad.float(), rtol=2e-2, atol=7e-2)


def test_gate_projection_without_rows_and_bad_shapes(pkg, dev):
    w = torch.randn(8, 64, device=dev).bfloat16()
    x = torch.empty(0, 64, device=dev, dtype=torch.bfloat16)
    assert pkg.ops.gate_fwd(x, w).shape == (0, 8)
    dx, dw = pkg.ops.gate_bwd(torch.empty(0, 8, device=dev, dtype=torch.bfloat16), x, w)
    assert dx.shape == (0, 64) and torch.count_nonzero(dw) == 0
    with pytest.raises(RuntimeError):   # H not a multiple of the 16-byte piece
        pkg.ops.gate_fwd(torch.zeros(4, 12, device=dev, dtype=torch.bfloat16),
                         torch.zeros(8, 12, device=dev, dtype=torch.bfloat16))
    # beyond 16 experts the table is padded to a multiple of 8 rows: 20 experts come back as 20
    dx, dw = pkg.ops.gate_bwd(torch.zeros(4, 20, device=dev, dtype=torch.bfloat16),
                              torch.zeros(4, 64, device=dev, dtype=torch.bfloat16),
                              torch.zeros(20, 64, device=dev, dtype=torch.bfloat16))
    assert dx.shape == (4, 64) and dw.shape == (20, 64)
    with pytest.raises(RuntimeError):   # more experts than the dense products take
        pkg.ops.gate_fwd(torch.zeros(4, 64, device=dev, dtype=torch.bfloat16),
                         torch.zeros(4104, 64, device=dev, dtype=torch.bfloat16))
    # no rows with many experts: zeros for the weight gradient
    w64 = torch.randn(64, 64, device=dev).bfloat16()
    dx, dw = pkg.ops.gate_bwd(torch.empty(0, 64, device=dev, dtype=torch.bfloat16), x, w64)
    assert dx.shape == (0, 64) and dw.shape == (64, 64) and torch.count_nonzero(dw) == 0


def test_router_gating_any_expert_count_and_refused_dtypes(pkg, dev):
    """router.py:49-68 for an expert count the dense products do not take as it is (60), for a
    gate weight kept in fp32 beside bf16 activations, and for fp64, which is refused."""
    cfg = pkg.MoEConfig(hidden_size=256, num_moe_experts=60, moe_ffn_hidden_size=64, moe_router_topk=6,
                        params_dtype=torch.bfloat16)
    router = pkg.TopKRouter(cfg).to(dev)
    with torch.no_grad():
        router.weight.copy_(torch.randn(60, 256, device=dev) * 0.05)
    x = torch.randn(40, 2, 256, device=dev).bfloat16().requires_grad_(True)
    logits = router.gating(x)
    assert logits.shape == (40, 2, 60) and logits.dtype == torch.bfloat16
    go = torch.randn(40, 2, 60, device=dev).bfloat16()
    logits.backward(go)
    x2 = x.detach().clone().requires_grad_(True)
    w2 = router.weight.detach().clone().requires_grad_(True)
    ref = torch.nn.functional.linear(x2, w2)
    ref.backward(go)
    tol = dict(rtol=2e-2, atol=1e-2)
    torch.testing.assert_close(logits.float(), ref.float(), **tol)
    torch.testing.assert_close(x.grad.float(), x2.grad.float(), **tol)
    torch.testing.assert_close(router.weight.grad.float(), w2.grad.float(), rtol=2e-2, atol=7e-2)
    # fp32 gate weight, bf16 activations: the weight is cast as F.linear(input, weight.to(rd)) would
    router.weight.data = router.weight.data.float()
    router.weight.grad = None
    l2 = router.gating(x.detach())
    assert l2.dtype == torch.bfloat16
    torch.testing.assert_close(l2.float(), ref.detach().float(), **tol)
    l2.sum().backward()
    assert router.weight.grad.dtype == torch.float32
    cfg64 = pkg.MoEConfig(hidden_size=256, num_moe_experts=8, moe_ffn_hidden_size=64,
                          moe_router_dtype="fp64", params_dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        pkg.TopKRouter(cfg64).to(dev).gating(x.detach())
