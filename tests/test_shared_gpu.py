"""Shared experts (moe/mlp.py:215-400) and the layer around them on the GPU: parameter names and
layouts of the reference, the sigmoid gate, the staged (overlapped) interface, the additions fused
into the combine kernel, SequentialMLP inside the layer, and the Hugging Face loaders of router,
experts and pre-router norm."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=2e-3, atol=2e-4), torch.bfloat16: dict(rtol=2e-2, atol=1e-2)}


def shared_reference(orc, x, fc1_w, fc2_w, gate_w):
    """The oracle's shared MLP (weights in its [H,2Fs] / [Fs,H] layout) and the sigmoid gate of
    moe/mlp.py:271-278, fp32 math on the given (already rounded) values."""
    out = orc.shared_expert_mlp(x, fc1_w.t(), fc2_w.t())
    if gate_w is not None:
        out = out * torch.sigmoid(torch.nn.functional.linear(x, gate_w))
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gate", [False, True])
@pytest.mark.parametrize("T,H,Fs", [(300, 128, 192), (2048, 512, 1024)])
def test_shared_expert_mlp_forward_backward(pkg, orc, dev, dtype, gate, T, H, Fs):
    cfg = pkg.MoEConfig(hidden_size=H, moe_shared_expert_intermediate_size=Fs, params_dtype=dtype)
    m = pkg.SharedExpertMLP(cfg, gate=gate, device=dev)
    names = dict(m.named_parameters())
    assert names["linear_fc1.weight"].shape == (2 * Fs, H) and names["linear_fc2.weight"].shape == (H, Fs)
    assert ("gate_weight" in names) == gate and (not gate or names["gate_weight"].shape == (1, H))
    g = torch.Generator().manual_seed(T + Fs)
    x = torch.randn(6, T // 6, H, generator=g).to(dtype)
    go = torch.randn(6, T // 6, H, generator=g).to(dtype)
    with torch.no_grad():
        m.linear_fc1.weight.copy_((torch.randn(2 * Fs, H, generator=g) / H ** 0.5).to(dev))
        m.linear_fc2.weight.copy_((torch.randn(H, Fs, generator=g) / Fs ** 0.5).to(dev))
        if gate:
            m.gate_weight.copy_((torch.randn(1, H, generator=g) / H ** 0.5).to(dev))
    xg = x.to(dev).requires_grad_(True)
    out = m(xg)
    assert out.shape == x.shape and out.dtype == dtype
    out.backward(go.to(dev))
    # the oracle on the tensors in their storage type: fp32 accumulation inside every product, fc1,
    # the activation and the output rounded to the storage type between the ops, as the kernels do
    xo = x.clone().requires_grad_(True)
    po = {k: v.detach().cpu().clone().requires_grad_(True) for k, v in names.items()}
    ref = shared_reference(orc, xo.view(-1, H), po["linear_fc1.weight"], po["linear_fc2.weight"],
                           po.get("gate_weight")).view(x.shape)
    ref.backward(go)
    tol = TOL[dtype]
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach().float(), **tol)
    torch.testing.assert_close(xg.grad.cpu().float(), xo.grad.float(), **tol)
    # weight gradients sum T products of intermediates that each side rounds to the storage type at
    # its own places (the oracle's autograd rounds out * grad elementwise before the row sum of the
    # gate's gradient, the kernel rounds the fp32 row sum): errors of rtol relative to the terms, so
    # the bound is taken relative to the tensor's largest value
    for k in names:
        want = po[k].grad.float()
        torch.testing.assert_close(names[k].grad.cpu().float(), want, rtol=tol["rtol"],
                                   atol=tol["rtol"] * want.abs().max().item())


def build(pkg, dev, dtype, overlap, dispatcher="alltoall", grouped=True, E=8, H=256, F=128, Fs=384, k=2):
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=F, moe_router_topk=k,
                        moe_router_load_balancing_type="none", moe_token_dispatcher_type=dispatcher,
                        params_dtype=dtype, moe_shared_expert_intermediate_size=Fs,
                        moe_shared_expert_overlap=overlap, moe_grouped_gemm=grouped)
    torch.manual_seed(5)
    return cfg, pkg.GalvatronMoERouter(cfg, device=dev), pkg.GalvatronMoEMLP(cfg, device=dev)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dispatcher", ["allgather", "alltoall"])
def test_layer_overlapped_shared_experts_give_the_same_bits(pkg, dev, dtype, dispatcher):
    """The staged interface on its own stream against the plain call: same kernels, same bits in
    the output and in every gradient; and the fused additions against separate adds."""
    cfg, router, mlp = build(pkg, dev, dtype, overlap=False, dispatcher=dispatcher)
    cfg2, router2, mlp2 = build(pkg, dev, dtype, overlap=True, dispatcher=dispatcher)
    mlp2.load_state_dict(mlp.state_dict())
    router2.load_state_dict(router.state_dict())
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 4, 256, generator=g).to(dtype).to(dev)
    dy = torch.randn(64, 4, 256, generator=g).to(dtype).to(dev)
    res = torch.randn(64, 4, 256, generator=g).to(dtype).to(dev)
    outs = []
    for r, m in ((router, mlp), (router2, mlp2)):
        xg = x.clone().requires_grad_(True)
        probs, rmap = r(xg)
        out = m(xg, res, probs, rmap)
        out.backward(dy)
        torch.cuda.synchronize()
        outs.append([out.detach(), xg.grad] + [p.grad for p in m.parameters()])
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # separate adds (the reference's order: combine, += shared, + residual) give the same bits
    xg = x.clone().requires_grad_(True)
    probs, rmap = router(xg)
    d, tpe = mlp.token_dispatcher.token_permutation(xg, probs, rmap)
    eo, _ = mlp.experts(d, tpe)
    sep, _ = mlp.token_dispatcher.token_unpermutation(eo, None)
    sep = sep + mlp.shared_experts(xg)
    sep = sep + res
    assert torch.equal(sep.detach(), outs[0][0])


def test_layer_with_shared_experts_against_the_oracle(pkg, orc, dev):
    E, H, F, Fs, k = 8, 256, 128, 384, 2
    cfg, router, mlp = build(pkg, dev, torch.float32, overlap=True)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(48, 2, H, generator=g)
    dy = torch.randn(48, 2, H, generator=g)
    xg = x.to(dev).requires_grad_(True)
    probs, rmap = router(xg)
    out = mlp(xg, xg, probs, rmap)
    out.backward(dy.to(dev))
    xo = x.clone().requires_grad_(True)
    w1 = mlp.experts.weight1.detach().cpu().view(E, H, 2 * F)
    w2 = mlp.experts.weight2.detach().cpu().view(E, F, H)
    ref, _, info = orc.moe_layer(xo, router.router.weight.detach().cpu(), w1, w2, k, residual=xo,
                                 dispatcher="alltoall",
                                 shared_w1=mlp.shared_experts.linear_fc1.weight.detach().cpu().t(),
                                 shared_w2=mlp.shared_experts.linear_fc2.weight.detach().cpu().t())
    ref.backward(dy)
    assert torch.equal(rmap.cpu(), info["routing_map"])
    torch.testing.assert_close(out.detach().cpu(), ref.detach(), **TOL[torch.float32])
    torch.testing.assert_close(xg.grad.cpu(), xo.grad, **TOL[torch.float32])


def test_layer_with_sequential_experts_matches_the_grouped_layer(pkg, dev):
    """moe_grouped_gemm=False builds SequentialMLP inside the layer (the layout the reference's
    checkpoints load into); same weights through the converters, same result within bf16 rounding."""
    cfg, router, mlp = build(pkg, dev, torch.bfloat16, overlap=False, grouped=True)
    cfg_s, router_s, mlp_s = build(pkg, dev, torch.bfloat16, overlap=False, grouped=False)
    assert isinstance(mlp_s.experts, pkg.SequentialMLP)
    state = pkg.checkpoint.hf_from_moe_layer(router, mlp)
    pkg.checkpoint.load_moe_layer_from_hf(state, router_s, mlp_s)
    mlp_s.shared_experts.load_state_dict(mlp.shared_experts.state_dict())
    g = torch.Generator().manual_seed(3)
    x = torch.randn(40, 4, 256, generator=g).bfloat16().to(dev)
    probs, rmap = router(x)
    probs_s, rmap_s = router_s(x)
    assert torch.equal(rmap, rmap_s) and torch.equal(probs, probs_s)
    torch.testing.assert_close(mlp_s(x, None, probs_s, rmap_s).float(), mlp(x, None, probs, rmap).float(),
                               rtol=2e-2, atol=1e-2)


def test_hf_loaders_round_trip_router_norm_and_experts(pkg, dev):
    cfg = pkg.MoEConfig(hidden_size=64, num_moe_experts=4, moe_ffn_hidden_size=96, moe_router_topk=2,
                        moe_router_score_function="sigmoid", moe_router_enable_expert_bias=True,
                        params_dtype=torch.bfloat16)
    router = pkg.GalvatronMoERouter(cfg, device=dev)
    mlp = pkg.GalvatronMoEMLP(cfg, device=dev)
    pre = pkg.PreRouterNorm(cfg, device=dev)
    with torch.no_grad():
        router.router.expert_bias.copy_(torch.tensor([0.1, -0.2, 0.3, 0.0]))
        pre.pre_router_norm.weight.copy_(torch.linspace(0.5, 1.5, 64))
    state = pkg.checkpoint.hf_from_moe_layer(router, mlp, pre)
    assert set(state) >= {"block_sparse_moe.gate.weight", "block_sparse_moe.expert_bias",
                          "post_attention_layernorm.weight", "block_sparse_moe.experts.3.w2.weight"}
    assert state["block_sparse_moe.experts.0.w1.weight"].shape == (96, 64)
    router2 = pkg.GalvatronMoERouter(cfg, device=dev)
    mlp2 = pkg.GalvatronMoEMLP(cfg, device=dev)
    pre2 = pkg.PreRouterNorm(cfg, device=dev)
    pkg.checkpoint.load_moe_layer_from_hf({k: v.cpu() for k, v in state.items()}, router2, mlp2, pre2)
    assert torch.equal(router2.router.weight, router.router.weight)
    assert torch.equal(router2.router.expert_bias, router.router.expert_bias)
    assert torch.equal(pre2.pre_router_norm.weight, pre.pre_router_norm.weight)
    assert torch.equal(mlp2.experts.weight1, mlp.experts.weight1)
    assert torch.equal(mlp2.experts.weight2, mlp.experts.weight2)
