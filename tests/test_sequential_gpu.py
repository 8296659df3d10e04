"""SequentialMLP (one expert after the other, `linear_fc1 [2F,H]` / `linear_fc2 [H,F]`) against
GroupedMLP on the same weights, both filled from Hugging Face Mixtral keys, and against the
oracle's expert MLP on those weights."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = dict(rtol=2e-2, atol=1e-2)


def hf_state(E, H, Fe, seed=0):
    g = torch.Generator().manual_seed(seed)
    st = {}
    for e in range(E):
        st["block_sparse_moe.experts.%d.w1.weight" % e] = (torch.randn(Fe, H, generator=g) / H ** 0.5).bfloat16()
        st["block_sparse_moe.experts.%d.w3.weight" % e] = (torch.randn(Fe, H, generator=g) / H ** 0.5).bfloat16()
        st["block_sparse_moe.experts.%d.w2.weight" % e] = (torch.randn(H, Fe, generator=g) / Fe ** 0.5).bfloat16()
    return st


@pytest.mark.parametrize("E,H,Fe,counts", [(4, 128, 256, [40, 0, 77, 11]), (1, 64, 128, [50]),
                                           (8, 256, 512, [600, 520, 512, 700, 0, 530, 640, 594])])
def test_sequential_and_grouped_agree_and_match_the_mixtral_formula(pkg, orc, dev, E, H, Fe, counts):
    st = hf_state(E, H, Fe, seed=E)
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=Fe,
                        params_dtype=torch.bfloat16)
    seq = pkg.SequentialMLP(E, cfg, device=dev)
    grp = pkg.GroupedMLP(E, cfg, device=dev)
    pkg.checkpoint.load_experts_from_hf(st, seq, range(E))
    pkg.checkpoint.load_experts_from_hf(st, grp, range(E))
    # the two layouts hold the same matrices
    grp2 = pkg.GroupedMLP(E, cfg, device=dev)
    pkg.checkpoint.copy_sequential_to_grouped(seq, grp2)
    assert torch.equal(grp2.weight1, grp.weight1) and torch.equal(grp2.weight2, grp.weight2)
    seq2 = pkg.SequentialMLP(E, cfg, device=dev)
    pkg.checkpoint.copy_grouped_to_sequential(grp, seq2)
    for a, b in zip(seq.parameters(), seq2.parameters()):
        assert torch.equal(a, b)

    bs = torch.tensor(counts, dtype=torch.int64)
    N = int(bs.sum())
    g = torch.Generator().manual_seed(9)
    x = torch.randn(N, H, generator=g).bfloat16()
    go = torch.randn(N, H, generator=g).bfloat16()
    outs = []
    for m in (seq, grp):
        xs = x.to(dev).requires_grad_(True)
        out, bias = m(xs, bs)
        assert bias is None
        out.backward(go.to(dev))
        outs.append((out.detach().cpu().float(), xs.grad.cpu().float()))
    # the oracle's expert MLP on the grouped layout of the same HF tensors (pinned to the Mixtral
    # formula w2(silu(w1 x) * w3 x) by the CPU tests); like the kernels it rounds fc1 and the
    # activation to bf16 between the ops
    w1g, w2g = pkg.checkpoint.grouped_from_hf(st, range(E))
    xo = x.clone().requires_grad_(True)
    ref = orc.grouped_mlp(xo, w1g.view(E, H, 2 * Fe), w2g.view(E, Fe, H), bs)
    ref.backward(go)
    for out, gx in outs:
        torch.testing.assert_close(out, ref.detach().float(), **TOL)
        torch.testing.assert_close(gx, xo.grad.float(), **TOL)
    # weight gradients of the two layouts are the same matrices too
    g1, g2 = pkg.checkpoint.fc_from_grouped(grp.weight1.grad, grp.weight2.grad, E)
    for e in range(E):
        a = seq.local_experts[e].linear_fc1.weight.grad
        b = seq.local_experts[e].linear_fc2.weight.grad
        if counts[e] == 0:
            assert a is None or torch.count_nonzero(a) == 0
            continue
        tol = dict(rtol=2e-2, atol=1e-2 * max(1.0, counts[e] ** 0.5))
        torch.testing.assert_close(a.float(), g1[e].float(), **tol)
        torch.testing.assert_close(b.float(), g2[e].float(), **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("N,M,counts", [(300, 256, None), (77, 100, None), (0, 64, None),
                                        (1000, 384, [100, 0, 333, 7, 500]), (64, 24, [10, 20, 30])])
def test_bias_rows_and_their_gradient(pkg, dev, dtype, N, M, counts):
    """out[r] = x[r] + bias[expert of r], bit for bit torch's add; the gradient is the per-expert column
    sum in fp32.  Rows past the last offset (a buffer sized by an upper bound) keep x."""
    g = torch.Generator().manual_seed(N + M)
    x = torch.randn(N, M, generator=g).to(dtype)
    if counts is None:
        bias = torch.randn(M, generator=g).to(dtype)
        out = pkg.ops.bias_rows(x.to(dev), bias.to(dev))
        assert torch.equal(out.cpu(), x + bias)
        alone = pkg.ops.bias_rows(None, bias.to(dev), num_rows=N)
        assert torch.equal(alone.cpu(), bias.expand(N, M))
        gb = pkg.ops.bias_rows_bwd(x.to(dev))
        want = x.double().sum(0)
    else:
        E = len(counts)
        off = torch.zeros(E + 1, dtype=torch.int64)
        off[1:] = torch.tensor(counts).cumsum(0)
        used = int(off[-1])
        assert used <= N
        bias = torch.randn(E, M, generator=g).to(dtype)
        expert_of_row = torch.repeat_interleave(torch.arange(E), torch.tensor(counts))
        want_out = x.clone()
        want_out[:used] = x[:used] + bias[expert_of_row]
        out = pkg.ops.bias_rows(x.to(dev), bias.to(dev), expert_offsets=off.to(dev))
        assert torch.equal(out.cpu(), want_out)
        gb = pkg.ops.bias_rows_bwd(x.to(dev), off.to(dev), E)
        want = torch.zeros(E, M, dtype=torch.float64).index_add_(0, expert_of_row, x[:used].double())
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -22}[dtype]
    bound = eps * want.abs() + 2.0 ** -20 * (x.double().abs().sum(0).max() if N else 0.0) + 1e-30
    assert ((gb.cpu().double() - want).abs() <= bound).all()


@pytest.mark.parametrize("E,H,Fe,counts", [(4, 128, 256, [40, 0, 77, 11]), (1, 64, 128, [50])])
def test_sequential_experts_with_bias_against_the_oracle(pkg, orc, dev, E, H, Fe, counts):
    """`add_bias_linear`: fc1 bias in front of the activation, fc2 bias handed back as rows (a single
    expert hands back its [H] vector), gradients of both biases."""
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=Fe,
                        params_dtype=torch.bfloat16, add_bias_linear=True)
    torch.manual_seed(3)
    seq = pkg.SequentialMLP(E, cfg, device=dev)
    g = torch.Generator().manual_seed(4)
    for ex in seq.local_experts:
        assert torch.count_nonzero(ex.linear_fc1.bias) == 0 and torch.count_nonzero(ex.linear_fc2.bias) == 0
        with torch.no_grad():
            ex.linear_fc1.weight.copy_((torch.randn(2 * Fe, H, generator=g) / H ** 0.5).to(dev))
            ex.linear_fc2.weight.copy_((torch.randn(H, Fe, generator=g) / Fe ** 0.5).to(dev))
            ex.linear_fc1.bias.copy_(torch.randn(2 * Fe, generator=g).to(dev))
            ex.linear_fc2.bias.copy_(torch.randn(H, generator=g).to(dev))
    bs = torch.tensor(counts, dtype=torch.int64)
    N = int(bs.sum())
    x = torch.randn(N, H, generator=g).bfloat16()
    go = torch.randn(N, H, generator=g).bfloat16()
    gob = torch.randn(N, H, generator=g).bfloat16()
    xs = x.to(dev).requires_grad_(True)
    out, out_bias = seq(xs, bs)
    rows_bias = out_bias if E > 1 else out_bias.expand(N, H)
    (out * go.to(dev) + rows_bias * gob.to(dev)).sum().backward()

    stack = lambda f: torch.stack([f(ex).detach().cpu() for ex in seq.local_experts])  # noqa: E731
    ref_p = [stack(lambda ex: ex.linear_fc1.weight), stack(lambda ex: ex.linear_fc2.weight),
             stack(lambda ex: ex.linear_fc1.bias), stack(lambda ex: ex.linear_fc2.bias)]
    ref_p = [p.requires_grad_(True) for p in ref_p]
    xo = x.clone().requires_grad_(True)
    ref, ref_bias = orc.sequential_mlp(xo, ref_p[0], ref_p[1], bs, ref_p[2], ref_p[3])
    (ref * go + ref_bias * gob).sum().backward()
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach().float(), **TOL)
    assert torch.equal(rows_bias.detach().cpu(), ref_bias.detach())
    torch.testing.assert_close(xs.grad.cpu().float(), xo.grad.float(), **TOL)
    for e, ex in enumerate(seq.local_experts):
        if counts[e] == 0:
            continue
        tol = dict(rtol=2e-2, atol=1e-2 * max(1.0, counts[e] ** 0.5))
        torch.testing.assert_close(ex.linear_fc1.bias.grad.cpu().float(), ref_p[2].grad[e].float(), **tol)
        torch.testing.assert_close(ex.linear_fc2.bias.grad.cpu().float(), ref_p[3].grad[e].float(), **tol)
        torch.testing.assert_close(ex.linear_fc1.weight.grad.cpu().float(), ref_p[0].grad[e].float(), **tol)


def test_layer_with_expert_bias_combines_the_bias_beside_the_output(pkg, orc, dev):
    """The AllGather dispatcher weights and combines the experts' bias rows like their output and
    returns them beside it (token_dispatcher.py:246-284); the layer, like the reference's
    (models/moe_modules.py:125-128), does not add them."""
    E, H, Fe, k, S, B = 4, 128, 256, 2, 48, 2
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=Fe, moe_router_topk=k,
                        moe_router_load_balancing_type="none", moe_token_dispatcher_type="allgather",
                        moe_grouped_gemm=False, params_dtype=torch.bfloat16, add_bias_linear=True)
    torch.manual_seed(5)
    router = pkg.GalvatronMoERouter(cfg, device=dev)
    mlp = pkg.GalvatronMoEMLP(cfg, device=dev)
    g = torch.Generator().manual_seed(6)
    with torch.no_grad():
        for ex in mlp.experts.local_experts:
            ex.linear_fc1.bias.copy_(torch.randn(2 * Fe, generator=g).to(dev))
            ex.linear_fc2.bias.copy_(torch.randn(H, generator=g).to(dev))
    x = torch.randn(S, B, H, generator=g).bfloat16().to(dev)
    probs, rmap = router(x)
    permuted, tpe = mlp.token_dispatcher.token_permutation(x, probs, rmap)
    expert_out, bias_rows = mlp.experts(permuted, tpe)
    out, out_bias = mlp.token_dispatcher.token_unpermutation(expert_out, bias_rows)
    # oracle on the same expert output and bias rows
    _, sorted_indices = orc.permute(torch.zeros(S * B, H), rmap.cpu())
    ref, ref_bias = orc.allgather_combine(expert_out.detach().cpu(), probs.detach().cpu(), rmap.cpu(),
                                          sorted_indices, (S * B, H), bias=bias_rows.detach().cpu())
    torch.testing.assert_close(out.detach().cpu().float().view(-1, H), ref.float(), **TOL)
    torch.testing.assert_close(out_bias.detach().cpu().float().view(-1, H), ref_bias.float(), **TOL)
    # the whole layer equals the combine without the bias, plus the residual
    resid = torch.randn(S, B, H, generator=g).bfloat16().to(dev)
    layer = mlp(x, resid, probs, rmap)
    assert torch.equal(layer, out + resid)


def test_bias_is_refused_where_the_reference_refuses_it(pkg, dev):
    """GroupedMLP (moe/mlp.py:43-45), the shared experts (moe/mlp.py:227-228) and the AlltoAll
    dispatcher (moe/token_dispatcher.py:626) take no bias."""
    kw = dict(hidden_size=64, num_moe_experts=4, moe_ffn_hidden_size=128, params_dtype=torch.bfloat16,
              add_bias_linear=True)
    with pytest.raises(AssertionError, match="bias not supported in Grouped GEMM"):
        pkg.GroupedMLP(4, pkg.MoEConfig(**kw), device=dev)
    with pytest.raises(AssertionError, match="bias is not supported in the shared experts"):
        pkg.mlp.SharedExpertMLP(pkg.MoEConfig(moe_shared_expert_intermediate_size=128, **kw), device=dev)
    cfg = pkg.MoEConfig(moe_token_dispatcher_type="alltoall", moe_router_topk=2, **kw)
    disp = pkg.token_dispatcher.MoEAlltoAllTokenDispatcher(4, list(range(4)), cfg)
    x = torch.randn(8, 1, 64, device=dev, dtype=torch.bfloat16)
    logits = torch.randn(8, 4, device=dev)
    probs, rmap, _ = pkg.topk_softmax_with_capacity(logits, 2)
    permuted, _ = disp.token_permutation(x, probs.to(torch.bfloat16), rmap)
    with pytest.raises(AssertionError, match="Bias is not supported in MoEAlltoAllTokenDispatcher"):
        disp.token_unpermutation(permuted, bias=torch.zeros_like(permuted))
