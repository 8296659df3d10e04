"""Router parity on the GPU, through the C ABI: expert selection, routing map and token counts are
bit-exact against the oracle on the same logits; gate values and gradients within fp tolerance."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
# probs are rounded once to the logits dtype; allow one unit in the last place of that dtype
PROB_TOL = {torch.float32: dict(rtol=1e-5, atol=1e-6), torch.bfloat16: dict(rtol=1e-2, atol=1e-3),
            torch.float16: dict(rtol=2e-3, atol=2e-4)}


def make_logits(T, E, dtype, seed, scale=0.02 * 64):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(T, E, generator=g)).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,E,k", [(2048, 8, 2), (8192, 64, 8), (777, 4, 2), (1000, 60, 6),
                                   (512, 256, 8), (64, 160, 6), (1, 8, 2), (300, 8, 1), (130, 16, 16)])
def test_topk_routing_bit_exact(pkg, orc, dev, dtype, T, E, k):
    logits = make_logits(T, E, dtype, seed=T + E)
    print("case", dtype, T, E, k, flush=True)
    probs, rmap, counts, _, idx = pkg.ops.route_topk(logits.to(dev), k, want_topk_idx=True)
    o_probs, o_map, o_counts, o_idx = orc.topk_softmax_with_capacity(logits, k, return_topk=True)
    assert torch.equal(idx.cpu().long(), o_idx), "selected experts differ"
    assert torch.equal(rmap.cpu(), o_map)
    assert torch.equal(counts.cpu(), o_counts) and counts.dtype == torch.int64
    assert probs.dtype == dtype
    torch.testing.assert_close(probs.cpu().float(), o_probs.float(), **PROB_TOL[dtype])


def test_ties_resolve_to_lowest_index(pkg, orc, dev):
    # bf16 logits drawn from 5 distinct values: almost every row ties at the k-th place
    g = torch.Generator().manual_seed(3)
    logits = (torch.randint(0, 5, (4096, 8), generator=g).float() * 0.125).bfloat16()
    _, rmap, counts, _, idx = pkg.ops.route_topk(logits.to(dev), 2, want_topk_idx=True)
    _, o_map, o_counts, o_idx = orc.topk_softmax_with_capacity(logits, 2, return_topk=True)
    assert torch.equal(idx.cpu().long(), o_idx)
    assert torch.equal(rmap.cpu(), o_map) and torch.equal(counts.cpu(), o_counts)
    # all-equal row: the first k experts
    flat = torch.zeros(3, 64, dtype=torch.float32)
    _, m, _, _, _ = pkg.ops.route_topk(flat.to(dev), 8)
    assert torch.all(m.cpu()[:, :8]) and not torch.any(m.cpu()[:, 8:])


def test_special_values(pkg, orc, dev):
    logits = torch.tensor([[0.0, -0.0, float("-inf"), 1.0, float("inf"), -1.0, 2.0, 0.5],
                           [float("-inf")] * 6 + [0.0, -5.0]], dtype=torch.float32)
    _, rmap, _, _, idx = pkg.ops.route_topk(logits.to(dev), 3, want_topk_idx=True)
    _, o_map, _, o_idx = orc.topk_softmax_with_capacity(logits, 3, return_topk=True)
    assert torch.equal(idx.cpu().long(), o_idx) and torch.equal(rmap.cpu(), o_map)


def rows_decided_by_the_mathematics(score64, logits, sel_map, rank_dtype, bias=None, eps=2e-6):
    """Rows whose top-k selection cannot depend on the last bits of the score function.

    The reference ranks the scores after rounding them to `rank_dtype` (moe/moe_utils.py:489-504).
    Two evaluations of exp / sigmoid agree to a relative eps, so the rounded score of expert i lies
    in [lo_i, hi_i] = [round(s_i (1 - eps)), round(s_i (1 + eps))].  The pair (i selected, j not)
    is decided when lo_i > hi_j, when both rounded scores are fixed (lo == hi: then the order,
    ties by lowest index included, is the same for every evaluation), or when the two logits are
    equal (same input, same score, tie rule).  A row is decided when all its pairs are."""
    def rounded(v):
        r = v.to(torch.float32).to(rank_dtype).to(torch.float32)
        return r + bias.float() if bias is not None else r
    lo, hi = rounded(score64 * (1 - eps)), rounded(score64 * (1 + eps))
    fixed = lo == hi
    pair_ok = (lo[:, :, None] > hi[:, None, :]) | (fixed[:, :, None] & fixed[:, None, :]) | (
        logits[:, :, None] == logits[:, None, :])
    need = sel_map[:, :, None] & ~sel_map[:, None, :]
    return (~need | pair_ok).all(2).all(1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k", [(1024, 16, 4), (4096, 64, 8), (2048, 256, 8), (3000, 8, 2)])
def test_pre_softmax_and_sigmoid_bias_selection_bit_exact(pkg, orc, dev, dtype, T, E, k):
    """moe/moe_utils.py:489-504: softmax before top-k and sigmoid (+ expert bias) rank scores that
    went through exp.  The selection must equal the oracle's on every row that the mathematics
    decides (see rows_decided_by_the_mathematics); the undecided rows are counted and are few."""
    logits = make_logits(T, E, dtype, seed=5 * T + E)
    lg = logits.to(dev)
    l64 = logits.double()
    print("case", dtype, T, E, k, flush=True)
    # softmax before top-k
    p, m, c = pkg.topk_softmax_with_capacity(lg, k, use_pre_softmax=True)
    op, om, oc = orc.topk_softmax_with_capacity(logits, k, use_pre_softmax=True)
    decided = rows_decided_by_the_mathematics(torch.softmax(l64, -1), logits, om, dtype)
    same = (m.cpu() == om).all(1)
    print("pre-softmax: undecided rows", int((~decided).sum()), "of", T, "; rows that differ",
          int((~same).sum()), flush=True)
    assert (~decided).float().mean().item() < 0.01
    assert torch.equal(m.cpu()[decided], om[decided]), "selection differs on a decided row"
    assert int(c.sum()) == T * k and torch.equal(c.cpu(), m.cpu().sum(0))
    torch.testing.assert_close(p.cpu().float()[same], op.float()[same], **PROB_TOL[dtype])
    # sigmoid scores with an expert bias that changes the selection
    bias = torch.linspace(-0.5, 0.5, E)
    p, m, c = pkg.topk_softmax_with_capacity(lg, k, score_function="sigmoid", expert_bias=bias.to(dev))
    op, om, oc = orc.topk_softmax_with_capacity(logits, k, score_function="sigmoid", expert_bias=bias)
    _, om_nobias, _ = orc.topk_softmax_with_capacity(logits, k, score_function="sigmoid")
    assert not torch.equal(om, om_nobias), "the bias must change the selection for this to test it"
    decided = rows_decided_by_the_mathematics(torch.sigmoid(l64), logits, om, dtype, bias=bias)
    same = (m.cpu() == om).all(1)
    print("sigmoid + bias: undecided rows", int((~decided).sum()), "of", T, "; rows that differ",
          int((~same).sum()), flush=True)
    assert (~decided).float().mean().item() < 0.01
    assert torch.equal(m.cpu()[decided], om[decided]), "selection differs on a decided row"
    assert torch.equal(c.cpu(), m.cpu().sum(0))
    torch.testing.assert_close(p.cpu().float()[same], op.float()[same], **PROB_TOL[dtype])
    # sigmoid without bias
    p, m, c = pkg.topk_softmax_with_capacity(lg, k, score_function="sigmoid")
    decided = rows_decided_by_the_mathematics(torch.sigmoid(l64), logits, om_nobias, dtype)
    assert (~decided).float().mean().item() < 0.01
    assert torch.equal(m.cpu()[decided], om_nobias[decided])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_public_signature_and_variants(pkg, orc, dev, dtype):
    T, E, k = 1024, 16, 4
    logits = make_logits(T, E, dtype, seed=11)
    lg = logits.to(dev)
    # scaling factor
    p, m, c = pkg.topk_softmax_with_capacity(lg, k, scaling_factor=2.5)
    op, om, oc = orc.topk_softmax_with_capacity(logits, k, scaling_factor=2.5)
    assert torch.equal(m.cpu(), om) and torch.equal(c.cpu(), oc)
    torch.testing.assert_close(p.cpu().float(), op.float(), **PROB_TOL[dtype])
    with pytest.raises(ValueError):
        pkg.topk_softmax_with_capacity(lg, k, score_function="tanh")
    with pytest.raises(AssertionError):
        pkg.topk_softmax_with_capacity(lg.view(-1), k)


def test_group_limited_routing(pkg, orc, dev):
    T, E, k, G, gk = 2048, 64, 8, 8, 4
    logits = make_logits(T, E, torch.float32, seed=21)
    p, m, c = pkg.topk_softmax_with_capacity(logits.to(dev), k, num_groups=G, group_topk=gk)
    op, om, oc = orc.topk_softmax_with_capacity(logits, k, num_groups=G, group_topk=gk)
    assert torch.equal(m.cpu(), om) and torch.equal(c.cpu(), oc)
    torch.testing.assert_close(p.cpu(), op, rtol=1e-5, atol=1e-6)
    # every token stays inside gk groups
    groups = m.cpu().view(T, G, E // G).any(-1).sum(-1)
    assert torch.all(groups <= gk)
    v, i = pkg.moe_utils.group_limited_topk(logits.to(dev), k, T, E, G, gk)
    ov, oi = orc.group_limited_topk(logits, k, T, E, G, gk)
    assert torch.equal(i.cpu(), oi) and torch.equal(v.cpu(), ov)


@pytest.mark.parametrize("T,E,k,dtype,factor", [(512, 8, 2, torch.float32, 0.75),
                                                (3000, 60, 6, torch.float32, 0.5),
                                                (2048, 8, 2, torch.bfloat16, 0.6),   # many equal gates
                                                (100, 4, 2, torch.float32, 4.0),     # capacity > routed
                                                (1500, 256, 8, torch.bfloat16, 1.0)])
def test_capacity_variants(pkg, orc, dev, T, E, k, dtype, factor):
    """Capacity selection bit-exact against the oracle for both drop policies, with and without
    padding: the same tie rule (lowest token index among equal keys) on both sides."""
    logits = make_logits(T, E, dtype, seed=31 + T)
    for policy in ("probs", "position"):
        for pad in (False, True):
            p, m, c = pkg.topk_softmax_with_capacity(logits.to(dev), k, capacity_factor=factor,
                                                     pad_to_capacity=pad, drop_policy=policy)
            op, om, oc = orc.topk_softmax_with_capacity(logits, k, capacity_factor=factor,
                                                        pad_to_capacity=pad, drop_policy=policy)
            assert torch.equal(c.cpu(), oc)
            assert torch.equal(m.cpu(), om), (policy, pad)
            assert p.dtype == dtype
            torch.testing.assert_close(p.cpu().float(), op.float(), rtol=1e-5, atol=1e-6)
            cap = orc.get_capacity(T * k, E, factor)
            assert int(m.sum(0).max()) <= cap
            if pad:
                assert torch.all(m.sum(0).cpu() == min(cap, T))


def test_capacity_gradient_flows_only_through_kept_gates(pkg, orc, dev):
    T, E, k = 700, 8, 2
    logits = make_logits(T, E, torch.float32, seed=77)
    lg = logits.to(dev).requires_grad_(True)
    p, m, _ = pkg.topk_softmax_with_capacity(lg, k, capacity_factor=0.5)
    g = torch.randn(T, E, generator=torch.Generator().manual_seed(1))
    p.backward(g.to(dev))
    lo = logits.clone().requires_grad_(True)
    op, om, _ = orc.topk_softmax_with_capacity(lo, k, capacity_factor=0.5)
    op.backward(g)
    assert torch.equal(m.cpu(), om)
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("E,k", [(8, 2), (64, 8), (12, 3), (256, 8), (512, 4), (100, 6)])
def test_loss_statistics(pkg, orc, dev, E, k):
    T = 3000
    logits = make_logits(T, E, torch.float32, seed=41, scale=1.0)
    _, _, counts, stats, _ = pkg.ops.route_topk(logits.to(dev), k, want_stats=True)
    scores = torch.softmax(logits.double(), -1)
    torch.testing.assert_close(stats[:E].cpu().double(), scores.sum(0), rtol=1e-5, atol=1e-4)
    lse2 = torch.logsumexp(logits.double(), -1).square().sum()
    torch.testing.assert_close(stats[E].cpu().double(), lse2, rtol=1e-5, atol=1e-4)
    # the loss values the router logs
    aux = orc.switch_load_balancing_loss(scores.float(), counts.cpu(), k, 0.01)
    got = (stats[:E].cpu() * counts.cpu()).sum() * (E * 0.01 / (T * T * k))
    torch.testing.assert_close(got, aux, rtol=1e-5, atol=1e-8)
    # deterministic: same bits on a second run
    _, _, _, stats2, _ = pkg.ops.route_topk(logits.to(dev), k, want_stats=True)
    assert torch.equal(stats, stats2)


@pytest.mark.parametrize("variant", ["default", "scaling", "pre_softmax", "sigmoid", "sigmoid_k1"])
def test_router_backward(pkg, orc, dev, variant):
    T, E, k = 600, 16, 4
    kw = {}
    if variant == "scaling":
        kw = dict(scaling_factor=1.7)
    elif variant == "pre_softmax":
        kw = dict(use_pre_softmax=True)
    elif variant.startswith("sigmoid"):
        kw = dict(score_function="sigmoid")
        if variant == "sigmoid_k1":
            k = 1
    logits = make_logits(T, E, torch.float32, seed=51, scale=1.0)
    g = torch.Generator().manual_seed(52)
    go = torch.randn(T, E, generator=g)
    lg = logits.to(dev).requires_grad_(True)
    p, m, _ = pkg.topk_softmax_with_capacity(lg, k, **kw)
    p.backward(go.to(dev))
    lo = logits.clone().requires_grad_(True)
    op, om, _ = orc.topk_softmax_with_capacity(lo, k, **kw)
    assert torch.equal(m.cpu(), om)
    op.backward(go)
    torch.testing.assert_close(lg.grad.cpu(), lo.grad, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("score_fn", ["softmax", "sigmoid"])
def test_router_module_aux_and_z_loss_gradients(pkg, orc, dev, score_fn):
    """TopKRouter with aux-loss + z-loss: the fused backward equals autograd of main + aux + z."""
    S, B, H, E, k = 64, 4, 128, 8, 2
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_router_topk=k,
                        moe_router_load_balancing_type="aux_loss", moe_aux_loss_coeff=0.01,
                        moe_z_loss_coeff=0.001, moe_router_score_function=score_fn,
                        moe_router_dtype="fp32", params_dtype=torch.float32)
    g = torch.Generator().manual_seed(61)
    x = torch.randn(S, B, H, generator=g)
    w = 0.02 * torch.randn(E, H, generator=g) * 10
    go = torch.randn(S * B, E, generator=g)
    router = pkg.GalvatronMoERouter(cfg, device=dev).train()
    with torch.no_grad():
        router.router.weight.copy_(w.to(dev))
    pkg.moe_utils.MoEAuxLossAutoScaler.set_loss_scale(torch.tensor(2.0, device=dev))
    try:
        xg = x.to(dev).requires_grad_(True)
        probs, rmap = router(xg)
        probs.backward(go.to(dev))
    finally:
        pkg.moe_utils.MoEAuxLossAutoScaler.main_loss_backward_scale = None
    xo = x.clone().requires_grad_(True)
    wo = w.clone().requires_grad_(True)
    kw = dict(score_function=score_fn)
    o_probs, o_map, aux_total = orc.router_forward(xo.view(-1, H), wo, k, "fp32", "aux_loss", 0.01,
                                                   0.001, **kw)
    assert torch.equal(rmap.cpu(), o_map)
    ((o_probs * go).sum() + 2.0 * aux_total).backward()
    torch.testing.assert_close(probs.detach().cpu(), o_probs.detach(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(xg.grad.cpu(), xo.grad, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(router.router.weight.grad.cpu(), wo.grad, rtol=1e-3, atol=1e-5)
    # logged loss values
    lg = orc.gate_logits(x.view(-1, H), w, "fp32")
    torch.testing.assert_close(router.router.last_z_loss.cpu(), orc.z_loss(lg, 0.001), rtol=1e-5, atol=1e-9)
    if score_fn == "softmax":
        aux = orc.switch_load_balancing_loss(torch.softmax(lg, -1), o_map.sum(0), k, 0.01)
        torch.testing.assert_close(router.router.last_aux_loss.cpu(), aux, rtol=1e-5, atol=1e-9)
