"""Sequence-level load-balancing loss, sinkhorn routing and the router bookkeeping on the GPU,
through the C ABI, against the oracle: counts and selections bit-exact, loss values and gradients
within fp32 tolerance (written at each comparison)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def make_logits(T, E, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(T, E, generator=g)).to(dtype)


def oracle_scores(logits, score_fn, k):
    if score_fn == "softmax":
        return torch.softmax(logits, dim=-1, dtype=torch.float32)
    s = torch.sigmoid(logits)
    return s / (s.sum(dim=-1, keepdim=True) + 1e-20) if k > 1 else s


# ------------------------------------------------------------------------------------------
# sequence-level loss
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("score_fn", ["softmax", "sigmoid"])
@pytest.mark.parametrize("S,B,E,k", [(64, 4, 8, 2), (33, 5, 64, 8), (17, 3, 60, 6), (16, 2, 256, 8),
                                     (1, 7, 8, 1), (300, 1, 16, 1)])
def test_seq_aux_loss_kernel(pkg, orc, dev, score_fn, S, B, E, k):
    print("case", score_fn, S, B, E, k, flush=True)
    coeff = 0.03
    logits = make_logits(S * B, E, torch.float32, seed=S + E)
    logits[torch.arange(S * B) % B == 0] += torch.linspace(0, 2, E)  # sequence 0 is skewed
    _, rmap, _ = orc.topk_softmax_with_capacity(logits, k, score_function=score_fn)
    lo = logits.clone().requires_grad_(True)
    want = orc.sequence_load_balancing_loss(oracle_scores(lo, score_fn, k), rmap, B, S, k, coeff)
    want.backward()
    loss, counts, scores = pkg.ops.seq_aux_loss(logits.to(dev), rmap.to(dev), B, S, k, coeff, score_fn)
    assert torch.equal(counts.cpu(), rmap.view(S, B, E).sum(0).float())  # integers: exact
    torch.testing.assert_close(scores.cpu(), oracle_scores(logits, score_fn, k).view(S, B, E).sum(0),
                               rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(loss.cpu(), want.detach(), rtol=1e-5, atol=1e-9)
    grad = pkg.ops.seq_aux_loss_bwd(logits.to(dev), counts, B, S, k, coeff, score_fn,
                                    torch.tensor([2.5], device=dev))
    torch.testing.assert_close(grad.cpu(), 2.5 * lo.grad, rtol=1e-4, atol=1e-9)
    # same bits on a second run (fixed summation order)
    loss2, _, scores2 = pkg.ops.seq_aux_loss(logits.to(dev), rmap.to(dev), B, S, k, coeff, score_fn)
    assert torch.equal(loss, loss2) and torch.equal(scores, scores2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_seq_aux_loss_16bit_logits(pkg, orc, dev, dtype):
    S, B, E, k, coeff = 128, 4, 8, 2, 0.01
    logits = make_logits(S * B, E, dtype, seed=5)
    _, rmap, _ = orc.topk_softmax_with_capacity(logits, k)
    want = orc.sequence_load_balancing_loss(oracle_scores(logits, "softmax", k), rmap, B, S, k, coeff)
    loss, _, _ = pkg.ops.seq_aux_loss(logits.to(dev), rmap.to(dev), B, S, k, coeff)
    torch.testing.assert_close(loss.cpu(), want, rtol=1e-5, atol=1e-9)


def test_sequence_load_balancing_loss_func_on_scores(pkg, orc, dev):
    """The reference-named function: scores in, differentiable in the scores."""
    S, B, E, k, coeff = 40, 3, 12, 3, 0.2
    logits = make_logits(S * B, E, torch.float32, seed=9)
    _, rmap, _ = orc.topk_softmax_with_capacity(logits, k)
    so = torch.softmax(logits, -1).requires_grad_(True)
    want = orc.sequence_load_balancing_loss(so, rmap, B, S, k, coeff)
    (3.0 * want).backward()
    sg = so.detach().to(dev).requires_grad_(True)
    got = pkg.moe_utils.sequence_load_balancing_loss_func(sg, rmap.to(dev), B, S, k, coeff)
    (3.0 * got).backward()
    torch.testing.assert_close(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(sg.grad.cpu(), so.grad, rtol=1e-5, atol=1e-10)


@pytest.mark.parametrize("score_fn,capacity", [("softmax", None), ("sigmoid", None), ("softmax", 0.6)])
def test_router_module_seq_aux_loss(pkg, orc, dev, score_fn, capacity):
    """TopKRouter(seq_aux_loss): routing bit-exact, loss value and the gradients of input and gate
    weight equal autograd of main + scale * (seq aux + z) on the oracle."""
    S, B, H, E, k = 48, 3, 64, 8, 2
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_router_topk=k,
                        moe_router_load_balancing_type="seq_aux_loss", moe_aux_loss_coeff=0.02,
                        moe_z_loss_coeff=0.001, moe_router_score_function=score_fn,
                        moe_expert_capacity_factor=capacity, moe_router_dtype="fp32",
                        params_dtype=torch.float32)
    g = torch.Generator().manual_seed(71)
    x = torch.randn(S, B, H, generator=g)
    w = 0.2 * torch.randn(E, H, generator=g)
    go = torch.randn(S * B, E, generator=g)
    router = pkg.GalvatronMoERouter(cfg, device=dev).train()
    with torch.no_grad():
        router.router.weight.copy_(w.to(dev))
    pkg.moe_utils.clear_aux_losses_tracker()
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
    if capacity is not None:
        kw.update(capacity_factor=capacity)
    o_probs, o_map, aux_total = orc.router_forward(xo.view(-1, H), wo, k, "fp32", "seq_aux_loss", 0.02,
                                                   0.001, seq_shape=(S, B), **kw)
    assert torch.equal(rmap.cpu(), o_map)
    ((o_probs * go).sum() + 2.0 * aux_total).backward()
    torch.testing.assert_close(probs.detach().cpu(), o_probs.detach(), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(xg.grad.cpu(), xo.grad, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(router.router.weight.grad.cpu(), wo.grad, rtol=1e-3, atol=1e-5)
    lg = orc.gate_logits(x.view(-1, H), w, "fp32")
    want = orc.sequence_load_balancing_loss(oracle_scores(lg, score_fn, k), o_map, B, S, k, 0.02)
    torch.testing.assert_close(router.router.last_aux_loss.cpu(), want, rtol=1e-5, atol=1e-9)
    tracker = pkg.moe_utils.get_moe_layer_wise_logging_tracker()
    torch.testing.assert_close(tracker["load_balancing_loss"]["values"].cpu()[0], want / 0.02,
                               rtol=1e-5, atol=1e-9)
    pkg.moe_utils.clear_aux_losses_tracker()


# ------------------------------------------------------------------------------------------
# sinkhorn
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("T,E", [(2048, 8), (1000, 64), (513, 60), (256, 256), (4, 3), (16384, 8)])
def test_sinkhorn_kernel(pkg, orc, dev, T, E):
    print("case", T, E, flush=True)
    logits = make_logits(T, E, torch.float32, seed=T + E) + torch.linspace(0, 1.5, E)
    want = orc.sinkhorn(logits.clone())
    got, iters = pkg.ops.sinkhorn(logits.to(dev), want_iters=True)
    assert got.dtype == torch.float32 and 1 <= int(iters) < 1000
    # same iteration in another summation order; the stopping test may fall one iteration apart
    torch.testing.assert_close(got.cpu(), want, rtol=2e-3, atol=1e-9)
    torch.testing.assert_close(got.cpu().sum(0), torch.full((E,), 1.0 / E), rtol=1e-4, atol=0)
    again, _ = pkg.ops.sinkhorn(logits.to(dev), want_iters=True)
    assert torch.equal(got, again)
    # tolerance at or above the initial error: no iteration, exp(logits) comes back
    none, iters0 = pkg.ops.sinkhorn(logits.to(dev), tol=2e9, want_iters=True)
    assert int(iters0) == 0
    torch.testing.assert_close(none.cpu(), torch.exp(logits), rtol=1e-5, atol=0)
    # the iteration cap ends the loop
    _, capped = pkg.ops.sinkhorn(logits.to(dev), tol=0.0, max_iters=3, want_iters=True)
    assert int(capped) == 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,k", [(8, 2), (8, 1), (64, 6)])
def test_router_module_sinkhorn(pkg, orc, dev, dtype, E, k):
    """TopKRouter(sinkhorn).  Training: the map is the oracle's top-k (lowest index on ties) of the
    normalised costs the device computed, bit-exact, and agrees with the all-CPU oracle wherever
    the k-th and (k+1)-th cost are not within rounding of each other; scores and gradients follow
    autograd of the oracle with that map.  Evaluation: bit-exact top-k of the activation."""
    S, B, H = 96, 4, 64
    T = S * B
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_router_topk=k,
                        moe_router_load_balancing_type="sinkhorn", moe_aux_loss_coeff=0.0,
                        moe_z_loss_coeff=0.002, params_dtype=dtype)
    g = torch.Generator().manual_seed(81)
    x = torch.randn(S, B, H, generator=g).to(dtype)
    w = (0.2 * torch.randn(E, H, generator=g)).to(dtype)
    go = torch.randn(T, E, generator=g).to(dtype)
    router = pkg.GalvatronMoERouter(cfg, device=dev).train()
    with torch.no_grad():
        router.router.weight.copy_(w.to(dev))
    xg = x.to(dev).requires_grad_(True)
    scores, rmap = router(xg)
    scores.backward(go.to(dev))
    logits = router.router.gating(x.to(dev)).detach().view(T, E)  # the very logits the device routed
    norm = pkg.ops.sinkhorn(logits).cpu()
    _, idx = orc.topk_tie_low_index(norm, k)
    want_map = torch.zeros(T, E).scatter(1, idx, 1).bool()
    assert torch.equal(rmap.cpu(), want_map)
    _, cpu_map = orc.sinkhorn_routing(logits.cpu(), k, training=True)
    assert (rmap.cpu() != cpu_map).any(1).float().mean() < 0.01
    # floating point: oracle in fp32 on the same logits with the selection held fixed
    lo = logits.cpu().float().requires_grad_(True)
    act = torch.sigmoid(lo) if k == 1 else torch.softmax(lo, -1)
    loss = (act * want_map * go.float()).sum() + orc.z_loss(lo, 0.002)
    loss.backward()
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=1e-2)
    torch.testing.assert_close(scores.detach().cpu().float(), (act * want_map).detach(), **tol)
    # d logits -> d x through the gate weight; compare at the logits level via the weight gradient
    wo = w.float()
    torch.testing.assert_close(xg.grad.cpu().float(), (lo.grad @ wo).view(S, B, H),
                               **(dict(rtol=1e-3, atol=1e-5) if dtype == torch.float32 else tol))
    # evaluation mode
    router.eval()
    with torch.no_grad():
        e_scores, e_map = router(x.to(dev))
    o_scores, o_map = orc.sinkhorn_routing(logits.cpu(), k, training=False)
    assert torch.equal(e_map.cpu(), o_map)
    torch.testing.assert_close(e_scores.cpu().float(), o_scores.float(), **tol)


# ------------------------------------------------------------------------------------------
# bookkeeping
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("E", [8, 60, 256])
def test_router_bookkeeping_kernel(pkg, orc, dev, E):
    T, k = 2000, 2
    logits = make_logits(T, E, torch.float32, seed=E)
    _, _, counts, stats, _ = pkg.ops.route_topk(logits.to(dev), k, want_stats=True)
    slot = torch.tensor([1.5, 7.0], device=dev)
    zslot = torch.tensor([0.25], device=dev)
    local = torch.arange(E, dtype=torch.float32, device=dev)
    aux_f, z_f = E * 0.01 / (T * T * k), 0.001 / T
    aux, z = pkg.ops.router_bookkeeping(stats, counts, E, aux_factor=aux_f, z_factor=z_f, want_aux=True,
                                        want_z=True, aux_slot=slot.narrow(0, 1, 1), aux_slot_scale=100.0,
                                        z_slot=zslot, z_slot_scale=1000.0, local_tokens=local)
    _, o_map, o_counts = orc.topk_softmax_with_capacity(logits, k)
    want_aux = orc.switch_load_balancing_loss(torch.softmax(logits, -1), o_counts, k, 0.01)
    want_z = orc.z_loss(logits, 0.001)
    torch.testing.assert_close(aux.cpu(), want_aux, rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(z.cpu(), want_z, rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(slot.cpu(), torch.stack([torch.tensor(1.5), 7.0 + 100.0 * want_aux]),
                               rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(zslot.cpu(), (0.25 + 1000.0 * want_z).reshape(1), rtol=1e-5, atol=1e-9)
    assert torch.equal(local.cpu(), torch.arange(E, dtype=torch.float32) + o_counts.float())
    # counts only
    local2 = torch.zeros(E, device=dev)
    pkg.ops.router_bookkeeping(None, counts, E, local_tokens=local2)
    assert torch.equal(local2.cpu(), o_counts.float())


def test_expert_bias_update_kernel(pkg, orc, dev):
    g = torch.Generator().manual_seed(3)
    tokens = torch.randint(0, 50, (6, 72), generator=g).float()
    tokens[2] = 7.0                      # every expert at the mean: no change
    tokens[3, :36], tokens[3, 36:] = 10.0, 20.0
    bias = torch.randn(6, 72, generator=g)
    got = pkg.moe_utils.get_updated_expert_bias(tokens.to(dev), bias.to(dev), 1e-3)
    assert torch.equal(got.cpu(), orc.get_updated_expert_bias(tokens, bias, 1e-3))
    one = pkg.moe_utils.get_updated_expert_bias(tokens[0].to(dev), bias[0].to(dev), 0.5)
    assert torch.equal(one.cpu(), orc.get_updated_expert_bias(tokens[0], bias[0], 0.5))


def test_router_accumulates_local_tokens_and_tracker(pkg, orc, dev):
    """TopKRouter with expert bias: two forwards add their histograms to local_tokens_per_expert on
    the device; the aux-loss tracker holds loss / coeff summed over the calls."""
    S, B, H, E, k = 64, 2, 64, 16, 4
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_router_topk=k,
                        moe_router_load_balancing_type="aux_loss", moe_aux_loss_coeff=0.01,
                        moe_router_score_function="sigmoid", moe_router_enable_expert_bias=True,
                        moe_router_dtype="fp32", params_dtype=torch.float32, num_layers=3)
    router = pkg.GalvatronMoERouter(cfg, layer_idx=2, device=dev).train()
    pkg.moe_utils.get_moe_layer_wise_logging_tracker().clear()  # other tests tracked one layer
    g = torch.Generator().manual_seed(91)
    total = torch.zeros(E)
    aux_sum = 0.0
    for _ in range(2):
        x = torch.randn(S, B, H, generator=g)
        _, rmap = router(x.to(dev))
        total += rmap.cpu().sum(0).float()
        aux_sum += float(router.router.last_aux_loss) / 0.01
    assert torch.equal(router.router.local_tokens_per_expert.cpu(), total)
    values = pkg.moe_utils.get_moe_layer_wise_logging_tracker()["load_balancing_loss"]["values"].cpu()
    assert values.shape == (3,) and values[0] == 0 and values[2] == 0
    torch.testing.assert_close(values[1], torch.tensor(aux_sum), rtol=1e-5, atol=1e-9)
    pkg.moe_utils.get_moe_layer_wise_logging_tracker().clear()


# ------------------------------------------------------------------------------------------
# the reference's free loss functions (moe/moe_utils.py:14-59, 115-127) on the device kernels
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,k", [(2048, 8, 2), (8192, 64, 8), (777, 60, 6), (4096, 256, 8), (1, 8, 2)])
def test_switch_load_balancing_loss_func(pkg, orc, dev, dtype, T, E, k):
    """Value against the oracle's closed form on the same probs (fp64 sum as the yardstick for the
    fp32 accumulation), gradient against autograd of the oracle; counts above 256 with bf16 probs
    are not rounded (the sums run in fp32)."""
    print("case", dtype, T, E, k, flush=True)
    coeff = 0.02
    logits = make_logits(T, E, torch.float32, seed=T + E)
    probs = torch.softmax(logits, -1).to(dtype)
    _, rmap, counts = orc.topk_softmax_with_capacity(logits, k)
    po = probs.float().clone().requires_grad_(True)
    want = orc.switch_load_balancing_loss(po, counts, k, coeff)
    want.backward()
    exact = (probs.double().sum(0) * counts.double()).sum() * (E * coeff / (T * T * k))
    pg = probs.to(dev).requires_grad_(True)
    got = pkg.moe_utils.switch_load_balancing_loss_func(pg, counts.to(dev), k, coeff)
    assert got.dtype == dtype and got.dim() == 0
    if dtype == torch.float32:
        torch.testing.assert_close(got.cpu().double(), exact, rtol=1e-5, atol=1e-12)
        torch.testing.assert_close(got.cpu(), want.detach(), rtol=1e-5, atol=1e-12)
    else:
        torch.testing.assert_close(got.cpu().double(), exact, rtol=1e-2, atol=1e-12)  # one bf16 rounding
    (got * 3.0).backward()
    assert pg.grad.dtype == dtype
    torch.testing.assert_close(pg.grad.cpu().float(), 3.0 * po.grad,
                               **(dict(rtol=1e-6, atol=1e-12) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-12)))
    # float counts are accepted too (the reference multiplies whatever it is given)
    again = pkg.moe_utils.switch_load_balancing_loss_func(probs.to(dev), counts.float().to(dev), k, coeff)
    assert torch.equal(again, got.detach())


def test_switch_loss_equals_coeff_under_uniform_routing(pkg, dev):
    T, E, k, coeff = 1024, 8, 2, 0.05
    probs = torch.full((T, E), 1.0 / E, device=dev)
    counts = torch.full((E,), T * k // E, dtype=torch.int64, device=dev)
    got = pkg.moe_utils.switch_load_balancing_loss_func(probs, counts, k, coeff)
    torch.testing.assert_close(got.cpu(), torch.tensor(coeff), rtol=1e-6, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E", [(2048, 8), (8192, 64), (777, 60), (4096, 256), (3, 5)])
def test_z_loss_func(pkg, orc, dev, dtype, T, E):
    print("case", dtype, T, E, flush=True)
    coeff = 1e-3
    logits = make_logits(T, E, dtype, seed=3 * T + E, scale=2.0)
    lo = logits.float().clone().requires_grad_(True)
    want = orc.z_loss(lo, coeff)
    want.backward()
    lg = logits.to(dev).requires_grad_(True)
    got = pkg.moe_utils.z_loss_func(lg, coeff)
    assert got.dtype == dtype and got.dim() == 0
    tol = dict(rtol=1e-5, atol=1e-10) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-10)
    torch.testing.assert_close(got.cpu().float(), want.detach(), **tol)
    (got * 2.0).backward()
    # the gradient is stored in the dtype of the logits; fp16 has a spacing of 6e-8 near zero
    gtol = {torch.float32: dict(rtol=1e-4, atol=1e-10), torch.bfloat16: dict(rtol=1e-2, atol=1e-9),
            torch.float16: dict(rtol=1e-2, atol=1e-7)}[dtype]
    torch.testing.assert_close(lg.grad.cpu().float(), 2.0 * lo.grad, **gtol)
    # constant rows: logsumexp = c + log E exactly representable cases
    flat = torch.full((64, 16), 0.5, device=dev)
    got = pkg.moe_utils.z_loss_func(flat, 1.0)
    torch.testing.assert_close(got.cpu(), ((0.5 + torch.log(torch.tensor(16.0))) ** 2).clone(),
                               rtol=1e-6, atol=0)


def test_sinkhorn_free_function_keeps_the_dtype_of_its_input(pkg, orc, dev):
    cost = make_logits(256, 8, torch.bfloat16, seed=9)
    got = pkg.moe_utils.sinkhorn(cost.to(dev))
    assert got.dtype == torch.bfloat16
    want = orc.sinkhorn(cost.float().clone())
    torch.testing.assert_close(got.cpu().float(), want, rtol=2e-2, atol=1e-4)
    assert pkg.ops.SINKHORN_MAX_ITERS <= 10000
    _, iters = pkg.ops.sinkhorn(cost.to(dev), tol=0.0, want_iters=True)
    assert int(iters.item()) <= pkg.ops.SINKHORN_MAX_ITERS


def test_input_jitter_promotes_like_the_reference(pkg, dev):
    """moe/router.py:350-369: the noise is an fp32 sample, so a bf16 input comes back as fp32,
    inside [x (1 - eps), x (1 + eps)]; the router still runs on it."""
    cfg = pkg.MoEConfig(hidden_size=64, num_moe_experts=8, moe_ffn_hidden_size=64,
                        moe_input_jitter_eps=0.01, params_dtype=torch.bfloat16)
    router = pkg.TopKRouter(cfg).to(dev)
    x = torch.randn(16, 2, 64, device=dev).bfloat16()
    j = router.apply_input_jitter(x)
    assert j.dtype == torch.float32
    r = j / x.float()
    assert float(r.min()) >= 0.99 - 1e-6 and float(r.max()) <= 1.01 + 1e-6 and float(r.std()) > 0
    probs, rmap = router(x)
    assert probs.dtype == torch.float32 and int(rmap.sum()) == 32 * cfg.moe_router_topk


# ------------------------------------------------------------------------------------------
# the router's step-by-step methods (moe/router.py:173-231, 278-348)
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("score_fn,k", [("softmax", 2), ("sigmoid", 4), ("sigmoid", 1)])
def test_router_step_by_step_methods_compose_to_the_fused_routing(pkg, orc, dev, score_fn, k):
    """Routing composed as the reference composes it (apply_z_loss, topk_softmax_with_capacity,
    compute_routing_scores_for_aux_loss, switch_load_balancing_loss_func, apply_load_balancing_loss)
    gives the probabilities, map, tracked losses and logits gradient of the fused `routing`."""
    from functools import partial

    T, E, H = 512, 16, 64
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_router_topk=k,
                        moe_router_load_balancing_type="aux_loss", moe_aux_loss_coeff=0.02,
                        moe_z_loss_coeff=1e-3, moe_router_score_function=score_fn,
                        moe_router_dtype="fp32", params_dtype=torch.float32, num_layers=1)
    router = pkg.GalvatronMoERouter(cfg, layer_idx=1, device=dev).train().router
    logits = make_logits(T, E, torch.float32, seed=17 + k, scale=2.0).to(dev)
    gp = torch.randn(T, E, generator=torch.Generator().manual_seed(3)).to(dev)
    tracker = pkg.moe_utils.get_moe_layer_wise_logging_tracker

    # scores against the oracle's formula
    scores = router.compute_routing_scores_for_aux_loss(logits)
    torch.testing.assert_close(scores.cpu(), oracle_scores(logits.cpu(), score_fn, k), rtol=1e-5, atol=1e-7)
    assert scores.dtype == torch.float32

    def run(fused):
        tracker().clear()
        x = logits.clone().requires_grad_(True)
        if fused:
            probs, rmap = router.routing(x.view(T, 1, E))
        else:
            lz = router.apply_z_loss(x)
            probs, rmap, tokens = pkg.topk_softmax_with_capacity(lz, k, score_function=score_fn)
            sc = router.compute_routing_scores_for_aux_loss(lz)
            probs = router.apply_load_balancing_loss(
                probs, partial(pkg.moe_utils.switch_load_balancing_loss_func, probs=sc,
                               tokens_per_expert=tokens, topk=k))
        (probs * gp).sum().backward()
        tr = {n: v["values"].cpu().clone() for n, v in tracker().items()}
        return probs.detach().cpu(), rmap.cpu(), x.grad.cpu(), tr

    pf, mf, gf, tf = run(True)
    ps, ms, gs, ts = run(False)
    tracker().clear()
    assert torch.equal(mf, ms)
    torch.testing.assert_close(ps, pf, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(gs, gf, rtol=1e-4, atol=1e-7)
    for name in ("load_balancing_loss", "z_loss"):
        torch.testing.assert_close(ts[name], tf[name], rtol=1e-5, atol=1e-9)
    # the same two through the remaining method
    tracker().clear()
    pa, ma = router.aux_loss_load_balancing(logits.clone().requires_grad_(True))
    tracker().clear()
    assert torch.equal(ma.cpu(), mf) and torch.equal(pa.detach().cpu(), pf)
