"""Pins the CPU oracle (oracle/moe_oracle.py) against what the mathematics fixes: brute force on
tiny inputs, closed forms, library routines on special cases and invariants.  The reference holds
no golden vectors for this path, so these checks are what stands between a typo in the oracle and
a wrong parity verdict; each one is chosen so that a dropped term, a wrong index or a transposed
operand fails it.  CPU only."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F


# ------------------------------------------------------------------------------------------
# top-k
# ------------------------------------------------------------------------------------------

def brute_topk(row, k):
    """Pure-Python top-k: repeatedly take the largest remaining value, lowest index on ties."""
    taken, out = set(), []
    for _ in range(k):
        best = None
        for e, v in enumerate(row):
            if e in taken:
                continue
            if best is None or v > row[best]:
                best = e
        taken.add(best)
        out.append(best)
    return out


def test_topk_matches_brute_force_with_ties(orc):
    g = torch.Generator().manual_seed(0)
    # few distinct values -> many ties, including ties at the k-th place
    scores = torch.randint(0, 4, (200, 12), generator=g).float()
    for k in (1, 2, 5):
        _, idx = orc.topk_tie_low_index(scores, k)
        for t in range(scores.shape[0]):
            assert idx[t].tolist() == brute_topk(scores[t].tolist(), k)


def test_topk_equals_torch_topk_on_tie_free_rows(orc):
    g = torch.Generator().manual_seed(1)
    scores = torch.randn(512, 64, generator=g)
    vals, idx = orc.topk_tie_low_index(scores, 8)
    tv, ti = torch.topk(scores, 8, dim=1)
    assert torch.equal(idx, ti) and torch.equal(vals, tv)


def test_routing_invariants_and_closed_form_probs(orc):
    g = torch.Generator().manual_seed(2)
    T, E, k = 300, 16, 4
    logits = 0.02 * torch.randn(T, E, generator=g)
    probs, rmap, counts = orc.topk_softmax_with_capacity(logits, k)
    assert rmap.dtype == torch.bool and counts.dtype == torch.int64
    assert torch.all(rmap.sum(1) == k)
    assert counts.sum().item() == T * k
    assert torch.equal(counts, rmap.sum(0))
    assert torch.all((probs > 0) == rmap)
    torch.testing.assert_close(probs.sum(1), torch.ones(T), rtol=1e-6, atol=1e-6)
    # brute force on every row: selected set and gate values by hand
    for t in range(0, T, 7):
        sel = brute_topk(logits[t].tolist(), k)
        assert sorted(sel) == torch.nonzero(rmap[t]).flatten().tolist()
        z = [math.exp(logits[t, e].item()) for e in sel]
        for e, ze in zip(sel, z):
            assert abs(probs[t, e].item() - ze / sum(z)) < 1e-6


def test_gates_equal_softmax_then_renormalise(orc):
    """HF-Mixtral computes softmax over all experts, takes top-k, renormalises: same gates."""
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(128, 8, generator=g)
    probs, rmap, _ = orc.topk_softmax_with_capacity(logits, 2)
    full = torch.softmax(logits, dim=-1)
    w, sel = torch.topk(full, 2, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    dense = torch.zeros_like(logits).scatter(1, sel, w)
    torch.testing.assert_close(probs, dense, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(orc.probs_from_map(logits, rmap), probs, rtol=1e-6, atol=1e-7)


def test_pre_softmax_sigmoid_and_scaling_variants(orc):
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(64, 8, generator=g)
    p, m, _ = orc.topk_softmax_with_capacity(logits, 2, use_pre_softmax=True, scaling_factor=2.5)
    full = torch.softmax(logits, -1)
    torch.testing.assert_close(p, full * m * 2.5)
    assert torch.equal(m, orc.topk_softmax_with_capacity(logits, 2)[1])  # softmax is monotone
    bias = torch.tensor([10.0] + [0.0] * 7)
    p, m, _ = orc.topk_softmax_with_capacity(logits, 2, score_function="sigmoid", expert_bias=bias)
    assert torch.all(m[:, 0])  # a large bias forces expert 0 in
    s = torch.sigmoid(logits) * m
    torch.testing.assert_close(p, s / s.sum(-1, keepdim=True))
    with pytest.raises(ValueError):
        orc.topk_softmax_with_capacity(logits, 2, score_function="tanh")


def test_group_limited_topk_brute_force(orc):
    g = torch.Generator().manual_seed(5)
    T, E, G, gk, k = 50, 16, 4, 2, 4
    scores = torch.rand(T, E, generator=g)
    _, idx = orc.group_limited_topk(scores, k, T, E, G, gk)
    for t in range(T):
        row = scores[t].tolist()
        gs = []
        for gi in range(G):
            members = sorted(row[gi * 4:(gi + 1) * 4], reverse=True)
            gs.append(sum(members[: k // gk]))
        keep = brute_topk(gs, gk)
        masked = [v if (e // 4) in keep else -float("inf") for e, v in enumerate(row)]
        assert idx[t].tolist() == brute_topk(masked, k)


def test_capacity_drops_lowest_probs(orc):
    g = torch.Generator().manual_seed(6)
    T, E, k = 64, 4, 2
    logits = torch.randn(T, E, generator=g)
    p0, m0, c0 = orc.topk_softmax_with_capacity(logits, k)
    cap = orc.get_capacity(T * k, E, 0.5)
    assert cap == math.ceil(T * k / E * 0.5)
    p, m, c = orc.topk_softmax_with_capacity(logits, k, capacity_factor=0.5)
    assert torch.equal(c, c0)  # counts are reported before dropping
    assert torch.all(m.sum(0) <= cap) and torch.all(m <= m0)
    for e in range(E):
        kept = p0[:, e][m[:, e]]
        dropped = p0[:, e][m0[:, e] & ~m[:, e]]
        if kept.numel() and dropped.numel():
            assert kept.min() >= dropped.max()
    # position policy keeps the earliest tokens
    p, m, _ = orc.topk_softmax_with_capacity(logits, k, capacity_factor=0.5, drop_policy="position")
    for e in range(E):
        routed = torch.nonzero(m0[:, e]).flatten()[:cap]
        assert torch.equal(torch.nonzero(m[:, e]).flatten(), routed)


# ------------------------------------------------------------------------------------------
# losses
# ------------------------------------------------------------------------------------------

def test_aux_loss_uniform_routing_equals_coeff(orc):
    T, E, k, coeff = 64, 8, 2, 0.01
    probs = torch.full((T, E), 1.0 / E)
    counts = torch.full((E,), T * k // E)
    assert abs(orc.switch_load_balancing_loss(probs, counts, k, coeff).item() - coeff) < 1e-9


def test_aux_loss_matches_paper_formula(orc):
    g = torch.Generator().manual_seed(7)
    T, E, k, coeff = 40, 4, 2, 0.3
    probs = torch.softmax(torch.randn(T, E, generator=g), -1)
    counts = torch.tensor([30, 20, 20, 10])
    want = sum((probs[:, e].sum().item() / T) * (counts[e].item() / (T * k)) for e in range(E)) * E * coeff
    assert abs(orc.switch_load_balancing_loss(probs, counts, k, coeff).item() - want) < 1e-7


def _seq_loss_brute_force(scores, rmap, B, S, k, coeff):
    """Per-sequence loss written out: for each sequence b, f[e] = share of its S*k routed slots that
    expert e took times E, P[e] = mean score of e over the sequence; loss_b = sum_e f P; mean over b."""
    E = scores.shape[1]
    total = 0.0
    for b in range(B):
        loss_b = 0.0
        for e in range(E):
            cnt = sum(1 for s in range(S) if bool(rmap[s * B + b, e]))
            mean_score = sum(float(scores[s * B + b, e]) for s in range(S)) / S
            loss_b += (cnt * E / (S * k)) * mean_score
        total += loss_b
    return coeff * total / B


def test_seq_aux_loss_brute_force(orc):
    """Unequal sequences, B != S: a swapped (seq, batch) view or a per-batch instead of per-sequence
    count changes the value."""
    g = torch.Generator().manual_seed(11)
    B, S, E, k, coeff = 3, 5, 6, 2, 0.7
    logits = torch.randn(S * B, E, generator=g, dtype=torch.float64)
    logits[torch.arange(S * B) % B == 1] += torch.linspace(0, 3, E, dtype=torch.float64)  # skew sequence 1
    scores = torch.softmax(logits, -1)
    _, rmap, _ = orc.topk_softmax_with_capacity(logits, k)
    got = orc.sequence_load_balancing_loss(scores, rmap, B, S, k, coeff).item()
    want = _seq_loss_brute_force(scores, rmap, B, S, k, coeff)
    assert abs(got - want) < 1e-6 * abs(want), (got, want)
    wrong = _seq_loss_brute_force(scores.view(B, S, E).transpose(0, 1).reshape(S * B, E),
                                  rmap.view(B, S, E).transpose(0, 1).reshape(S * B, E), B, S, k, coeff)
    assert abs(got - wrong) > 1e-3 * abs(want), "the check cannot tell s*B+b from b*S+s"


def test_seq_aux_loss_uniform_routing_equals_coeff(orc):
    """Every sequence sends S*k/E tokens to every expert: cost_coeff == 1, rows of softmax scores
    sum to 1, so the loss is exactly coeff whatever the scores."""
    g = torch.Generator().manual_seed(12)
    B, S, E, k, coeff = 4, 8, 4, 2, 0.01
    scores = torch.softmax(torch.randn(S * B, E, generator=g, dtype=torch.float64), -1)
    rmap = torch.zeros(S, B, E, dtype=torch.bool)
    for s in range(S):
        for j in range(k):
            rmap[s, :, (s * k + j) % E] = True
    rmap = rmap.view(S * B, E)
    assert torch.equal(rmap.view(S, B, E).sum(0), torch.full((B, E), S * k // E))
    assert abs(orc.sequence_load_balancing_loss(scores, rmap, B, S, k, coeff).item() - coeff) < 1e-9


def test_seq_aux_loss_single_sequence_is_switch_loss(orc):
    g = torch.Generator().manual_seed(13)
    S, E, k, coeff = 32, 8, 2, 0.05
    logits = torch.randn(S, E, generator=g, dtype=torch.float64)
    scores = torch.softmax(logits, -1)
    _, rmap, counts = orc.topk_softmax_with_capacity(logits, k)
    a = orc.sequence_load_balancing_loss(scores, rmap, 1, S, k, coeff).item()
    b = orc.switch_load_balancing_loss(scores, counts, k, coeff).item()
    assert abs(a - b) < 1e-7 * abs(b)


def test_sinkhorn_against_float64_loop_and_marginals(orc):
    import numpy as np
    g = torch.Generator().manual_seed(14)
    T, E = 48, 6
    logits = torch.randn(T, E, generator=g)
    got = orc.sinkhorn(logits.clone(), tol=1e-6).double().numpy()
    cost = np.exp(logits.double().numpy())
    d0, d1 = np.ones(T), np.ones(E)
    iters = 0
    while True:
        d0 = (1.0 / T) / (cost @ d1 + 1e-8)
        d1_new = (1.0 / E) / (cost.T @ d0 + 1e-8)
        err = np.mean(np.abs(d1 - d1_new))
        d1 = d1_new
        iters += 1
        if not err > 1e-6:
            break
    want = d1[None, :] * cost * d0[:, None]
    assert iters > 1
    np.testing.assert_allclose(got, want, rtol=2e-4)
    # at convergence every expert column carries 1/E of the mass, every token row about 1/T
    np.testing.assert_allclose(got.sum(0), np.full(E, 1.0 / E), rtol=1e-5)
    np.testing.assert_allclose(got.sum(1), np.full(T, 1.0 / T), rtol=1e-3)
    # the error starts at 1e9: any smaller tolerance gives at least one iteration, a larger one none
    np.testing.assert_allclose(orc.sinkhorn(logits.clone(), tol=1e30).double().numpy(), cost, rtol=1e-6)
    once = orc.sinkhorn(logits.clone(), tol=1e8).double().numpy()
    d0 = (1.0 / T) / (cost @ np.ones(E) + 1e-8)
    d1 = (1.0 / E) / (cost.T @ d0 + 1e-8)
    np.testing.assert_allclose(once, d1[None, :] * cost * d0[:, None], rtol=1e-5)


@pytest.mark.parametrize("k", [1, 2])
def test_sinkhorn_routing_invariants(orc, k):
    g = torch.Generator().manual_seed(15)
    T, E = 64, 8
    logits = torch.randn(T, E, generator=g)
    for training in (True, False):
        scores, rmap = orc.sinkhorn_routing(logits, k, training=training)
        assert torch.equal(rmap.sum(1), torch.full((T,), k))
        act = torch.sigmoid(logits) if k == 1 else torch.softmax(logits, -1)
        torch.testing.assert_close(scores, act * rmap)
        if not training:  # evaluation: plain top-k of the logits (the activation is monotonic per row)
            assert torch.equal(rmap, torch.zeros(T, E).scatter(1, torch.topk(logits, k)[1], 1).bool())
    # training: sinkhorn balances the load better than plain top-k on skewed logits
    skew = logits + torch.linspace(0, 2, E)
    _, m_train = orc.sinkhorn_routing(skew, k, training=True)
    _, m_eval = orc.sinkhorn_routing(skew, k, training=False)
    assert m_train.sum(0).float().std() < m_eval.sum(0).float().std()


def test_expert_bias_update_hand_example(orc):
    tokens = torch.tensor([[10.0, 30.0, 20.0], [5.0, 5.0, 5.0]])
    bias = torch.tensor([[0.0, 0.5, -0.5], [1.0, 2.0, 3.0]])
    got = orc.get_updated_expert_bias(tokens, bias, 0.1)
    want = torch.tensor([[0.1, 0.4, -0.5], [1.0, 2.0, 3.0]])  # under mean: +, over: -, at mean: 0
    torch.testing.assert_close(got, want)


def test_z_loss_constant_rows(orc):
    E = 8
    logits = torch.full((10, E), 3.0)
    want = (3.0 + math.log(E)) ** 2 * 0.5
    assert abs(orc.z_loss(logits, 0.5).item() - want) < 1e-5


def test_sinkhorn_balances_columns(orc):
    g = torch.Generator().manual_seed(8)
    out = orc.sinkhorn(torch.randn(32, 4, generator=g), tol=1e-6)
    torch.testing.assert_close(out.sum(0), torch.full((4,), 0.25), rtol=1e-3, atol=1e-4)


# ------------------------------------------------------------------------------------------
# permute / unpermute
# ------------------------------------------------------------------------------------------

def random_map(T, E, k, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    for e in empty:
        logits[:, e] = -1e9
    idx = torch.topk(logits, k, dim=1)[1]
    return torch.zeros(T, E, dtype=torch.bool).scatter_(1, idx, True)


def test_sorted_indices_closed_form_and_invariants(orc):
    T, E, k, H = 97, 8, 2, 16
    rmap = random_map(T, E, k, 9, empty=(3,))
    x = torch.arange(T * H, dtype=torch.float32).view(T, H)
    permuted, si = orc.permute(x, rmap)
    e_idx, t_idx = np.nonzero(rmap.numpy().T)  # row-major scan of [E,T]: expert-major, token-ascending
    assert si.dtype == torch.int64 and si.tolist() == t_idx.tolist()
    counts = rmap.sum(0)
    assert counts[3] == 0
    start = 0
    for e in range(E):
        blk = si[start:start + counts[e]]
        assert torch.all(blk[1:] > blk[:-1]) and torch.all(rmap[blk, e])
        start += counts[e]
    assert torch.equal(permuted, x[si])
    rid = orc.row_id_map_te(rmap)
    assert rid.shape == (E, T) and torch.equal(rid == -1, ~rmap.T)
    for e in range(E):
        for t in range(T):
            if rid[e, t] >= 0:
                assert si[rid[e, t]] == t and e_idx[rid[e, t]] == e


def test_unpermute_is_index_add_and_round_trip(orc):
    T, E, k, H = 64, 8, 2, 32
    rmap = random_map(T, E, k, 10)
    g = torch.Generator().manual_seed(10)
    x = torch.randn(T, H, generator=g)
    permuted, si = orc.permute(x, rmap)
    y = torch.randn_like(permuted)
    want = torch.zeros(T, H).index_add_(0, si, y)
    torch.testing.assert_close(orc.unpermute(y, si, (T, H)), want)
    # probs = map / k undoes the duplication exactly (k a power of two)
    back = orc.unpermute(permuted, si, (T, H), probs=rmap.float() / k, routing_map=rmap)
    assert torch.equal(back, x)
    # fused (row_id_map) restatement agrees with the unfused one
    rid = orc.row_id_map_te(rmap)
    probs = torch.rand(T, E, generator=g) * rmap
    a = orc.unpermute(y, si, (T, H), probs=probs, routing_map=rmap)
    b = orc.unpermute_fused(y, rid, probs)
    torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-6)


def test_unpermute_bwd_matches_autograd(orc):
    T, E, k, H = 40, 4, 2, 8
    rmap = random_map(T, E, k, 11)
    g = torch.Generator().manual_seed(11)
    n = int(rmap.sum())
    y = torch.randn(n, H, generator=g, requires_grad=True)
    probs = (torch.rand(T, E, generator=g) * rmap).requires_grad_(True)
    si = orc.permute(torch.zeros(T, H), rmap)[1]
    out = orc.unpermute(y, si, (T, H), probs=probs, routing_map=rmap)
    go = torch.randn(T, H, generator=g)
    out.backward(go)
    ga, gp = orc.unpermute_bwd_with_probs(go, orc.row_id_map_te(rmap), y.detach(), probs.detach())
    torch.testing.assert_close(ga, y.grad, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(gp, probs.grad, rtol=1e-5, atol=1e-6)


def test_drop_and_pad_permute(orc):
    T, E, H, cap = 32, 4, 8, 5
    g = torch.Generator().manual_seed(12)
    # exactly `cap` tokens per expert, as pad_to_capacity guarantees
    rmap = torch.zeros(T, E, dtype=torch.bool)
    for e in range(E):
        rmap[torch.randperm(T, generator=g)[:cap], e] = True
    x = torch.randn(T, H, generator=g)
    permuted, si = orc.permute(x, rmap, num_out_tokens=cap * E, drop_and_pad=True)
    assert si.numel() == cap * E
    for e in range(E):
        assert si[e * cap:(e + 1) * cap].tolist() == torch.nonzero(rmap[:, e]).flatten().tolist()


def test_sort_chunks(orc):
    x = torch.arange(10.0).view(10, 1)
    out = orc.sort_chunks_by_idxs(x, torch.tensor([3, 0, 5, 2]), torch.tensor([2, 0, 3, 1]))
    assert out.flatten().tolist() == [3, 4, 5, 6, 7, 0, 1, 2, 8, 9]


# ------------------------------------------------------------------------------------------
# experts
# ------------------------------------------------------------------------------------------

def test_gmm_special_cases(orc):
    g = torch.Generator().manual_seed(13)
    a = torch.randn(20, 6, generator=g, dtype=torch.float64)
    b = torch.randn(3, 6, 5, generator=g, dtype=torch.float64)
    # one group == dense matmul
    torch.testing.assert_close(orc.gmm(a, b[:1], torch.tensor([20]), compute_dtype=torch.float64), a @ b[0])
    # groups, one of them empty; element-wise closed form
    bs = torch.tensor([7, 0, 13])
    out = orc.gmm(a, b, bs, compute_dtype=torch.float64)
    for r, e in ((0, 0), (6, 0), (7, 2), (19, 2)):
        want = [sum(a[r, kk].item() * b[e, kk, m].item() for kk in range(6)) for m in range(5)]
        np.testing.assert_allclose(out[r].numpy(), want, rtol=1e-12)
    # trans_b reads b[e] as [M,K]
    bt = b.transpose(1, 2).contiguous()
    torch.testing.assert_close(orc.gmm(a, bt, bs, trans_b=True, compute_dtype=torch.float64), out)
    # weight gradient: a_e^T g_e, zero for the empty expert
    bb = b.clone().requires_grad_(True)
    go = torch.randn(20, 5, generator=g, dtype=torch.float64)
    orc.gmm(a, bb, bs, compute_dtype=torch.float64).backward(go)
    torch.testing.assert_close(bb.grad[0], a[:7].T @ go[:7])
    assert torch.count_nonzero(bb.grad[1]) == 0
    torch.testing.assert_close(bb.grad[2], a[7:].T @ go[7:])


def test_swiglu_and_back(orc):
    g = torch.Generator().manual_seed(14)
    y = torch.randn(9, 12, generator=g, dtype=torch.float64, requires_grad=True)
    out = orc.swiglu(y)
    y1, y2 = y[:, :6], y[:, 6:]
    torch.testing.assert_close(out, y1 / (1 + torch.exp(-y1)) * y2)
    go = torch.randn(9, 6, generator=g, dtype=torch.float64)
    out.backward(go)
    torch.testing.assert_close(orc.swiglu_back(go, y.detach()), y.grad)


def e4m3fn_round_numpy(x):
    """fp64 values -> the e4m3fn value they round to (nearest, ties to even; steps of 2^(e-3) with
    e >= -6, so 2^-9 in the subnormal range), NaN where the result would exceed 448."""
    import numpy as np

    x = np.asarray(x, dtype=np.float64)
    ax = np.abs(x)
    e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
    e = np.maximum(e, -6.0)
    step = 2.0 ** (e - 3)
    with np.errstate(all="ignore"):
        q = np.round(ax / step) * step      # numpy rounds halves to even
    q = np.where(q > 448.0, np.nan, q)
    q = np.where(np.isnan(x), np.nan, q)
    return np.copysign(q, x)


def test_fp8_input_store_cast_on_every_bf16_value_and_backward(orc):
    """The cast SwiGLUFunction stores (transformer/fused_kernels.py:193) against an independent
    restatement of e4m3fn rounding on all 65536 bf16 bit patterns; the backward is swiglu_back on
    the stored (rounded) input, the forward untouched."""
    import numpy as np

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    got = x.to(torch.float8_e4m3fn).to(torch.float64).numpy()
    want = e4m3fn_round_numpy(x.to(torch.float64).numpy())
    both_nan = np.isnan(got) & np.isnan(want)
    assert np.array_equal(np.where(both_nan, 0.0, got), np.where(both_nan, 0.0, want))
    assert np.array_equal(np.signbit(got[~both_nan]), np.signbit(want[~both_nan]))
    # spot values: exact ones stay, a tie goes to the even neighbour, 464 is the last finite input
    for v, w in ((448.0, 448.0), (0.0625, 0.0625), (17.0, 16.0), (19.0, 20.0), (464.0, 448.0),
                 (2.0 ** -9, 2.0 ** -9), (2.0 ** -10, 0.0), (3 * 2.0 ** -10, 2.0 ** -8)):
        assert torch.tensor(v).to(torch.float8_e4m3fn).float().item() == w, v
    assert torch.isnan(torch.tensor(466.0).to(torch.float8_e4m3fn).float())

    g = torch.Generator().manual_seed(31)
    y = (torch.randn(16, 24, generator=g) * 3).bfloat16().requires_grad_(True)
    out = orc.swiglu_fp8_input_store(y)
    assert torch.equal(out, orc.swiglu(y.detach()))
    go = torch.randn(16, 12, generator=g).bfloat16()
    out.backward(go)
    y8 = y.detach().to(torch.float8_e4m3fn).to(torch.bfloat16)
    assert torch.equal(y.grad, orc.swiglu_back(go, y8))
    assert not torch.equal(y.grad, orc.swiglu_back(go, y.detach()))


def test_layer_equals_dense_mixture(orc):
    """out[t] = sum_{e in top-k(t)} p[t,e] * MLP_e(x[t]) computed token by token."""
    g = torch.Generator().manual_seed(15)
    T, H, Fd, E, k = 24, 16, 32, 4, 2
    x = torch.randn(T, H, generator=g)
    w_r = torch.randn(E, H, generator=g) * 0.1
    w1 = torch.randn(E, H, 2 * Fd, generator=g) * 0.1
    w2 = torch.randn(E, Fd, H, generator=g) * 0.1
    for disp in ("allgather", "alltoall"):
        out, _, info = orc.moe_layer(x, w_r, w1, w2, k, dispatcher=disp)
        logits = x @ w_r.T
        for t in range(T):
            sel = brute_topk(logits[t].tolist(), k)
            z = torch.softmax(logits[t, sel], 0)
            want = torch.zeros(H)
            for p, e in zip(z, sel):
                h = x[t] @ w1[e]
                want += p * ((F.silu(h[:Fd]) * h[Fd:]) @ w2[e])
            torch.testing.assert_close(out[t], want, rtol=1e-4, atol=1e-5)
    assert info["tokens_per_expert"].sum() == T * k


def test_fp8_block_quantisation_round_trip(orc):
    g = torch.Generator().manual_seed(16)
    w = 0.02 * torch.randn(2, 256, 384, generator=g)
    q, s = orc.quantize_fp8_block(w)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (2, 2, 3) and s.dtype == torch.bfloat16
    back = orc.dequantize_fp8_block(q, s)
    # e4m3 keeps 3 mantissa bits: relative error <= 2^-4 of the tile maximum
    tile_max = w.view(2, 2, 128, 3, 128).abs().amax(dim=(2, 4))
    err = (back - w).view(2, 2, 128, 3, 128).abs().amax(dim=(2, 4))
    assert torch.all(err <= tile_max * 2 ** -4 + 1e-12)
    assert torch.all(q.float().abs() <= 448)


@pytest.mark.parametrize("dispatcher", ["allgather", "alltoall"])
def test_layer_matches_the_hf_mixtral_block(orc, dispatcher):
    """An independent library implementation of the same layer (the model the reference's own
    correctness test compares with, tests/models/test_moe_correctness.py): transformers'
    MixtralSparseMoeBlock with the oracle's weights, forward and input / weight gradients in fp32."""
    mm = pytest.importorskip("transformers.models.mixtral.modeling_mixtral")
    from transformers import MixtralConfig

    E, H, Fe, k = 6, 32, 48, 2
    cfg = MixtralConfig(hidden_size=H, intermediate_size=Fe, num_local_experts=E, num_experts_per_tok=k,
                        num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=2, vocab_size=64)
    torch.manual_seed(3)
    blk = mm.MixtralSparseMoeBlock(cfg).float().eval()
    if not hasattr(blk.experts, "gate_up_proj"):
        pytest.skip("this transformers version keeps per-expert modules")
    with torch.no_grad():
        for p in blk.parameters():
            p.normal_(0.0, 0.2)
    x = torch.randn(3, 7, H, requires_grad=True)
    want = blk(x)
    want = want[0] if isinstance(want, tuple) else want
    go = torch.randn_like(want)
    want.backward(go)
    # gate_up_proj[e] = [w1; w3] ([2F,H]), down_proj[e] = w2 ([H,F]): the grouped layout is their transpose
    w_r = blk.gate.weight.detach().clone().requires_grad_(True)
    w1 = blk.experts.gate_up_proj.detach().transpose(1, 2).contiguous().requires_grad_(True)
    w2 = blk.experts.down_proj.detach().transpose(1, 2).contiguous().requires_grad_(True)
    xo = x.detach().clone().requires_grad_(True)
    got, _, _ = orc.moe_layer(xo, w_r, w1, w2, k, dispatcher=dispatcher)
    got.backward(go)
    torch.testing.assert_close(got, want.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(xo.grad, x.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w_r.grad, blk.gate.weight.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w1.grad, blk.experts.gate_up_proj.grad.transpose(1, 2), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w2.grad, blk.experts.down_proj.grad.transpose(1, 2), rtol=1e-4, atol=1e-5)


def test_rms_norm_against_library_forms(orc):
    """The pre-router norm: torch's own rms_norm, transformers' MixtralRMSNorm (fp32, where its
    intermediate rounding vanishes), the closed form on rows of constant magnitude, invariance
    under a positive rescaling of x (eps = 0), and the bf16 output being the fp32 result rounded once."""
    from transformers.models.mixtral.modeling_mixtral import MixtralRMSNorm

    g = torch.Generator().manual_seed(3)
    x = 3.0 * torch.randn(37, 96, generator=g)
    w = 1.0 + 0.3 * torch.randn(96, generator=g)
    y = orc.rms_norm(x, w, 1e-5)
    torch.testing.assert_close(y, F.rms_norm(x, (96,), w, 1e-5), rtol=1e-6, atol=1e-6)
    hf = MixtralRMSNorm(96, eps=1e-5)
    with torch.no_grad():
        hf.weight.copy_(w)
    torch.testing.assert_close(y, hf(x).detach(), rtol=1e-6, atol=1e-6)
    # |x| = c everywhere: mean(x^2) = c^2, so y = sign(x) * w * c / sqrt(c^2 + eps)
    c = 0.5
    xs = c * torch.sign(torch.randn(5, 96, generator=g))
    want = torch.sign(xs) * w * (c / math.sqrt(c * c + 1e-5))
    torch.testing.assert_close(orc.rms_norm(xs, w, 1e-5), want, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(orc.rms_norm(7.0 * x, w, 0.0), orc.rms_norm(x, w, 0.0), rtol=1e-5, atol=1e-6)
    # a wrong axis or a missing mean would not survive this: one row scaled alone changes only itself
    x2 = x.clone()
    x2[4] *= 100.0
    y2 = orc.rms_norm(x2, w, 0.0)
    torch.testing.assert_close(y2[:4], orc.rms_norm(x, w, 0.0)[:4])
    torch.testing.assert_close(y2[4], orc.rms_norm(x, w, 0.0)[4], rtol=1e-5, atol=1e-6)
    xb = x.bfloat16()
    assert torch.equal(orc.rms_norm(xb, w.bfloat16(), 1e-5),
                       orc.rms_norm(xb.float(), w.bfloat16().float(), 1e-5).bfloat16())


# ------------------------------------------------------------------------------------------
# shared expert
# ------------------------------------------------------------------------------------------

def test_shared_expert_mlp_token_by_token_fp64(orc):
    """Dense SwiGLU written out per token and per hidden unit in fp64: gate = columns [0, Fs) of w1s,
    up = columns [Fs, 2 Fs); a swapped half or a missing activation fails."""
    import math
    g = torch.Generator().manual_seed(21)
    T, H, Fs = 5, 6, 4
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    w1s = torch.randn(H, 2 * Fs, generator=g, dtype=torch.float64)
    w2s = torch.randn(Fs, H, generator=g, dtype=torch.float64)
    got = orc.shared_expert_mlp(x, w1s, w2s, compute_dtype=torch.float64)
    for t in range(T):
        act = []
        for f in range(Fs):
            gate = sum(float(x[t, h]) * float(w1s[h, f]) for h in range(H))
            up = sum(float(x[t, h]) * float(w1s[h, Fs + f]) for h in range(H))
            act.append(gate / (1.0 + math.exp(-gate)) * up)
        for h in range(H):
            want = sum(act[f] * float(w2s[f, h]) for f in range(Fs))
            assert abs(float(got[t, h]) - want) < 1e-9 * max(1.0, abs(want))


def test_shared_expert_mlp_against_transformers_gated_mlp(orc):
    """transformers' LlamaMLP (down(silu(gate(x)) * up(x))), an independent library implementation
    of the same SiLU-gated MLP, with the oracle's weights: forward and all gradients."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP
    g = torch.Generator().manual_seed(22)
    T, H, Fs = 24, 32, 48
    x = torch.randn(T, H, generator=g).requires_grad_(True)
    w1s = (0.2 * torch.randn(H, 2 * Fs, generator=g)).requires_grad_(True)
    w2s = (0.2 * torch.randn(Fs, H, generator=g)).requires_grad_(True)
    mlp = LlamaMLP(LlamaConfig(hidden_size=H, intermediate_size=Fs, hidden_act="silu", mlp_bias=False))
    with torch.no_grad():
        mlp.gate_proj.weight.copy_(w1s[:, :Fs].t())
        mlp.up_proj.weight.copy_(w1s[:, Fs:].t())
        mlp.down_proj.weight.copy_(w2s.t())
    xr = x.detach().clone().requires_grad_(True)
    dy = torch.randn(T, H, generator=g)
    orc.shared_expert_mlp(x, w1s, w2s).backward(dy)
    mlp(xr).backward(dy)
    torch.testing.assert_close(orc.shared_expert_mlp(x, w1s, w2s), mlp(xr), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(x.grad, xr.grad, rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(w1s.grad[:, :Fs], mlp.gate_proj.weight.grad.t(), rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(w1s.grad[:, Fs:], mlp.up_proj.weight.grad.t(), rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(w2s.grad, mlp.down_proj.weight.grad.t(), rtol=1e-4, atol=1e-6)


def test_fp8_row_quantisation_exponents_and_round_trip(orc):
    """The build's activation format (not in the reference): per row and 128 elements the smallest
    power of two that keeps the block within +-448, found here by brute force over the exponents;
    blocks of exactly representable values come back without error."""
    import math

    g = torch.Generator().manual_seed(5)
    x = torch.randn(37, 300, generator=g) * torch.logspace(-6, 6, 37).unsqueeze(1)
    x[3, :128] = 0                         # an all-zero block
    x[4, 128:256] = 448.0                  # amax exactly 448: exponent 0
    x[5, :128] = 456.0                     # the next bf16 value worth a test above 448: exponent 1
    x = x.bfloat16()
    q, e = orc.quantize_fp8_rows(x)
    assert q.dtype == torch.float8_e4m3fn and e.shape == (3, 37) and e.dtype == torch.int32
    xf = x.float()
    for r in range(37):
        for b in range(3):
            amax = xf[r, 128 * b:128 * (b + 1)].abs().max().item()
            if amax == 0:
                assert int(e[b, r]) == -127
                continue
            want = next(k for k in range(-127, 128) if amax * 2.0 ** -k <= 448.0)
            assert int(e[b, r]) == want, (r, b, amax)
            assert amax * 2.0 ** -want > 224.0 or want == -127
    assert int(e[1, 4]) == 0 and int(e[0, 5]) == 1
    back = orc.dequantize_fp8_rows(q, e)
    step = torch.ldexp(torch.ones(()), e.t().repeat_interleave(128, 1)[:, :300]) * 16  # half of 32 at the top binade
    assert torch.all((back - xf).abs() <= step)
    # powers of two and small integers times a power of two are representable: exact round trip
    y = torch.tensor([[1.0, -2.0, 0.5, 3.0, -3.5, 0.0, 448.0, 0.25]]).repeat(2, 16) * 2.0 ** 20
    qy, ey = orc.quantize_fp8_rows(y)
    assert torch.equal(orc.dequantize_fp8_rows(qy, ey), y)



def test_sequential_mlp_with_bias_token_by_token_fp64(orc):
    """Experts with `add_bias_linear` (moe/mlp.py:176-211 over transformer/mlp.py:104-138): fc1 bias in
    front of the activation, fc2 bias returned as rows and not added."""
    g = torch.Generator().manual_seed(21)
    E, H, Fe = 3, 12, 10
    counts = torch.tensor([5, 0, 7])
    N = int(counts.sum())
    x = torch.randn(N, H, generator=g, dtype=torch.float64)
    fc1_w = torch.randn(E, 2 * Fe, H, generator=g, dtype=torch.float64)
    fc2_w = torch.randn(E, H, Fe, generator=g, dtype=torch.float64)
    fc1_b = torch.randn(E, 2 * Fe, generator=g, dtype=torch.float64)
    fc2_b = torch.randn(E, H, generator=g, dtype=torch.float64)
    out, out_bias = orc.sequential_mlp(x, fc1_w, fc2_w, counts, fc1_b, fc2_b, compute_dtype=torch.float64)
    expert_of_row = np.repeat(np.arange(E), counts.numpy())
    for r in range(N):
        e = int(expert_of_row[r])
        t = [sum(float(fc1_w[e, j, h]) * float(x[r, h]) for h in range(H)) + float(fc1_b[e, j]) for j in range(2 * Fe)]
        act = [t[j] / (1.0 + math.exp(-t[j])) * t[Fe + j] for j in range(Fe)]
        for h in range(H):
            want = sum(float(fc2_w[e, h, j]) * act[j] for j in range(Fe))   # no fc2 bias in the output
            assert abs(float(out[r, h]) - want) < 1e-9 * max(1.0, abs(want))
        assert torch.equal(out_bias[r], fc2_b[e])
    # a zero fc1 bias changes nothing; without biases it is grouped_mlp on the transposed weights
    out0, none = orc.sequential_mlp(x, fc1_w, fc2_w, counts, compute_dtype=torch.float64)
    assert none is None
    outz, _ = orc.sequential_mlp(x, fc1_w, fc2_w, counts, torch.zeros_like(fc1_b), fc2_b, compute_dtype=torch.float64)
    assert torch.equal(out0, outz)
    grouped = orc.grouped_mlp(x, fc1_w.transpose(1, 2), fc2_w.transpose(1, 2), counts, compute_dtype=torch.float64)
    torch.testing.assert_close(out0, grouped, rtol=1e-12, atol=1e-12)
    # one expert: the library's linear with bias
    x1 = x[:5]
    o1, b1 = orc.sequential_mlp(x1, fc1_w[:1], fc2_w[:1], torch.tensor([5]), fc1_b[:1], fc2_b[:1],
                                compute_dtype=torch.float64)
    t = F.linear(x1, fc1_w[0], fc1_b[0])
    torch.testing.assert_close(o1, F.linear(F.silu(t[:, :Fe]) * t[:, Fe:], fc2_w[0]), rtol=1e-12, atol=1e-12)
    assert torch.equal(b1, fc2_b[0].expand(5, H))


def test_allgather_combine_with_bias_per_token_loop(orc):
    """moe/token_dispatcher.py:233-258: output and bias rows weighted by the gates and summed per token."""
    g = torch.Generator().manual_seed(22)
    T, E, H, k = 9, 4, 6, 2
    logits = torch.randn(T, E, generator=g, dtype=torch.float64)
    probs, rmap, counts = orc.topk_softmax_with_capacity(logits, k)
    n = int(rmap.sum())
    rows = torch.randn(n, H, generator=g, dtype=torch.float64)
    bias = torch.randn(n, H, generator=g, dtype=torch.float64)
    _, sorted_indices = orc.permute(torch.zeros(T, H, dtype=torch.float64), rmap)
    out, out_bias = orc.allgather_combine(rows, probs, rmap, sorted_indices, (T, H), bias=bias)
    # expert-major row order: row index of (t, e) = number of selected pairs before it in map.T order
    pos = {}
    i = 0
    for e in range(E):
        for t in range(T):
            if rmap[t, e]:
                pos[(t, e)] = i
                i += 1
    for t in range(T):
        want = torch.zeros(H, dtype=torch.float64)
        wantb = torch.zeros(H, dtype=torch.float64)
        for e in range(E):
            if rmap[t, e]:
                want += rows[pos[(t, e)]] * probs[t, e]
                wantb += bias[pos[(t, e)]] * probs[t, e]
        torch.testing.assert_close(out[t], want, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(out_bias[t], wantb, rtol=1e-12, atol=1e-12)
    # the same bias row b everywhere combines to b * (sum of the token's gates) = b here
    b = torch.randn(H, generator=g, dtype=torch.float64)
    _, ob = orc.allgather_combine(rows, probs, rmap, sorted_indices, (T, H), bias=b.expand(n, H))
    torch.testing.assert_close(ob, b.expand(T, H) * probs.sum(1, keepdim=True), rtol=1e-12, atol=1e-12)
    _, none = orc.allgather_combine(rows, probs, rmap, sorted_indices, (T, H))
    assert none is None
