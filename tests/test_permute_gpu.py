"""Permute / unpermute parity on the GPU through the C ABI.  Indices and counts bit-exact; row data
exact for pure data movement, fp tolerance where a weighted sum is taken."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]
SUM_TOL = {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
           torch.float16: dict(rtol=2e-3, atol=2e-3)}


def random_map(T, E, k, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    for e in empty:
        logits[:, e] = -1e9
    idx = torch.topk(logits, k, dim=1)[1]
    return torch.zeros(T, E, dtype=torch.bool).scatter_(1, idx, True)


CASES = [  # T, E, k, H, empty experts
    (2048, 8, 2, 512, ()),
    (1000, 64, 8, 256, (5, 63)),
    (777, 4, 2, 128, ()),
    (300, 60, 6, 68, (0,)),       # E not a multiple of 8, 16-bit rows not a multiple of 16 bytes
    (513, 256, 8, 64, tuple(range(100, 140))),
    (1, 8, 2, 4096, ()),
    (4096, 8, 2, 7168, (7,)),     # rows longer than one 8 KiB piece
]


@pytest.mark.parametrize("T,E,k,H,empty", CASES)
def test_plan_bit_exact(pkg, orc, dev, T, E, k, H, empty):
    rmap = random_map(T, E, k, seed=T + E, empty=empty)
    print("case", T, E, k, flush=True)
    plan = pkg.ops.permute_plan(rmap.to(dev), T * k, want_row_id_map=True)
    _, o_si = orc.permute(torch.zeros(T, 1), rmap)
    assert plan.sorted_indices.dtype == torch.int64
    assert torch.equal(plan.sorted_indices.cpu(), o_si)
    assert torch.equal(plan.tokens_per_expert.cpu(), rmap.sum(0))
    off = torch.zeros(E + 1, dtype=torch.int64)
    off[1:] = rmap.sum(0).cumsum(0)
    assert torch.equal(plan.expert_offsets.cpu(), off)
    o_rid = orc.row_id_map_te(rmap)
    assert torch.equal(plan.row_id_map.cpu(), o_rid)
    assert torch.equal(plan.dst_map.cpu().long(), o_rid.T)
    assert torch.equal(pkg.fused_kernels.row_id_map_reference_layout(plan.dst_map).cpu(), o_rid)


def test_plan_arbitrary_mask_and_empty_input(pkg, orc, dev):
    g = torch.Generator().manual_seed(5)
    rmap = torch.rand(1500, 24, generator=g) < 0.3  # variable experts per token, some tokens unrouted
    rmap[10] = False
    n = int(rmap.sum())
    plan = pkg.ops.permute_plan(rmap.to(dev), n)
    assert torch.equal(plan.sorted_indices.cpu(), orc.permute(torch.zeros(1500, 1), rmap)[1])
    assert torch.equal(plan.tokens_per_expert.cpu(), rmap.sum(0))
    empty = torch.zeros(0, 8, dtype=torch.bool, device=dev)
    plan = pkg.ops.permute_plan(empty, 0)
    assert plan.tokens_per_expert.cpu().tolist() == [0] * 8
    assert plan.expert_offsets.cpu().tolist() == [0] * 9


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,E,k,H,empty", CASES)
@pytest.mark.parametrize("fused", [False, True])
def test_permute_unpermute_forward(pkg, orc, dev, dtype, T, E, k, H, empty, fused):
    rmap = random_map(T, E, k, seed=T + E, empty=empty)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, H, generator=g).to(dtype)
    probs = (torch.rand(T, E, generator=g) * rmap).to(dtype)
    print("case", dtype, T, E, k, H, fused, flush=True)
    permuted, mapping = pkg.permute(x.to(dev), rmap.to(dev), num_out_tokens=T * k, fused=fused)
    o_perm, o_si = orc.permute(x, rmap)
    assert torch.equal(permuted.cpu(), o_perm), "permuted rows differ"
    if not fused:
        assert torch.equal(mapping.cpu(), o_si)
    # unweighted restore == index_add in fp32
    y = torch.randn(T * k, H, generator=g).to(dtype)
    out = pkg.unpermute(y.to(dev), mapping, (T, H), routing_map=rmap.to(dev), fused=fused)
    want = orc.unpermute(y, o_si, (T, H), accumulate_dtype=torch.float32)
    assert out.dtype == dtype
    torch.testing.assert_close(out.cpu().float(), want.float(), **SUM_TOL[dtype])
    # weighted restore
    out = pkg.unpermute(y.to(dev), mapping, (T, H), probs=probs.to(dev), routing_map=rmap.to(dev),
                        fused=fused)
    want = orc.unpermute_fused(y, orc.row_id_map_te(rmap), probs)
    torch.testing.assert_close(out.cpu().float(), want.float(), **SUM_TOL[dtype])


def test_permute_without_num_out_tokens_and_te_names(pkg, orc, dev):
    T, E, k, H = 640, 8, 2, 256
    rmap = random_map(T, E, k, seed=3)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g).bfloat16()
    o_perm, o_si = orc.permute(x, rmap)
    permuted, si = pkg.permute(x.to(dev), rmap.to(dev))
    assert torch.equal(permuted.cpu(), o_perm) and torch.equal(si.cpu(), o_si)
    out, row_id_map = pkg.moe_permute(x.to(dev), rmap.to(dev).int(), num_out_tokens=T * k)
    assert torch.equal(out.cpu(), o_perm)
    probs = (torch.rand(T, E, generator=g) * rmap)
    back = pkg.moe_unpermute(out, row_id_map, merging_probs=probs.to(dev), restore_shape=x.shape)
    want = orc.unpermute_fused(o_perm, orc.row_id_map_te(rmap), probs)
    torch.testing.assert_close(back.cpu().float(), want.float(), rtol=2e-2, atol=1e-2)
    # index-style routing map
    idx = torch.topk(torch.randn(T, E, generator=g), k, dim=1)[1]
    out2, rid2 = pkg.moe_permute(x.to(dev), idx.to(dev).int(), num_out_tokens=T * k, map_type="index",
                                 num_experts=E)
    m2 = torch.zeros(T, E, dtype=torch.bool).scatter_(1, idx, True)
    assert torch.equal(out2.cpu(), orc.permute(x, m2)[0])
    with pytest.raises(ValueError):
        pkg.moe_permute(x.to(dev), rmap.to(dev), map_type="other")
    # unpermute from the index list alone (no plan, no routing map)
    plain = pkg.unpermute(o_perm.to(dev), o_si.to(dev), (T, H))
    torch.testing.assert_close(plain.cpu().float(), orc.unpermute(o_perm, o_si, (T, H),
                               accumulate_dtype=torch.float32).float(), rtol=2e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,k,H", [(512, 8, 2, 256), (300, 64, 8, 68), (256, 8, 2, 7168)])
def test_backward(pkg, orc, dev, dtype, T, E, k, H):
    rmap = random_map(T, E, k, seed=T)
    g = torch.Generator().manual_seed(T + 1)
    x = torch.randn(T, H, generator=g).to(dtype)
    probs = (torch.rand(T, E, generator=g) * rmap).float()
    go = torch.randn(T, H, generator=g).to(dtype)
    gperm = torch.randn(T * k, H, generator=g).to(dtype)
    tol = SUM_TOL[dtype]
    # permute backward: sum of the k row gradients per token
    xg = x.to(dev).requires_grad_(True)
    permuted, mapping = pkg.permute(xg, rmap.to(dev), num_out_tokens=T * k)
    permuted.backward(gperm.to(dev))
    xo = x.float().requires_grad_(True)
    orc.permute(xo, rmap)[0].backward(gperm.float())
    torch.testing.assert_close(xg.grad.cpu().float(), xo.grad, **tol)
    # weighted unpermute backward: rows and gate gradients
    yg = permuted.detach().clone().requires_grad_(True)
    pg = probs.to(dev).requires_grad_(True)
    out = pkg.unpermute(yg, mapping, (T, H), probs=pg, routing_map=rmap.to(dev))
    out.backward(go.to(dev))
    want_rows, want_probs = orc.unpermute_bwd_with_probs(go, orc.row_id_map_te(rmap),
                                                         permuted.detach().cpu(), probs)
    torch.testing.assert_close(yg.grad.cpu().float(), want_rows.float(), **tol)
    ptol = dict(rtol=1e-4, atol=2e-3)  # fp32 dot products of identical inputs: order of summation only
    torch.testing.assert_close(pg.grad.cpu(), want_probs, **ptol)
    assert torch.all(pg.grad.cpu()[~rmap] == 0)
    # unweighted unpermute backward: a plain gather
    yg2 = permuted.detach().clone().requires_grad_(True)
    pkg.unpermute(yg2, mapping, (T, H), routing_map=rmap.to(dev)).backward(go.to(dev))
    assert torch.equal(yg2.grad.cpu(), go[orc.permute(x, rmap)[1]])


def test_drop_and_pad(pkg, orc, dev):
    T, E, H, cap = 256, 8, 128, 40
    g = torch.Generator().manual_seed(9)
    rmap = torch.zeros(T, E, dtype=torch.bool)
    for e in range(E):
        rmap[torch.randperm(T, generator=g)[:cap], e] = True
    x = torch.randn(T, H, generator=g).bfloat16()
    permuted, si = pkg.permute(x.to(dev), rmap.to(dev), num_out_tokens=cap * E, drop_and_pad=True)
    o_perm, o_si = orc.permute(x, rmap, num_out_tokens=cap * E, drop_and_pad=True)
    assert torch.equal(si.cpu(), o_si) and torch.equal(permuted.cpu(), o_perm)
    probs = (torch.rand(T, E, generator=g) * rmap)
    out = pkg.unpermute(permuted, si, (T, H), probs=probs.to(dev), routing_map=rmap.to(dev),
                        drop_and_pad=True)
    want = orc.unpermute(o_perm, o_si, (T, H), probs=probs, routing_map=rmap, drop_and_pad=True,
                         accumulate_dtype=torch.float32)
    torch.testing.assert_close(out.cpu().float(), want.float(), rtol=2e-2, atol=1e-2)
    # more routed tokens than capacity: only the first `cap` of each expert are kept
    rmap2 = torch.rand(T, E, generator=g) < 0.5
    permuted2, si2 = pkg.permute(x.to(dev), rmap2.to(dev), num_out_tokens=cap * E, drop_and_pad=True)
    for e in range(E):
        first = torch.nonzero(rmap2[:, e]).flatten()[:cap]
        assert torch.equal(si2.cpu()[e * cap:e * cap + first.numel()], first)
        assert torch.equal(permuted2.cpu()[e * cap:e * cap + first.numel()], x[first])


def test_sort_chunks(pkg, orc, dev):
    g = torch.Generator().manual_seed(13)
    splits = torch.tensor([5, 0, 17, 3, 40, 1, 9, 25])
    order = torch.tensor([4, 0, 7, 2, 1, 6, 3, 5])
    n = int(splits.sum())
    x = torch.randn(n, 96, generator=g).bfloat16()
    xg = x.to(dev).requires_grad_(True)
    out = pkg.sort_chunks_by_idxs(xg, splits, order)
    want = orc.sort_chunks_by_idxs(x, splits, order)
    assert torch.equal(out.cpu(), want)
    assert torch.equal(pkg.moe_sort_chunks_by_index(x.to(dev), splits.to(dev), order.to(dev)).cpu(), want)
    go = torch.randn(n, 96, generator=g).bfloat16()
    out.backward(go.to(dev))
    xo = x.float().requires_grad_(True)
    orc.sort_chunks_by_idxs(xo, splits, order).backward(go.float())
    assert torch.equal(xg.grad.cpu().float(), xo.grad)
    # inverse order restores the input (token_dispatcher.py:341-351, 643-648)
    sizes_after = splits[order]
    inv = torch.argsort(order)
    assert torch.equal(pkg.sort_chunks_by_idxs(out.detach(), sizes_after, inv).cpu(), x)


def test_sort_chunks_with_bad_tables(pkg, dev):
    """Tables on the device cannot be checked on the host: an index that names no chunk moves no
    rows, output rows that no chunk covers are marked -1 in the row map and left alone; tables on
    the host are refused outright (torch.split in the reference raises there too)."""
    x = torch.arange(12 * 8, dtype=torch.float32).view(12, 8).bfloat16().to(dev)
    splits = torch.tensor([4, 3, 5], device=dev)
    out, row_map = pkg.ops.sort_chunks(x, splits, torch.tensor([2, 7, 0], device=dev))
    assert row_map.tolist() == [7, 8, 9, 10, 11, 0, 1, 2, 3, -1, -1, -1]
    assert torch.equal(out[:9].cpu(), x.cpu()[[7, 8, 9, 10, 11, 0, 1, 2, 3]])
    out, row_map = pkg.ops.sort_chunks(x, torch.tensor([4, 3, 2], device=dev), torch.tensor([1, 0, 2], device=dev))
    assert row_map.tolist() == [4, 5, 6, 0, 1, 2, 3, 7, 8, -1, -1, -1]
    with pytest.raises(AssertionError):
        pkg.ops.sort_chunks(x, torch.tensor([4, 3, 2]), torch.tensor([1, 0, 2]))
    with pytest.raises(AssertionError):
        pkg.ops.sort_chunks(x, torch.tensor([4, 3, 5]), torch.tensor([1, 0, 3]))


def test_full_size_round_trip_properties(pkg, dev):
    """Mixtral-shape permute at full size: size-independent properties instead of a CPU replay."""
    T, E, k, H = 16384, 8, 2, 4096
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(T, H, generator=g, device=dev, dtype=torch.bfloat16)
    logits = torch.randn(T, E, generator=g, device=dev)
    probs, rmap, counts = pkg.topk_softmax_with_capacity(logits, k)
    permuted, si = pkg.permute(x, rmap, num_out_tokens=T * k)
    assert counts.sum().item() == T * k
    # expert-major, token-ascending inside every expert block
    off = torch.zeros(E + 1, dtype=torch.int64)
    off[1:] = counts.cpu().cumsum(0)
    sic = si.cpu()
    for e in range(E):
        blk = sic[off[e]:off[e + 1]]
        assert torch.all(blk[1:] > blk[:-1])
        assert torch.all(rmap.cpu()[blk, e])
    assert torch.equal(permuted, x[si])
    # gates sum to one, so the weighted restore of the duplicated rows returns x (up to bf16 rounding)
    back = pkg.unpermute(permuted, si, (T, H), probs=probs, routing_map=rmap)
    torch.testing.assert_close(back.float(), x.float(), rtol=1e-2, atol=1e-2)
    # linearity of the unweighted restore: restore(permute(x)) == k * x exactly (k = 2)
    twice = pkg.unpermute(permuted, si, (T, H), routing_map=rmap)
    assert torch.equal(twice, x * 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,E,k,H", [(512, 8, 2, 256), (300, 60, 6, 68), (256, 8, 2, 7168)])
def test_unpermute_with_residual_equals_unpermute_then_add(pkg, dev, dtype, T, E, k, H):
    """The residual added inside the combine kernel gives the bits of `unpermute(...) + residual`,
    and its gradient is the incoming gradient."""
    rmap = random_map(T, E, k, seed=T + 3)
    g = torch.Generator().manual_seed(T + 4)
    x = torch.randn(T, H, generator=g).to(dtype)
    resid = torch.randn(T, H, generator=g).to(dtype)
    probs = (torch.rand(T, E, generator=g) * rmap).float()
    go = torch.randn(T, H, generator=g).to(dtype)
    permuted, mapping = pkg.permute(x.to(dev), rmap.to(dev), num_out_tokens=T * k)
    for p in (probs.to(dev), None):
        yg = permuted.detach().clone().requires_grad_(True)
        rg = resid.to(dev).requires_grad_(True)
        fused = pkg.unpermute(yg, mapping, (T, H), probs=p, routing_map=rmap.to(dev), residual=rg)
        fused.backward(go.to(dev))
        y2 = permuted.detach().clone().requires_grad_(True)
        plain = pkg.unpermute(y2, mapping, (T, H), probs=p, routing_map=rmap.to(dev)) + resid.to(dev)
        plain.backward(go.to(dev))
        assert fused.dtype == dtype and torch.equal(fused, plain)
        assert torch.equal(rg.grad, go.to(dev)) and torch.equal(yg.grad, y2.grad)
