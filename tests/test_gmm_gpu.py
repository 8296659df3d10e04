"""Grouped GEMM and gated activation parity on the GPU through the C ABI, against the oracle's
per-expert fp32 matmul loop on the same (already rounded) inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu

# outputs are rounded once to the storage dtype after fp32 accumulation
TOL = {torch.float32: dict(rtol=1e-4, atol=1e-4), torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
       torch.float16: dict(rtol=2e-3, atol=2e-3)}


def splits(total, E, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    p = torch.rand(E, generator=g) + 0.05
    for e in empty:
        p[e] = 0
    idx = torch.multinomial(p / p.sum(), total, replacement=True, generator=g)
    return torch.bincount(idx, minlength=E).to(torch.int64)


def ref_gmm(orc, a, b, bs, trans_b=False):
    return orc.gmm(a.float(), b.float(), bs, trans_b=trans_b)


CASES = [  # N, K, M, E, empty
    (512, 128, 256, 4, ()),           # small tiles, the reference's test model shape
    (300, 64, 72, 3, (1,)),           # ragged groups, M not a multiple of the tile, an empty expert
    (1, 8, 8, 1, ()),                 # a single row
    (4096, 512, 2048, 8, ()),         # >= 512 rows per expert but too few 256x256 tiles: small tiles
    (8192, 1024, 2048, 8, ()),        # large tiles (>= 512 rows per expert, >= 256 tiles)
    (8300, 1024, 2056, 8, (0, 7)),    # large tiles with ragged edges in every dimension
    (2100, 256, 512, 64, tuple(range(10, 20))),  # many small groups
    (16500, 512, 1024, 4, ()),        # >= 2048 rows per expert: short last row tiles in a split launch
    (16500, 264, 1032, 5, (2,)),      # the same with an empty expert and ragged K, M
    (1024, 2048, 256, 2, ()),         # few 128-row tiles, long reduction: split over idle CUs
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("N,K,M,E,empty", CASES)
def test_gmm_forward_all_modes(pkg, orc, dev, dtype, N, K, M, E, empty):
    bs = splits(N, E, seed=N + E, empty=empty)
    g = torch.Generator().manual_seed(N)
    a = torch.randn(N, K, generator=g).to(dtype)
    b = (torch.randn(E, K, M, generator=g) / K ** 0.5).to(dtype)
    go = torch.randn(N, M, generator=g).to(dtype)
    print("case", dtype, N, K, M, E, flush=True)
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    ad, bd, god = a.to(dev), b.to(dev), go.to(dev)
    # NN
    c = pkg.ops.gmm(ad, bd, off)
    assert c.dtype == dtype and c.shape == (N, M)
    torch.testing.assert_close(c.cpu().float(), ref_gmm(orc, a, b, bs), **TOL[dtype])
    # NT: b given as [E,M,K]
    bt = b.transpose(1, 2).contiguous()
    c = pkg.ops.gmm(ad, bt.to(dev), off, trans_b=True)
    torch.testing.assert_close(c.cpu().float(), ref_gmm(orc, a, bt, bs, trans_b=True), **TOL[dtype])
    # TN: per-expert a_e^T @ go_e, zeros for empty experts
    dw = pkg.ops.gmm(ad, god, off, trans_a=True)
    assert dw.shape == (E, K, M)
    want = torch.zeros(E, K, M)
    s = 0
    for e, n in enumerate(bs.tolist()):
        want[e] = a[s:s + n].float().T @ go[s:s + n].float()
        s += n
    # one GEMM on the same operands.  16-bit: only the output's own rounding differs, the stated
    # tolerance holds.  fp32: both sides round every one of the ~N/E additions of terms of
    # magnitude up to ~10, in different orders: 6e-8 * 10 * sqrt(N/E) per element
    tol = dict(TOL[dtype])
    if dtype == torch.float32:
        tol["atol"] = max(tol["atol"], 1e-5 * (N / E) ** 0.5)
    torch.testing.assert_close(dw.cpu().float(), want, **tol)
    for e in empty:
        assert torch.count_nonzero(dw[e]) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("r,c", [(1, 1), (2, 4), (3, 3), (15, 17), (16, 16), (1, 257), (7, 73), (16, 32),
                                 (19, 27), (21, 37), (32, 33)])
def test_tile_counts_around_the_resident_workgroups(pkg, orc, dev, dtype, r, c):
    """r experts of 128 rows and 128*c columns: r*c tiles of 128 x 128 in every mode, from one tile
    to two rounds of the 512 resident workgroups and a few more.  The last, partial round is dealt
    to the XCDs in equal shares: every tile must still be computed exactly once."""
    N, K, M = 128 * r, 128, 128 * c
    bs = torch.full((r,), 128, dtype=torch.int64)
    g = torch.Generator().manual_seed(1000 * r + c)
    a = torch.randn(N, K, generator=g).to(dtype)
    b = (torch.randn(r, K, M, generator=g) / K ** 0.5).to(dtype)
    go = torch.randn(N, M, generator=g).to(dtype)
    print("case", dtype, r, c, flush=True)
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    ad, bd, god = a.to(dev), b.to(dev), go.to(dev)
    got = pkg.ops.gmm(ad, bd, off)
    torch.testing.assert_close(got.cpu().float(), ref_gmm(orc, a, b, bs), **TOL[dtype])
    bt = b.transpose(1, 2).contiguous()
    got = pkg.ops.gmm(ad, bt.to(dev), off, trans_b=True)
    torch.testing.assert_close(got.cpu().float(), ref_gmm(orc, a, bt, bs, trans_b=True), **TOL[dtype])
    dw = pkg.ops.gmm(ad, god, off, trans_a=True)
    want = torch.einsum("enk,enm->ekm", a.float().view(r, 128, K), go.float().view(r, 128, M))
    tol = dict(TOL[dtype])
    if dtype == torch.float32:
        tol["atol"] = max(tol["atol"], 1e-5 * 128 ** 0.5)
    torch.testing.assert_close(dw.cpu().float(), want, **tol)


def test_gmm_fp32_output_and_dense_special_case(pkg, dev):
    g = torch.Generator().manual_seed(7)
    a = torch.randn(1024, 512, generator=g).bfloat16()
    b = (torch.randn(1, 512, 768, generator=g) / 512 ** 0.5).bfloat16()
    off = torch.tensor([0, 1024], dtype=torch.int64, device=dev)
    c = pkg.ops.gmm(a.to(dev), b.to(dev), off, out_dtype=torch.float32)
    assert c.dtype == torch.float32
    torch.testing.assert_close(c.cpu(), a.float() @ b[0].float(), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("trans_b", [False, True])
def test_grouped_gemm_dropin_autograd(pkg, orc, dev, dtype, trans_b):
    """`grouped_gemm.ops.gmm(a, b, batch_sizes, trans_b)` with CPU batch_sizes, as moe/mlp.py calls it."""
    N, K, M, E = 900, 256, 384, 6
    bs = splits(N, E, seed=5, empty=(2,))
    g = torch.Generator().manual_seed(5)
    a = torch.randn(N, K, generator=g).to(dtype)
    b = (torch.randn(E, M, K, generator=g) if trans_b else torch.randn(E, K, M, generator=g))
    b = (b / K ** 0.5).to(dtype)
    go = torch.randn(N, M, generator=g).to(dtype)
    ag = a.to(dev).requires_grad_(True)
    bg = b.to(dev).requires_grad_(True)
    out = pkg.grouped_gemm.ops.gmm(ag, bg, bs, trans_b=trans_b)
    out.backward(go.to(dev))
    ao = a.float().requires_grad_(True)
    bo = b.float().requires_grad_(True)
    ref = orc.gmm(ao, bo, bs, trans_b=trans_b)
    ref.backward(go.float())
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach(), **TOL[dtype])
    torch.testing.assert_close(ag.grad.cpu().float(), ao.grad, **TOL[dtype])
    torch.testing.assert_close(bg.grad.cpu().float(), bo.grad, **TOL[dtype])
    assert torch.count_nonzero(bg.grad[2]) == 0
    # device-side batch sizes give the same bits
    out2 = pkg.grouped_gemm.ops.gmm(ag.detach(), bg.detach(), bs.to(dev), trans_b=trans_b)
    assert torch.equal(out2, out.detach())
    # backend.gmm with trans_a
    dw = pkg.grouped_gemm.backend.gmm(ag.detach(), go.to(dev), bs, trans_a=True)
    assert dw.shape == (E, K, M)


def test_gmm_rejects_bad_arguments(pkg, dev):
    a = torch.zeros(16, 12, device=dev, dtype=torch.bfloat16)  # K not a multiple of 8
    b = torch.zeros(1, 12, 16, device=dev, dtype=torch.bfloat16)
    off = torch.tensor([0, 16], dtype=torch.int64, device=dev)
    with pytest.raises(RuntimeError):
        pkg.ops.gmm(a, b, off)
    with pytest.raises(AssertionError):
        pkg.ops.gmm(a, b.float(), off)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("N,F", [(1000, 1408), (37, 20), (4096, 1024)])
def test_glu_forward_backward(pkg, orc, dev, dtype, act, N, F):
    import torch.nn.functional as Fn

    g = torch.Generator().manual_seed(N + F)
    y = (2 * torch.randn(N, 2 * F, generator=g)).to(dtype)
    go = torch.randn(N, F, generator=g).to(dtype)
    yg = y.to(dev).requires_grad_(True)
    out = pkg.mlp.glu(yg, act)
    out.backward(go.to(dev))
    yo = y.float().requires_grad_(True)
    fn = Fn.silu if act == "silu" else Fn.gelu
    ref = fn(yo[:, :F]) * yo[:, F:]
    ref.backward(go.float())
    if act == "silu":
        torch.testing.assert_close(ref.detach(), orc.swiglu(y.float()))
        torch.testing.assert_close(yo.grad, orc.swiglu_back(go.float(), y.float()))
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach(), **TOL[dtype])
    torch.testing.assert_close(yg.grad.cpu().float(), yo.grad, **TOL[dtype])


FUSED_SHAPES = [(4096, 512, 1024, 8, ()), (8192, 1024, 1024, 8, ()), (8300, 1024, 1416, 8, (0, 7)),
                (8192, 512, 2048, 8, ()), (700, 128, 264, 4, (2,)), (2100, 256, 320, 64, (5,))]


def fused_cases():
    """Every (dtype, activation, shape); fp32 beyond 4096 rows only once: the one case whose d(act)
    product has enough 256x256 tiles to take the large-tile kernel with the fused activation backward
    working from the accumulators (the smaller fp32 cases cover the rest)."""
    out = []
    for dtype in (torch.bfloat16, torch.float32, torch.float16):
        for act in ("silu", "gelu"):
            for shape in FUSED_SHAPES:
                N, H, F = shape[:3]
                if dtype == torch.float32 and N > 4096 and not (act == "silu" and (N, H, F) == (8192, 512, 2048)):
                    continue
                out.append((dtype, act) + shape)
    return out


@pytest.mark.parametrize("dtype,act,N,H,F,E,empty", fused_cases())
def test_fused_gated_experts_match_the_three_op_sequence(pkg, orc, dev, dtype, act, N, H, F, E, empty):
    """GEMM+activation fused in the epilogues: bit-identical to gmm -> glu -> gmm and its autograd
    (with large groups: up to the summation order in the split short row tiles), and within
    tolerance of the oracle."""
    bs = splits(N, E, seed=N + F, empty=empty)
    g = torch.Generator().manual_seed(F)
    x = torch.randn(N, H, generator=g).to(dtype)
    w1 = (torch.randn(E, H, 2 * F, generator=g) / H ** 0.5).to(dtype)
    w2 = (torch.randn(E, F, H, generator=g) / F ** 0.5).to(dtype)
    go = torch.randn(N, H, generator=g).to(dtype)
    print("case", dtype, act, N, H, F, E, flush=True)

    def run(fused):
        xs = x.to(dev).requires_grad_(True)
        a = w1.to(dev).requires_grad_(True)
        b = w2.to(dev).requires_grad_(True)
        if fused:
            out = pkg.mlp.fused_gated_experts(xs, a, b, bs, act)
        else:
            fc1 = pkg.grouped_gemm.ops.gmm(xs, a, bs)
            out = pkg.grouped_gemm.ops.gmm(pkg.mlp.glu(fc1, act), b, bs)
        out.backward(go.to(dev))
        return out.detach(), xs.grad, a.grad, b.grad

    uo, ux, ua, ub = run(False)
    # large 16-bit groups run 256-row tiles plus a split launch for the short last row tiles
    large = dtype != torch.float32 and N // E >= 512
    fn = pkg.mlp._FusedGatedExperts
    saved = fn.fuse_backward
    try:
        for fuse_backward in (True, False):
            fn.fuse_backward = fuse_backward
            fo, fx, fa, fb = run(True)
            if large:
                # the plain GEMMs split the reduction of the experts' short last row tiles (another
                # order of the same fp32 additions), the fused launches do not: those rows agree to
                # rounding, all other rows bit for bit
                wtol = dict(rtol=TOL[dtype]["rtol"], atol=TOL[dtype]["atol"] * max(1.0, (N / E) ** 0.5))
                torch.testing.assert_close(fo.float(), uo.float(), **TOL[dtype])
                torch.testing.assert_close(fx.float(), ux.float(), **TOL[dtype])
                torch.testing.assert_close(fa.float(), ua.float(), **wtol)
                torch.testing.assert_close(fb.float(), ub.float(), **wtol)
                assert (fo != uo).any(dim=1).float().mean().item() <= 0.2
            else:
                assert torch.equal(fo, uo) and torch.equal(fx, ux)
                assert torch.equal(fa, ua) and torch.equal(fb, ub)
    finally:
        fn.fuse_backward = saved
    if act == "silu":
        # the oracle rounds fc1 and the activation to the storage dtype between the ops, as here
        xo = x.clone().requires_grad_(True)
        ref = orc.grouped_mlp(xo, w1, w2, bs)
        ref.backward(go)
        torch.testing.assert_close(fo.cpu().float(), ref.detach().float(), **TOL[dtype])
        torch.testing.assert_close(fx.cpu().float(), xo.grad.float(), **TOL[dtype])


def test_gmm_without_any_rows(pkg, dev):
    """No routed row at all (empty operand tensors): NN / NT return an empty result, the weight
    gradient is all zeros."""
    E, K, M = 3, 64, 72
    a = torch.empty(0, K, device=dev, dtype=torch.bfloat16)
    go = torch.empty(0, M, device=dev, dtype=torch.bfloat16)
    b = torch.randn(E, K, M, device=dev).bfloat16()
    off = torch.zeros(E + 1, dtype=torch.int64, device=dev)
    assert pkg.ops.gmm(a, b, off).shape == (0, M)
    assert pkg.ops.gmm(a, b.transpose(1, 2).contiguous(), off, trans_b=True).shape == (0, M)
    dw = pkg.ops.gmm(a, go, off, trans_a=True)
    assert dw.shape == (E, K, M) and torch.count_nonzero(dw) == 0


def test_full_size_mixtral_gemms_against_the_blas_library(pkg, dev):
    """The benchmark's own shapes (N 32768 rows over 8 experts, H 4096, F 14336, near-uniform ragged
    groups), too large for the CPU oracle: every mode against torch's per-expert matmul on the GPU
    (an independent implementation with fp32 accumulation), and the column checksum
    sum_m c[n,m] = a[n,:] . sum_m b[e,:,m], which a dropped or doubled K tile would break."""
    N, H, F2, E = 32768, 4096, 28672, 8
    bs = torch.tensor([4096 + d for d in (37, -52, 3, 60, -41, -7, 25, -25)], dtype=torch.int64)
    assert int(bs.sum()) == N
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    g = torch.Generator(device=dev).manual_seed(99)
    x = torch.randn(N, H, generator=g, device=dev).bfloat16()
    w1 = (torch.randn(E, H, F2, generator=g, device=dev) / H ** 0.5).bfloat16()
    go = torch.randn(N, F2, generator=g, device=dev).bfloat16()
    tol = dict(rtol=2e-2, atol=1e-2)
    starts = [0] + torch.cumsum(bs, 0).tolist()
    print("NN", flush=True)
    c = pkg.ops.gmm(x, w1, off)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        torch.testing.assert_close(c[s:t], x[s:t] @ w1[e], **tol)
        # checksum in fp32 from the unrounded product: the output's own rounding averages out over
        # 28672 columns (standard deviation ~ 2^-9 * |c| * sqrt(M))
        want = x[s:t].float() @ w1[e].float().sum(1)
        got = c[s:t].float().sum(1)
        assert (got - want).abs().max() < 0.05 * F2 ** 0.5
    del c
    print("NT", flush=True)
    dx = pkg.ops.gmm(go, w1, off, trans_b=True)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        torch.testing.assert_close(dx[s:t], go[s:t] @ w1[e].t(), rtol=2e-2, atol=2e-2 * (F2 / H) ** 0.5)
    del dx
    print("TN", flush=True)
    dw = pkg.ops.gmm(x, go, off, trans_a=True)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        torch.testing.assert_close(dw[e], x[s:t].t() @ go[s:t], rtol=2e-2, atol=1e-2)


@pytest.mark.parametrize("skew", [False, True])
def test_operands_beyond_two_gib(pkg, dev, skew):
    """Mixtral shape at batch 8 (N 65536 rows, H 4096, 2F 28672): the row-partitioned operands are
    3.8 GB, beyond what one 32-bit buffer resource spans; the kernels build theirs per tile (NN, NT)
    and per segment of an expert's rows (TN).  `skew`: two experts, one with 60000 rows, so that the
    weight gradient of that expert walks two segments.  Against torch's per-expert bf16 matmul."""
    N, H, F2 = 65536, 4096, 28672
    if skew:
        bs = torch.tensor([60000, 5536], dtype=torch.int64)
    else:
        bs = torch.tensor([8192 + d for d in (37, -52, 3, 60, -41, -7, 25, -25)], dtype=torch.int64)
    E = bs.numel()
    assert int(bs.sum()) == N
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    g = torch.Generator(device=dev).manual_seed(7)
    x = torch.randn(N, H, generator=g, device=dev).bfloat16()
    w1 = (torch.randn(E, H, F2, generator=g, device=dev) / H ** 0.5).bfloat16()
    go = torch.randn(N, F2, generator=g, device=dev).bfloat16()
    tol = dict(rtol=2e-2, atol=1e-2)
    starts = [0] + torch.cumsum(bs, 0).tolist()
    print("NN", flush=True)
    c = pkg.ops.gmm(x, w1, off)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        torch.testing.assert_close(c[s:t], x[s:t] @ w1[e], **tol)
    del c
    print("NT", flush=True)
    dx = pkg.ops.gmm(go, w1, off, trans_b=True)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        # sums of 28672 products of magnitude ~ 1/64: the result has unit-in-the-last-place ~ 0.02
        torch.testing.assert_close(dx[s:t], go[s:t] @ w1[e].t(), rtol=2e-2, atol=2e-2)
    del dx
    print("TN", flush=True)
    dw = pkg.ops.gmm(x, go, off, trans_a=True)
    for e in range(E):
        s, t = starts[e], starts[e + 1]
        want = x[s:t].t() @ go[s:t]
        # both are fp32-accumulated sums rounded once to bf16: they differ by the summation order
        torch.testing.assert_close(dw[e], want, rtol=2e-2, atol=1e-2)


def test_dropin_grouped_gemm_computes_on_the_gpu(pkg, orc, dev):
    """The reference's call `grouped_gemm.ops.gmm(a, b, batch_sizes, trans_b=False)` (moe/mlp.py:106-112)
    through the drop-in package name, CPU batch_sizes as upstream passes them."""
    import importlib
    import os
    import sys

    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "hetu-galvatron_amd", "dropin")
    sys.path.insert(0, path)
    try:
        gg = importlib.import_module("grouped_gemm")
    finally:
        sys.path.remove(path)
    bs = torch.tensor([5, 0, 11], dtype=torch.int64)
    g = torch.Generator().manual_seed(1)
    a = torch.randn(16, 64, generator=g).bfloat16()
    b = (torch.randn(3, 64, 32, generator=g) / 8).bfloat16()
    out = gg.ops.gmm(a.to(dev), b.to(dev), bs, trans_b=False)
    torch.testing.assert_close(out.cpu().float(), ref_gmm(orc, a, b, bs), **TOL[torch.bfloat16])
