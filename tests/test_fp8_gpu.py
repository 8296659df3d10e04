"""Block-scaled fp8 (e4m3) expert weights on the GPU through the C ABI: the quantiser bit for bit
against the oracle's, the decode of every fp8 code, and the grouped GEMMs / the expert MLP (forward
and dX) against the oracle run on the dequantised weights."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = dict(rtol=2e-2, atol=1e-2)


def splits(total, E, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    p = torch.rand(E, generator=g) + 0.05
    for e in empty:
        p[e] = 0
    idx = torch.multinomial(p / p.sum(), total, replacement=True, generator=g)
    return torch.bincount(idx, minlength=E).to(torch.int64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,K,M", [(3, 256, 384), (2, 200, 264), (1, 128, 8), (4, 1024, 512)])
def test_quantiser_matches_the_oracle_bit_for_bit(pkg, orc, dev, dtype, E, K, M):
    g = torch.Generator().manual_seed(K + M)
    w = torch.randn(E, K, M, generator=g) * torch.rand(E, 1, 1, generator=g) * 3
    w[0, :128, :8] = 0                      # an all-zero tile (when M == 8) or part of one
    if K >= 256:
        w[-1, 128:256, :128] = 0            # a whole zero tile: its scale must be 1
    w[0, -1, -1] = 1000.0                   # a tile dominated by one value
    w = w.to(dtype)
    q, s = pkg.ops.quantize_fp8_block(w.to(dev))
    rq, rs = orc.quantize_fp8_block(w)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.bfloat16
    assert torch.equal(s.cpu(), rs)
    assert torch.equal(q.cpu().view(torch.uint8), rq.view(torch.uint8))
    # the round trip stays within half an fp8 step of the tile's largest value
    back = orc.dequantize_fp8_block(q.cpu(), s.cpu())
    err = (back - w.float()).abs().amax()
    assert err <= w.float().abs().amax() / 448 * 16 + 1e-6


def test_every_fp8_code_is_decoded_exactly(pkg, dev):
    """c = I @ w reads the dequantised weights back: all 256 codes except the two NaNs, for the
    row-major (NN) and the transposed (NT) operand."""
    codes = torch.arange(256, dtype=torch.uint8)
    codes[codes == 0x7f] = 0
    codes[codes == 0xff] = 0
    K = M = 256
    wq = codes.repeat(K, 1).contiguous()            # [K, M]: column m holds code m
    wq = (wq + torch.arange(K, dtype=torch.uint8)[:, None]) .to(torch.uint8)  # every row a rotation
    wq[wq == 0x7f] = 0
    wq[wq == 0xff] = 0
    q = wq.view(torch.float8_e4m3fn).unsqueeze(0)
    scale = torch.tensor([[[1.0, 0.5], [2.0, 0.25]]], dtype=torch.bfloat16)
    want = q.float()[0] * scale.float()[0].repeat_interleave(128, 0).repeat_interleave(128, 1)
    eye = torch.eye(K, dtype=torch.bfloat16, device=dev)
    off = torch.tensor([0, K], dtype=torch.int64, device=dev)
    c = pkg.ops.gmm_fp8w(eye, q.to(dev), scale.to(dev), off)
    assert torch.equal(c.cpu().float(), want.bfloat16().float())
    ct = pkg.ops.gmm_fp8w(eye, q.to(dev), scale.to(dev), off, trans_b=True)
    assert torch.equal(ct.cpu().float(), want.t().bfloat16().float())


CASES = [  # N, K, M, E, empty
    (512, 256, 384, 4, ()),
    (300, 128, 144, 3, (1,)),            # M not a multiple of the tile or the scale block
    (1, 16, 16, 1, ()),
    (4096, 1024, 512, 32, (3, 17)),      # ~128 rows per expert
    (1000, 208, 1040, 5, (0,)),          # K not a multiple of 64 nor of 128
    # at most 256 rows per expert on average and K a multiple of 64: the weight-streaming kernel
    (1000, 256, 512, 4, ()),             # experts beyond 192 rows: two row chunks
    (700, 128, 528, 3, ()),              # a partial column strip and a partial scale block
    (37, 64, 16, 5, (2,)),               # one stage, one fragment
    (900, 448, 784, 9, (0, 8)),          # K an odd number of stages: the last scale block is half
    (3000, 128, 272, 300, (5, 299)),     # more experts than the kernel ranks by cost: the order as it is
    (2600, 64, 2064, 40, (0, 1, 2)),     # 9 strips x 37 experts: more items than workgroups, uneven runs
    # more rows per expert: the 128 x 128-tile kernel
    (3000, 256, 384, 4, ()),
]


@pytest.mark.parametrize("N,K,M,E,empty", CASES)
def test_gmm_fp8w_both_layouts(pkg, orc, dev, N, K, M, E, empty):
    bs = splits(N, E, seed=N + E, empty=empty)
    g = torch.Generator().manual_seed(N)
    a = torch.randn(N, K, generator=g).bfloat16()
    w = torch.randn(E, K, M, generator=g) / K ** 0.5
    print("case", N, K, M, E, flush=True)
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    q, s = orc.quantize_fp8_block(w)
    wd = orc.dequantize_fp8_block(q, s)
    c = pkg.ops.gmm_fp8w(a.to(dev), q.to(dev), s.to(dev), off)
    torch.testing.assert_close(c.cpu().float(), orc.gmm(a.float(), wd, bs), **TOL)
    # transposed operand: the same matrices stored [E, M, K]
    qt, st = orc.quantize_fp8_block(w.transpose(1, 2).contiguous())
    wtd = orc.dequantize_fp8_block(qt, st)
    ct = pkg.ops.gmm_fp8w(a.to(dev), qt.to(dev), st.to(dev), off, trans_b=True)
    torch.testing.assert_close(ct.cpu().float(), orc.gmm(a.float(), wtd, bs, trans_b=True), **TOL)


@pytest.mark.parametrize("act", ["silu"])
def test_fp8_expert_shard_forward_and_dx(pkg, orc, dev, act):
    """The DeepSeek-V3-shaped shard (32 local experts, ~128 rows each, some empty) at a reduced
    width: forward and dX against the oracle's expert MLP on the dequantised weights."""
    w = pkg.configs.scaled(pkg.configs.WORKLOADS["dsv3_shard"], hidden=1024, ffn=512)
    E, H, F = w.experts, w.hidden, w.ffn
    bs = pkg.configs.multinomial_counts(4096, E, seed=11, empty=2)
    N = int(bs.sum())
    g = torch.Generator().manual_seed(3)
    x = torch.randn(N, H, generator=g).bfloat16()
    w1 = (torch.randn(E, H, 2 * F, generator=g) / H ** 0.5).bfloat16()
    w2 = (torch.randn(E, F, H, generator=g) / F ** 0.5).bfloat16()
    go = torch.randn(N, H, generator=g).bfloat16()
    q1, s1 = pkg.ops.quantize_fp8_block(w1.to(dev))
    q2, s2 = pkg.ops.quantize_fp8_block(w2.to(dev))
    xs = x.to(dev).requires_grad_(True)
    out = pkg.mlp.fp8_gated_experts(xs, q1, s1, q2, s2, bs, act)
    out.backward(go.to(dev))
    d1 = orc.dequantize_fp8_block(q1.cpu(), s1.cpu())
    d2 = orc.dequantize_fp8_block(q2.cpu(), s2.cpu())
    xo = x.clone().requires_grad_(True)
    # the oracle rounds fc1 and the activation to bf16 between the ops, as the kernels do
    ref = orc.grouped_mlp(xo, d1, d2, bs)
    ref.backward(go)
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach().float(), **TOL)
    torch.testing.assert_close(xs.grad.cpu().float(), xo.grad.float(), **TOL)
    # the module form built from a GroupedMLP
    cfg = pkg.config.MoEConfig(hidden_size=H, moe_ffn_hidden_size=F, num_moe_experts=E,
                               moe_router_topk=8, params_dtype=torch.bfloat16)
    mlp = pkg.mlp.GroupedMLP(E, cfg, device=dev)
    with torch.no_grad():
        mlp.weight1.view(E, H, 2 * F).copy_(w1.to(dev))
        mlp.weight2.view(E, F, H).copy_(w2.to(dev))
    fp8 = pkg.mlp.Fp8GroupedMLP(mlp)
    out2, _ = fp8(x.to(dev), bs)
    assert torch.equal(out2, out.detach())


def test_full_size_fp8_expert_shard_against_the_oracle_evaluated_on_the_gpu(pkg, orc, dev):
    """The DeepSeek-V3-shaped shard at its real width (32 local experts, H 7168, F 2048, 4096 routed
    rows, two experts empty): quantiser bit-exact against the oracle's, forward and dX against the
    oracle's expert MLP on the dequantised weights, evaluated by torch on GPU tensors."""
    w = pkg.configs.WORKLOADS["dsv3_shard"]
    E, H, F = w.experts, w.hidden, w.ffn
    bs = pkg.configs.multinomial_counts(4096, E, seed=11, empty=2)
    N = int(bs.sum())
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(N, H, generator=g, device=dev).bfloat16()
    w1 = (torch.randn(E, H, 2 * F, generator=g, device=dev) / H ** 0.5).bfloat16()
    w2 = (torch.randn(E, F, H, generator=g, device=dev) / F ** 0.5).bfloat16()
    go = torch.randn(N, H, generator=g, device=dev).bfloat16()
    q1, s1 = pkg.ops.quantize_fp8_block(w1)
    q2, s2 = pkg.ops.quantize_fp8_block(w2)
    oq1, os1 = orc.quantize_fp8_block(w1)
    assert torch.equal(q1.view(torch.uint8), oq1.view(torch.uint8)) and torch.equal(s1, os1)
    xs = x.clone().requires_grad_(True)
    out = pkg.mlp.fp8_gated_experts(xs, q1, s1, q2, s2, bs, "silu")
    out.backward(go)
    d1 = orc.dequantize_fp8_block(q1, s1)
    d2 = orc.dequantize_fp8_block(q2, s2)
    xo = x.clone().requires_grad_(True)
    ref = orc.grouped_mlp(xo, d1, d2, bs)
    ref.backward(go)
    torch.testing.assert_close(out.detach().float(), ref.detach().float(), **TOL)
    torch.testing.assert_close(xs.grad.float(), xo.grad.float(), **TOL)


# ------------------------------------------------------------------------------------------
# fp8 on both sides: row-quantised activations on the block-scaled fp8 MFMA
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("N,K", [(37, 304), (256, 1024), (1, 8), (500, 7168), (64, 136)])
def test_row_quantiser_matches_the_oracle_bit_for_bit(pkg, orc, dev, dtype, N, K):
    g = torch.Generator().manual_seed(N + K)
    spread = torch.logspace(-4, 4, N) if dtype != torch.float16 else torch.logspace(-2, 2, N)
    x = torch.randn(N, K, generator=g) * spread.unsqueeze(1)
    x[0, : min(K, 128)] = 0                                  # an all-zero block
    if K >= 256:
        x[N - 1, 128:256] = 448.0                            # exponent 0 exactly
    x = x.to(dtype)
    q, s = pkg.ops.quantize_fp8_rows(x.to(dev))
    oq, oe = orc.quantize_fp8_rows(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.int32 and s.shape == ((K + 127) // 128, N)
    assert torch.equal(pkg.ops.row_scale_exponents(s).cpu(), oe)
    sb = s.cpu()
    assert torch.equal(sb & 0xFF, (sb >> 8) & 0xFF) and torch.equal(sb & 0xFF, (sb >> 24) & 0xFF)
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("N,F", [(37, 256), (500, 2048), (3, 128), (64, 1152)])
def test_activation_and_quantiser_in_one_pass_equal_the_two_launches(pkg, dev, dtype, act, N, F):
    """glu_fwd / glu_bwd followed by the row quantiser, fused: the same codes and scales, bit for bit
    (the fused kernels round the activation's result to the dtype before they quantise it)."""
    g = torch.Generator().manual_seed(N + F)
    spread = torch.logspace(-2, 2, N)
    y = (torch.randn(N, 2 * F, generator=g) * spread.unsqueeze(1)).to(dtype).to(dev)
    d = (torch.randn(N, F, generator=g) * spread.flip(0).unsqueeze(1)).to(dtype).to(dev)
    y[0, :128] = 0  # a block whose activation is all zero
    q2, s2 = pkg.ops.quantize_fp8_rows(pkg.ops.glu_fwd(y, act))
    q1, s1 = pkg.ops.glu_fwd_quantize_fp8_rows(y, act)
    assert torch.equal(s1, s2) and torch.equal(q1.view(torch.uint8), q2.view(torch.uint8))
    q2, s2 = pkg.ops.quantize_fp8_rows(pkg.ops.glu_bwd(d, y, act))
    q1, s1 = pkg.ops.glu_bwd_quantize_fp8_rows(d, y, act)
    assert s1.shape == (2 * F // 128, N)
    assert torch.equal(s1, s2) and torch.equal(q1.view(torch.uint8), q2.view(torch.uint8))


def test_activation_quantiser_refuses_what_it_is_not_built_for(pkg, dev):
    y = torch.randn(8, 2 * 192, device=dev, dtype=torch.bfloat16)      # F = 192: not a multiple of 128
    d = torch.randn(8, 192, device=dev, dtype=torch.bfloat16)
    q, s = pkg.ops.glu_fwd_quantize_fp8_rows(y)                           # the forward takes multiples of 8
    q2, s2 = pkg.ops.quantize_fp8_rows(pkg.ops.glu_fwd(y))
    assert torch.equal(s, s2) and torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    with pytest.raises(AssertionError):
        pkg.ops.glu_bwd_quantize_fp8_rows(d, y)
    lib = pkg._C.lib()
    q = torch.empty(8, 384, dtype=torch.uint8, device=dev)
    s = torch.empty(3, 8, dtype=torch.int32, device=dev)
    st = lib.gmoe_glu_bwd_quantize_fp8_rows(d.data_ptr(), y.data_ptr(), pkg._C.GMOE_BF16, 8, 192, 0,
                                            q.data_ptr(), s.data_ptr(), None)
    assert st != 0 and b"not supported" in lib.gmoe_status_string(st)


def test_fp8a_reads_every_weight_code_and_row_scale_exactly(pkg, orc, dev):
    """c = (2^r I) @ w with the rows of the identity scaled by powers of two: the row scales pass
    through the MFMA's scale operand, the weight codes through its fp8 operand, the weight scales
    through the fold; every output is one exact product (a bf16 value)."""
    codes = torch.arange(256, dtype=torch.uint8)
    K = M = 256
    wq = (codes.repeat(K, 1) + torch.arange(K, dtype=torch.uint8)[:, None]).to(torch.uint8)
    wq[wq == 0x7f] = 0
    wq[wq == 0xff] = 0
    q = wq.view(torch.float8_e4m3fn).unsqueeze(0)
    scale = torch.tensor([[[1.0, 0.5], [2.0, 0.25]]], dtype=torch.bfloat16)
    w = q.float()[0] * scale.float()[0].repeat_interleave(128, 0).repeat_interleave(128, 1)
    rows = torch.ldexp(torch.ones(K), torch.arange(K) % 23 - 11)          # 2^-11 .. 2^11
    a = torch.diag(rows).bfloat16()
    aq, asc = pkg.ops.quantize_fp8_rows(a.to(dev))
    assert torch.equal(orc.dequantize_fp8_rows(aq.cpu(), pkg.ops.row_scale_exponents(asc).cpu()), a.float())
    off = torch.tensor([0, K], dtype=torch.int64, device=dev)
    c = pkg.ops.gmm_fp8a(aq, asc, q.to(dev), scale.to(dev), off)
    want = rows.unsqueeze(1) * w
    assert torch.equal(c.cpu().float(), want.bfloat16().float())
    ct = pkg.ops.gmm_fp8a(aq, asc, q.to(dev), scale.to(dev), off, trans_b=True)
    assert torch.equal(ct.cpu().float(), (rows.unsqueeze(1) * w.t()).bfloat16().float())


FP8A_CASES = [  # N, K, M, E, empty: few rows per expert, K a multiple of 64
    (512, 256, 384, 4, ()),
    (300, 128, 144, 3, (1,)),
    (4096, 1024, 512, 32, (3, 17)),
    (1000, 256, 512, 4, ()),             # experts beyond 192 rows: two row chunks
    (700, 128, 528, 3, ()),
    (37, 64, 16, 5, (2,)),
    (900, 448, 784, 9, (0, 8)),          # an odd number of stages
    (3000, 128, 272, 300, (5, 299)),     # more experts than the kernel ranks by cost
    (2600, 64, 2064, 40, (0, 1, 2)),     # more items than workgroups, uneven runs
    (3000, 256, 384, 4, ()),             # many rows per expert: row chunks that stream the weights again
]


@pytest.mark.parametrize("N,K,M,E,empty", FP8A_CASES)
def test_gmm_fp8a_both_layouts(pkg, orc, dev, N, K, M, E, empty):
    """Against the oracle's matmul of the dequantised operands.  The products are exact on both sides;
    what remains is the output's bf16 rounding (half a unit in the last place, at most 2^-8 of the
    value) and the summation: the block-scaled MFMA adds its 64 products with an internal precision
    of its own (measured against an fp64 sum over these cases: typically within 2^-17 of the sum of the
    terms' magnitudes, 2^-14.9 at worst among 5 million outputs of a single-instruction reduction), the
    stages are added in fp32.  The bound allows 2^-14 of that sum."""
    bs = splits(N, E, seed=N + E, empty=empty)
    g = torch.Generator().manual_seed(N)
    a = (torch.randn(N, K, generator=g) * torch.logspace(-2, 2, N).unsqueeze(1)).bfloat16()
    w = torch.randn(E, K, M, generator=g) / K ** 0.5
    print("case", N, K, M, E, flush=True)
    off = pkg.ops.expert_offsets_from_batch_sizes(bs, dev)
    aq, asc = pkg.ops.quantize_fp8_rows(a.to(dev))
    ad = orc.dequantize_fp8_rows(aq.cpu(), pkg.ops.row_scale_exponents(asc).cpu())
    q, s = orc.quantize_fp8_block(w)
    wd = orc.dequantize_fp8_block(q, s)
    tol = dict(rtol=2.0 ** -8, atol=0.0)
    c = pkg.ops.gmm_fp8a(aq, asc, q.to(dev), s.to(dev), off)
    ref = orc.gmm(ad, wd, bs)
    err = (c.cpu().float() - ref).abs()
    bound = ref.abs() * tol["rtol"] + orc.gmm(ad.abs(), wd.abs(), bs) * 2.0 ** -14
    assert torch.all(err <= bound), float((err - bound).max())
    qt, st = orc.quantize_fp8_block(w.transpose(1, 2).contiguous())
    wtd = orc.dequantize_fp8_block(qt, st)
    ct = pkg.ops.gmm_fp8a(aq, asc, qt.to(dev), st.to(dev), off, trans_b=True)
    reft = orc.gmm(ad, wtd, bs, trans_b=True)
    errt = (ct.cpu().float() - reft).abs()
    boundt = reft.abs() * tol["rtol"] + orc.gmm(ad.abs(), wtd.abs(), bs, trans_b=True) * 2.0 ** -14
    assert torch.all(errt <= boundt), float((errt - boundt).max())
    # and within the bf16 tolerance of the product of the unquantised rows, for orientation only
    full = orc.gmm(a.float(), wd, bs)
    rel = (c.cpu().float() - full).norm() / full.norm()
    print("relative error against bf16 rows:", float(rel), flush=True)
    assert rel < 0.05


def test_gmm_fp8a_refuses_what_it_is_not_built_for(pkg, dev):
    a = torch.zeros(300, 96, device=dev, dtype=torch.bfloat16)
    aq, asc = pkg.ops.quantize_fp8_rows(a)
    q = torch.zeros(4, 96, 384, device=dev, dtype=torch.float8_e4m3fn)
    s = torch.ones(4, 1, 3, device=dev, dtype=torch.bfloat16)
    off = torch.tensor([0, 75, 150, 225, 300], dtype=torch.int64, device=dev)
    with pytest.raises(RuntimeError):     # K = 96: not whole 64-element stages
        pkg.ops.gmm_fp8a(aq, asc, q, s, off)


def test_fp8_expert_shard_with_fp8_activations(pkg, orc, dev):
    """The shard's expert MLP with the rows of all four products quantised as well: forward and dX
    against the oracle's MLP evaluated on the same quantised operands (the oracle quantises what the
    kernels quantise: x, the activation, dy and d(fc1))."""
    w = pkg.configs.scaled(pkg.configs.WORKLOADS["dsv3_shard"], hidden=1024, ffn=512)
    E, H, F = w.experts, w.hidden, w.ffn
    bs = pkg.configs.multinomial_counts(4096, E, seed=11, empty=2)
    N = int(bs.sum())
    g = torch.Generator().manual_seed(3)
    x = torch.randn(N, H, generator=g).bfloat16()
    w1 = (torch.randn(E, H, 2 * F, generator=g) / H ** 0.5).bfloat16()
    w2 = (torch.randn(E, F, H, generator=g) / F ** 0.5).bfloat16()
    go = torch.randn(N, H, generator=g).bfloat16()
    q1, s1 = pkg.ops.quantize_fp8_block(w1.to(dev))
    q2, s2 = pkg.ops.quantize_fp8_block(w2.to(dev))
    xs = x.to(dev).requires_grad_(True)
    out = pkg.mlp.fp8_gated_experts(xs, q1, s1, q2, s2, bs, "silu", fp8_activations=True)
    out.backward(go.to(dev))
    d1 = orc.dequantize_fp8_block(q1.cpu(), s1.cpu())
    d2 = orc.dequantize_fp8_block(q2.cpu(), s2.cpu())

    def rq(t):
        return orc.dequantize_fp8_rows(*orc.quantize_fp8_rows(t))

    fc1 = orc.gmm(rq(x), d1, bs).bfloat16()
    h = orc.swiglu(fc1.float()).bfloat16()
    ref = orc.gmm(rq(h), d2, bs).bfloat16()
    dact = orc.gmm(rq(go), d2, bs, trans_b=True).bfloat16()
    dfc1 = orc.swiglu_back(dact.float(), fc1.float()).bfloat16()
    dx = orc.gmm(rq(dfc1), d1, bs, trans_b=True).bfloat16()
    # A last-bit difference in a bf16 intermediate (fc1, the activation, d(fc1)) can move its fp8
    # code by one step (2^-3 relative), so a few elements of the chained result differ by more than
    # the bf16 tolerance: the bulk must be within it, the whole within 1 % in norm
    for what, got, want in (("out", out.detach().cpu().float(), ref.float()),
                            ("dx", xs.grad.cpu().float(), dx.float())):
        outside = ((got - want).abs() > TOL["atol"] + TOL["rtol"] * want.abs()).float().mean().item()
        rel = ((got - want).norm() / want.norm()).item()
        print(what, "outside rtol/atol:", outside, "relative error in norm:", rel, flush=True)
        assert outside < 2e-3 and rel < 1e-2
    # the unquantised-row path for orientation: the fp8 rows cost a few per cent
    out16 = pkg.mlp.fp8_gated_experts(x.to(dev), q1, s1, q2, s2, bs, "silu")
    rel = (out.detach().float() - out16.float()).norm() / out16.float().norm()
    print("fp8 rows against bf16 rows, relative:", float(rel), flush=True)
    assert rel < 0.08

