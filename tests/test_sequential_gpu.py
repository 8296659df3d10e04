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
