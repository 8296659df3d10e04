"""Expert-weight layout converters (CPU): Hugging Face Mixtral keys <-> SequentialMLP <-> GroupedMLP.
Pinned on the Mixtral expert formula w2(silu(w1 x) * w3 x) evaluated straight from the HF tensors."""
import torch
import torch.nn.functional as F


def hf_state(E, H, Fe, seed=0):
    g = torch.Generator().manual_seed(seed)
    st = {}
    for e in range(E):
        st["block_sparse_moe.experts.%d.w1.weight" % e] = torch.randn(Fe, H, generator=g) / H ** 0.5
        st["block_sparse_moe.experts.%d.w3.weight" % e] = torch.randn(Fe, H, generator=g) / H ** 0.5
        st["block_sparse_moe.experts.%d.w2.weight" % e] = torch.randn(H, Fe, generator=g) / Fe ** 0.5
    return st


def test_grouped_layout_computes_the_mixtral_expert(pkg, orc):
    E, H, Fe = 4, 24, 40
    st = hf_state(E, H, Fe)
    ck = pkg.checkpoint
    w1, w2 = ck.grouped_from_hf(st, range(E))
    assert w1.shape == (H, E * 2 * Fe) and w2.shape == (E * Fe, H)
    bs = torch.tensor([5, 0, 7, 3])
    x = torch.randn(int(bs.sum()), H, generator=torch.Generator().manual_seed(1))
    got = orc.grouped_mlp(x, w1.view(E, H, 2 * Fe), w2.view(E, Fe, H), bs)
    want, s = [], 0
    for e, n in enumerate(bs.tolist()):
        xe = x[s:s + n]
        k = "block_sparse_moe.experts.%d.%s.weight"
        want.append(F.linear(F.silu(F.linear(xe, st[k % (e, "w1")])) * F.linear(xe, st[k % (e, "w3")]),
                             st[k % (e, "w2")]))
        s += n
    torch.testing.assert_close(got, torch.cat(want), rtol=1e-5, atol=1e-5)


def test_layout_round_trips_are_exact(pkg):
    E, H, Fe = 3, 16, 24
    st = hf_state(E, H, Fe, seed=5)
    ck = pkg.checkpoint
    # a shard holding global experts 1 and 2
    w1, w2 = ck.grouped_from_hf(st, [1, 2])
    back = ck.hf_from_grouped(w1, w2, [1, 2])
    assert set(back) == {k for k in st if ".1." in k or ".2." in k}
    for k, v in back.items():
        assert torch.equal(v, st[k])
    fc1, fc2 = ck.fc_from_grouped(w1, w2, 2)
    assert torch.equal(fc1[0], torch.cat([st["block_sparse_moe.experts.1.w1.weight"],
                                          st["block_sparse_moe.experts.1.w3.weight"]]))
    assert torch.equal(fc2[1], st["block_sparse_moe.experts.2.w2.weight"])
    g1, g2 = ck.grouped_from_fc(fc1, fc2)
    assert torch.equal(g1, w1) and torch.equal(g2, w2)


def test_aux_loss_tracker_and_metrics_logging(pkg):
    """save_to_aux_losses_tracker / track_moe_metrics / clear (moe_utils.py:547-642) on the CPU."""
    mu = pkg.moe_utils
    mu.get_moe_layer_wise_logging_tracker().clear()
    for layer in (1, 2, 3):
        mu.save_to_aux_losses_tracker("load_balancing_loss", torch.tensor(0.5 * layer), layer, 3)
    mu.save_to_aux_losses_tracker("z_loss", torch.tensor(2.0), 2, 3)

    class Writer:
        def __init__(self):
            self.rows = []

        def add_scalar(self, name, value, it):
            self.rows.append((name, float(value), it))

    w, totals = Writer(), {}
    mu.track_moe_metrics(loss_scale=2.0, iteration=7, writer=w, total_loss_dict=totals,
                         per_layer_logging=True)
    got = dict((n, v) for n, v, _ in w.rows)
    assert got["load_balancing_loss"] == 2.0 and got["moe/load_balancing_loss_layer_2"] == 3.0
    assert abs(got["z_loss"] - 4.0 / 3) < 1e-6 and float(totals["load_balancing_loss"]) == 2.0
    assert all(it == 7 for _, _, it in w.rows)
    assert float(mu.get_moe_layer_wise_logging_tracker()["z_loss"]["values"].abs().sum()) == 0.0
    # totals accumulate over calls, a second metric call with wandb-style writer logs per layer
    mu.save_to_aux_losses_tracker("z_loss", torch.tensor(3.0), 1, 3)

    class Wandb:
        def __init__(self):
            self.logged = {}

        def log(self, d, it):
            self.logged.update(d)

    wb = Wandb()
    mu.track_moe_metrics(loss_scale=1.0, iteration=8, writer=w, wandb_writer=wb, total_loss_dict=totals,
                         per_layer_logging=True)
    assert abs(float(totals["z_loss"]) - (4.0 / 3 + 1.0)) < 1e-6
    assert abs(float(wb.logged["z_loss"]) - 1.0) < 1e-6 and wb.logged["moe/z_loss_layer_0"] == 3.0
    t = torch.arange(3)
    assert mu.maybe_move_tensor_to_cpu(t) is t and mu.maybe_move_tensor_to_cpu(None) is None
