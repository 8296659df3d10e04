"""Committed input / expected-output vectors (tests/golden/*.npz, written by tests/golden/
make_golden.py from the pinned oracle): the oracle must keep reproducing them on the CPU, and the HIP
path must reproduce them on the GPU: integers bit for bit, floats within the stated tolerance."""
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

ROUTING = {
    "softmax_top2": (2, {}), "top8_of_64": (8, {}), "pre_softmax": (3, dict(use_pre_softmax=True)),
    "sigmoid_bias": (4, dict(score_function="sigmoid")),
    "group_limited": (4, dict(num_groups=4, group_topk=2)),
    "capacity_probs": (2, dict(capacity_factor=0.6)),
    "capacity_position_pad": (2, dict(capacity_factor=0.6, drop_policy="position", pad_to_capacity=True)),
}


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def routing_case(z, name, device="cpu"):
    k, kw = ROUTING[name]
    kw = dict(kw)
    if name + ".expert_bias" in z:
        kw["expert_bias"] = torch.from_numpy(z[name + ".expert_bias"]).to(device)
    return torch.from_numpy(z[name + ".logits"]).to(device), k, kw


@pytest.mark.parametrize("name", sorted(ROUTING))
def test_oracle_reproduces_golden_routing(orc, name):
    z = load("routing.npz")
    logits, k, kw = routing_case(z, name)
    probs, rmap, counts = orc.topk_softmax_with_capacity(logits, k, **kw)
    assert np.array_equal(rmap.numpy(), z[name + ".routing_map"])
    assert np.array_equal(counts.numpy(), z[name + ".tokens_per_expert"])
    np.testing.assert_allclose(probs.numpy(), z[name + ".probs"], rtol=1e-6, atol=1e-7)
    assert np.array_equal(orc.permute(torch.zeros(logits.shape[0], 1), rmap)[1].numpy(),
                          z[name + ".sorted_indices"])


def test_oracle_reproduces_golden_layer_and_losses(orc):
    z = load("layer_small.npz")
    t = {n: torch.from_numpy(z[n]) for n in ("x", "w_r", "w1", "w2", "dy", "residual")}
    leaf = {n: t[n].clone().requires_grad_(True) for n in ("x", "w_r", "w1", "w2")}
    out, _, _ = orc.moe_layer(leaf["x"], leaf["w_r"], leaf["w1"], leaf["w2"], 2, residual=t["residual"])
    out.backward(t["dy"])
    np.testing.assert_allclose(out.detach().numpy(), z["out"], rtol=1e-5, atol=1e-5)
    for n, v in leaf.items():
        np.testing.assert_allclose(v.grad.numpy(), z["grad_" + n], rtol=1e-4, atol=1e-5)
    zl = load("losses.npz")
    logits = torch.from_numpy(zl["logits"]).requires_grad_(True)
    _, _, counts = orc.topk_softmax_with_capacity(logits, 2)
    aux = orc.switch_load_balancing_loss(torch.softmax(logits, -1, dtype=torch.float32), counts, 2, 0.01)
    zloss = orc.z_loss(logits, 0.001)
    (aux + zloss).backward()
    np.testing.assert_allclose(aux.item(), zl["aux_loss"], rtol=1e-6)
    np.testing.assert_allclose(zloss.item(), zl["z_loss"], rtol=1e-6)
    np.testing.assert_allclose(logits.grad.numpy(), zl["grad_logits"], rtol=1e-5, atol=1e-8)


def test_skew_histogram_fixture_is_zipf_with_an_empty_expert():
    z = load("mixtral_skew_histogram.npz")
    counts = z["tokens_per_expert"]
    assert counts.sum() == 16384 * 2 and (counts == 0).sum() >= 1
    nz = np.sort(counts[counts > 0])[::-1].astype(np.float64)
    # load shares fall off like rank^-1.2 (each within a factor of two, 25 % on average in log)
    ideal = np.arange(1, len(nz) + 1) ** -1.2
    ratio = (nz / nz.sum()) / (ideal / ideal.sum())
    assert np.all(ratio < 2.0) and np.all(ratio > 0.5) and np.abs(np.log(ratio)).mean() < 0.25


# ---- GPU ------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(ROUTING))
def test_hip_routing_matches_golden(pkg, dev, name):
    z = load("routing.npz")
    logits, k, kw = routing_case(z, name, dev)
    probs, rmap, counts = pkg.topk_softmax_with_capacity(logits, k, **kw)
    assert np.array_equal(rmap.cpu().numpy(), z[name + ".routing_map"])
    assert np.array_equal(counts.cpu().numpy(), z[name + ".tokens_per_expert"])
    np.testing.assert_allclose(probs.cpu().numpy(), z[name + ".probs"], rtol=1e-5, atol=1e-6)
    T = logits.shape[0]
    n_out = int(z[name + ".sorted_indices"].shape[0])
    _, sorted_indices = pkg.permute(torch.zeros(T, 8, device=dev), rmap, num_out_tokens=n_out)
    assert np.array_equal(sorted_indices.cpu().numpy(), z[name + ".sorted_indices"])


def test_oracle_reproduces_golden_rms_norm(orc):
    z = load("rms_norm.npz")
    x = torch.from_numpy(z["x"]).requires_grad_(True)
    w = torch.from_numpy(z["weight"]).requires_grad_(True)
    y = orc.rms_norm(x, w, float(z["eps"]))
    y.backward(torch.from_numpy(z["dy"]))
    np.testing.assert_allclose(y.detach().numpy(), z["y"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(x.grad.numpy(), z["grad_x"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(w.grad.numpy(), z["grad_weight"], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_hip_rms_norm_matches_golden(pkg, dev):
    z = load("rms_norm.npz")
    x = torch.from_numpy(z["x"]).to(dev).requires_grad_(True)
    w = torch.from_numpy(z["weight"]).to(dev).requires_grad_(True)
    y = pkg.norm.rms_norm(x, w, float(z["eps"]))
    y.backward(torch.from_numpy(z["dy"]).to(dev))
    np.testing.assert_allclose(y.detach().cpu().numpy(), z["y"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(x.grad.cpu().numpy(), z["grad_x"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(w.grad.cpu().numpy(), z["grad_weight"], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dispatcher", ["allgather", "alltoall"])
def test_hip_layer_matches_golden(pkg, dev, dispatcher):
    z = load("layer_small.npz")
    E, H, F2 = z["w1"].shape
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=F2 // 2, moe_router_topk=2,
                        moe_router_load_balancing_type="none", moe_token_dispatcher_type=dispatcher,
                        params_dtype=torch.float32)
    router = pkg.GalvatronMoERouter(cfg, device=dev)
    mlp = pkg.GalvatronMoEMLP(cfg, device=dev)
    with torch.no_grad():
        router.router.weight.copy_(torch.from_numpy(z["w_r"]))
        mlp.experts.weight1.view(E, H, F2).copy_(torch.from_numpy(z["w1"]))
        mlp.experts.weight2.view(E, F2 // 2, H).copy_(torch.from_numpy(z["w2"]))
    x = torch.from_numpy(z["x"]).to(dev).requires_grad_(True)
    probs, rmap = router(x)
    out = mlp(x, torch.from_numpy(z["residual"]).to(dev), probs, rmap)
    out.backward(torch.from_numpy(z["dy"]).to(dev))
    tol = dict(rtol=2e-3, atol=2e-4)   # fp32 MFMA accumulation order against the CPU's
    np.testing.assert_allclose(out.detach().cpu().numpy(), z["out"], **tol)
    np.testing.assert_allclose(x.grad.cpu().numpy(), z["grad_x"], **tol)
    np.testing.assert_allclose(router.router.weight.grad.cpu().numpy(), z["grad_w_r"], **tol)
    np.testing.assert_allclose(mlp.experts.weight1.grad.view(E, H, F2).cpu().numpy(), z["grad_w1"], **tol)
    np.testing.assert_allclose(mlp.experts.weight2.grad.view(E, F2 // 2, H).cpu().numpy(), z["grad_w2"], **tol)


@pytest.mark.gpu
def test_hip_skewed_routing_reproduces_the_stored_histogram(pkg, dev):
    z = load("mixtral_skew_histogram.npz")
    w = pkg.configs.WORKLOADS["mixtral_skew"]
    inp = pkg.configs.make_inputs(w, with_weights=False)
    x = inp["x"].float().view(-1, w.hidden)
    logits = (x @ inp["w_r"].float().t()).to(w.dtype) + inp["logit_bias"].to(w.dtype)
    _, _, counts = pkg.topk_softmax_with_capacity(logits.to(dev), w.topk)
    assert np.array_equal(counts.cpu().numpy(), z["tokens_per_expert"])
