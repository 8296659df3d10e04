"""Writes tests/golden/*.npz: small input / expected-output vectors of the MoE hot path.

The reference holds no golden vectors for this path and its Python was read, not run, so the
expected values come from the CPU oracle (oracle/moe_oracle.py), whose functions are pinned by
tests/test_oracle.py against brute force, closed forms and transformers' Mixtral block.  The
fixtures freeze those values: a later change of the oracle, of torch or of the kernels that moves
an integer result or a float beyond tolerance fails tests/test_golden.py.

    python tests/golden/make_golden.py        # regenerates the files next to this script
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import moe_oracle as orc  # noqa: E402
import __graft_entry__ as entry  # noqa: E402


def routing_cases():
    out = {}
    g = torch.Generator().manual_seed(20240521)
    # (name, T, E, k, kwargs); logits in fp32, some rows with exact ties
    cases = [("softmax_top2", 96, 8, 2, {}), ("top8_of_64", 80, 64, 8, {}),
             ("pre_softmax", 64, 12, 3, dict(use_pre_softmax=True)),
             ("sigmoid_bias", 64, 16, 4, dict(score_function="sigmoid")),
             ("group_limited", 64, 32, 4, dict(num_groups=4, group_topk=2)),
             ("capacity_probs", 120, 8, 2, dict(capacity_factor=0.6)),
             ("capacity_position_pad", 120, 8, 2, dict(capacity_factor=0.6, drop_policy="position",
                                                       pad_to_capacity=True))]
    for name, T, E, k, kw in cases:
        logits = torch.randn(T, E, generator=g)
        logits[3] = logits[3, 0]            # a row of equal logits: lowest indices win
        logits[7, 1] = logits[7, 5]         # a pair of equal logits
        kw = dict(kw)
        if name == "sigmoid_bias":
            kw["expert_bias"] = 0.1 * torch.randn(E, generator=g)
            out[name + ".expert_bias"] = kw["expert_bias"].numpy()
        probs, rmap, counts = orc.topk_softmax_with_capacity(logits, k, **kw)
        out[name + ".logits"] = logits.numpy()
        out[name + ".probs"] = probs.numpy()
        out[name + ".routing_map"] = rmap.numpy()
        out[name + ".tokens_per_expert"] = counts.numpy()
        sorted_indices = orc.permute(torch.zeros(T, 1), rmap)[1]
        out[name + ".sorted_indices"] = sorted_indices.numpy()
    return out


def loss_cases():
    g = torch.Generator().manual_seed(77)
    T, E, k = 256, 8, 2
    logits = torch.randn(T, E, generator=g).requires_grad_(True)
    probs, rmap, counts = orc.topk_softmax_with_capacity(logits, k)
    scores = torch.softmax(logits, dim=-1, dtype=torch.float32)
    aux = orc.switch_load_balancing_loss(scores, counts, k, 0.01)
    z = orc.z_loss(logits, 0.001)
    (aux + z).backward()
    return {"logits": logits.detach().numpy(), "aux_loss": aux.detach().numpy(),
            "z_loss": z.detach().numpy(), "grad_logits": logits.grad.numpy()}


def layer_case():
    """A whole layer small enough to store: T=48 (S=24, B=2), H=32, F=48, E=4, top-2, fp32."""
    g = torch.Generator().manual_seed(5)
    S, B, H, Fe, E, k = 24, 2, 32, 48, 4, 2
    t = dict(x=torch.randn(S, B, H, generator=g), w_r=0.3 * torch.randn(E, H, generator=g),
             w1=torch.randn(E, H, 2 * Fe, generator=g) / H ** 0.5,
             w2=torch.randn(E, Fe, H, generator=g) / Fe ** 0.5, dy=torch.randn(S, B, H, generator=g),
             residual=torch.randn(S, B, H, generator=g))
    leaf = {n: v.clone().requires_grad_(True) for n, v in t.items() if n in ("x", "w_r", "w1", "w2")}
    out, _, info = orc.moe_layer(leaf["x"], leaf["w_r"], leaf["w1"], leaf["w2"], k,
                                 residual=t["residual"])
    out.backward(t["dy"])
    res = {n: v.numpy() for n, v in t.items()}
    res["out"] = out.detach().numpy()
    for n, v in leaf.items():
        res["grad_" + n] = v.grad.numpy()
    return res


def norm_case():
    """Pre-router RMS norm, fp32: 20 rows of 64 with mixed magnitudes, output and both gradients."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(20, 64, generator=g) * torch.logspace(-2, 2, 20).unsqueeze(1)
    w = 1.0 + 0.3 * torch.randn(64, generator=g)
    dy = torch.randn(20, 64, generator=g)
    xl, wl = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y = orc.rms_norm(xl, wl, 1e-5)
    y.backward(dy)
    return {"x": x.numpy(), "weight": w.numpy(), "dy": dy.numpy(), "eps": np.float32(1e-5),
            "y": y.detach().numpy(), "grad_x": xl.grad.numpy(), "grad_weight": wl.grad.numpy()}


def skew_histogram():
    """Config 4: the realised top-2 expert loads of the Mixtral-shape skewed-routing workload
    (Zipf(1.2) logit bias, one expert forced empty), T = 16384."""
    pkg = entry.load_package()
    w = pkg.configs.WORKLOADS["mixtral_skew"]
    inp = pkg.configs.make_inputs(w, with_weights=False)
    x = inp["x"].float().view(-1, w.hidden)
    logits = (x @ inp["w_r"].float().t()).to(w.dtype) + inp["logit_bias"].to(w.dtype)
    _, _, counts = orc.topk_softmax_with_capacity(logits, w.topk)
    return {"tokens_per_expert": counts.numpy(), "logit_bias": inp["logit_bias"].numpy()}


def main():
    torch.set_num_threads(1)  # summation order of the CPU matmuls fixed
    np.savez_compressed(os.path.join(HERE, "routing.npz"), **routing_cases())
    np.savez_compressed(os.path.join(HERE, "losses.npz"), **loss_cases())
    np.savez_compressed(os.path.join(HERE, "layer_small.npz"), **layer_case())
    np.savez_compressed(os.path.join(HERE, "mixtral_skew_histogram.npz"), **skew_histogram())
    np.savez_compressed(os.path.join(HERE, "rms_norm.npz"), **norm_case())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
