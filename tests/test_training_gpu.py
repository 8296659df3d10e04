"""A few optimiser steps of the MoE layer against transformers' Mixtral block on the GPU, in the
manner of the reference's own correctness test (tests/models/test_moe_correctness.py:104-214: the
mixtral-test shape, bf16, Adam, the same random batches for both, losses compared with
torch.allclose(rtol=5e-3))."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dispatcher", ["allgather", "alltoall"])
@pytest.mark.parametrize("pre_norm", [False, True])
def test_losses_track_the_hf_mixtral_block_over_adam_steps(pkg, dev, dispatcher, pre_norm):
    mm = pytest.importorskip("transformers.models.mixtral.modeling_mixtral")
    from transformers import MixtralConfig

    E, H, Fe, k, S, B = 4, 128, 256, 2, 32, 2     # tests/utils/model_configs/mixtral-test.yaml:3-27
    hf_cfg = MixtralConfig(hidden_size=H, intermediate_size=Fe, num_local_experts=E, num_experts_per_tok=k,
                           num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=2, vocab_size=64,
                           rms_norm_eps=1e-5)
    torch.manual_seed(11)
    blk = mm.MixtralSparseMoeBlock(hf_cfg)
    if not hasattr(blk.experts, "gate_up_proj"):
        pytest.skip("this transformers version keeps per-expert modules")
    with torch.no_grad():
        for p in blk.parameters():
            p.normal_(0.0, 0.05)
    hf_norm = mm.MixtralRMSNorm(H, eps=1e-5)
    blk = blk.to(dev, torch.bfloat16).train()
    hf_norm = hf_norm.to(dev, torch.bfloat16)

    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=Fe, moe_router_topk=k,
                        moe_router_load_balancing_type="none", moe_token_dispatcher_type=dispatcher,
                        params_dtype=torch.bfloat16, norm_epsilon=1e-5)
    router = pkg.GalvatronMoERouter(cfg, device=dev).train()
    mlp = pkg.GalvatronMoEMLP(cfg, device=dev).train()
    pre = pkg.PreRouterNorm(cfg, device=dev)
    with torch.no_grad():
        router.router.weight.copy_(blk.gate.weight)
        # gate_up_proj[e] = [w1; w3] ([2F,H]), down_proj[e] = w2 ([H,F]); the grouped layout is their transpose
        mlp.experts.weight1.view(E, H, 2 * Fe).copy_(blk.experts.gate_up_proj.transpose(1, 2))
        mlp.experts.weight2.view(E, Fe, H).copy_(blk.experts.down_proj.transpose(1, 2))
    ours = list(router.parameters()) + list(mlp.parameters()) + (list(pre.parameters()) if pre_norm else [])
    theirs = list(blk.parameters()) + (list(hf_norm.parameters()) if pre_norm else [])
    opt_a = torch.optim.Adam(ours, lr=1e-3)
    opt_b = torch.optim.Adam(theirs, lr=1e-3)
    g = torch.Generator(device=dev).manual_seed(5)
    losses_a, losses_b = [], []
    for step in range(6):
        x = torch.randn(S, B, H, generator=g, device=dev).bfloat16()
        target = torch.randn(S, B, H, generator=g, device=dev)
        # this build
        opt_a.zero_grad()
        if pre_norm:
            h, residual = pre(x)
        else:
            h, residual = x, None
        probs, rmap = router(h)
        out = mlp(h, residual, probs, rmap)
        la = (out.float() - target).pow(2).mean()
        la.backward()
        opt_a.step()
        # transformers
        opt_b.zero_grad()
        hb = hf_norm(x) if pre_norm else x
        ref = blk(hb)
        ref = ref[0] if isinstance(ref, tuple) else ref
        if pre_norm:
            ref = ref + x
        lb = (ref.float() - target).pow(2).mean()
        lb.backward()
        opt_b.step()
        losses_a.append(la.item())
        losses_b.append(lb.item())
    print("losses", losses_a, losses_b, flush=True)
    assert torch.allclose(torch.tensor(losses_a), torch.tensor(losses_b), rtol=5e-3)
    # and the weights moved together
    torch.testing.assert_close(router.router.weight.float(), blk.gate.weight.float(), rtol=0, atol=5e-3)
