"""The layer step (forward + backward) captured in a HIP graph: every replay gives the bits of the
eager step.  The library holds no state and never synchronises, its launches go to the stream it is
given, buffers are cleared by fill kernels (no memset nodes), and the dispatchers read no count on
the host, so the whole step records as it runs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def build(pkg, dev, dtype, E, H, F, k, shared, overlap, lb):
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=F, moe_router_topk=k,
                        moe_router_load_balancing_type=lb, moe_aux_loss_coeff=0.01,
                        moe_z_loss_coeff=1e-3 if lb == "aux_loss" else None,
                        moe_token_dispatcher_type="allgather", params_dtype=dtype,
                        moe_shared_expert_intermediate_size=shared,
                        moe_shared_expert_overlap=overlap)
    torch.manual_seed(7)
    return (pkg.GalvatronMoERouter(cfg, device=dev).train(), pkg.GalvatronMoEMLP(cfg, device=dev).train(),
            pkg.PreRouterNorm(cfg, device=dev).train())


@pytest.mark.parametrize("dtype,E,H,F,k,shared,overlap,lb", [
    (torch.float32, 8, 512, 1024, 2, None, False, "aux_loss"),     # the launch-bound small configuration
    (torch.bfloat16, 64, 256, 128, 8, 512, True, "aux_loss"),      # many experts, shared experts on their stream
    (torch.bfloat16, 8, 256, 384, 2, None, False, "seq_aux_loss"),
])
def test_captured_layer_step_replays_the_eager_bits(pkg, dev, dtype, E, H, F, k, shared, overlap, lb):
    S, B = 256, 4
    router, mlp, pre = build(pkg, dev, dtype, E, H, F, k, shared, overlap, lb)
    params = list(router.parameters()) + list(mlp.parameters()) + list(pre.parameters())
    g = torch.Generator().manual_seed(3)
    x = torch.randn(S, B, H, generator=g).to(dtype).to(dev).requires_grad_(True)
    dy = torch.randn(S, B, H, generator=g).to(dtype).to(dev)
    pkg.moe_utils.clear_aux_losses_tracker()

    def step():
        for p in params:
            p.grad = None
        x.grad = None
        h, residual = pre(x)
        probs, rmap = router(h)
        out = mlp(h, residual, probs, rmap)
        out.backward(dy)
        return out

    def snapshot(out):
        return [out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in params]

    # eager reference (also the warm-up that sets kernel attributes and fills the caches)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            want = snapshot(step())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    for p in params:
        p.grad = None
    x.grad = None
    with torch.cuda.graph(graph):
        out = step()
    for replay in range(4):
        graph.replay()
        torch.cuda.synchronize()
        got = [out.detach(), x.grad] + [p.grad for p in params]
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), "replay %d, tensor %d" % (replay, i)
        # the program's own eager work between the replays: another input, then the first again
        with torch.no_grad():
            scratch = torch.randn(S * B, E, device=dev)
            pkg.topk_softmax_with_capacity(scratch, k)
        torch.cuda.synchronize()
    # new input values in the captured buffers: the replay follows them
    with torch.no_grad():
        x.mul_(-0.5)
    graph.replay()
    torch.cuda.synchronize()
    got = [t.clone() for t in [out.detach(), x.grad] + [p.grad for p in params]]
    del graph
    want2 = snapshot(step())
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(got, want2)):
        assert torch.equal(a, b), "new input, tensor %d" % i


@pytest.mark.parametrize("fp8_activations", [False, True])
def test_captured_fp8_expert_step_replays_the_eager_bits(pkg, dev, fp8_activations):
    """Forward + input gradient of the experts on block-scaled fp8 weights (few rows per expert: the
    weight-streaming kernel, with and without the row quantiser in front) as graph replays."""
    E, H, F, N = 8, 512, 256, 640
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=F, params_dtype=torch.bfloat16)
    torch.manual_seed(11)
    fp8 = pkg.Fp8GroupedMLP(pkg.GroupedMLP(E, cfg, device=dev), fp8_activations=fp8_activations)
    counts = torch.tensor([96, 0, 160, 64, 80, 112, 16, 112])
    tpe = counts.to(dev)
    tpe._gmoe_offsets = pkg.ops.expert_offsets_from_batch_sizes(counts, dev)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, H, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    dy = torch.randn(N, H, generator=g).to(torch.bfloat16).to(dev)

    def step():
        x.grad = None
        out, _ = fp8(x, tpe)
        out.backward(dy)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            out = step()
            want = [out.detach().clone(), x.grad.clone()]
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert want[0].abs().max() > 0 and want[1].abs().max() > 0

    graph = torch.cuda.CUDAGraph()
    x.grad = None
    with torch.cuda.graph(graph):
        out = step()
    for replay in range(4):
        graph.replay()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip([out.detach(), x.grad], want)):
            assert torch.equal(a, b), "replay %d, tensor %d" % (replay, i)
        with torch.no_grad():  # eager work of the same kernels between the replays
            fp8(torch.randn(N, H, device=dev, dtype=torch.bfloat16), tpe)
        torch.cuda.synchronize()
    with torch.no_grad():
        x.mul_(-0.5)
    graph.replay()
    torch.cuda.synchronize()
    got = [out.detach().clone(), x.grad.clone()]
    del graph
    out2 = step()
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(got, [out2.detach(), x.grad])):
        assert torch.equal(a, b), "new input, tensor %d" % i
