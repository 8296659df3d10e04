#!/usr/bin/env python
"""Benchmark of the MoE expert-layer hot path on one MI355X.

A step is one forward + backward of the layer (router -> permute -> grouped SwiGLU MLP -> unpermute)
on seeded synthetic input already resident in HBM.  Prints ONE JSON line:
  value      whole-layer TFLOP/s with the grouped-GEMM numerator 18*N*H*F (N = T*k routed rows)
  roofline   the grouped GEMM launches, timed with HIP events inside the timed steps
  permute    achieved GB/s of the permute / unpermute row kernels (HBM roofline)
  cpu_baseline  the oracle (CPU restatement of the reference's torch-native path) timed on this
             box's host cores on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_PEAK = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}  # dense TFLOP/s, MI355X
HBM_PEAK_GBPS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="mixtral",
                    help="mixtral (default, the configuration the metric is quoted on), tiny, "
                         "finegrained, mixtral_skew")
    ap.add_argument("--dispatcher", default="allgather", choices=["allgather", "alltoall"])
    ap.add_argument("--pre-router-norm", action="store_true",
                    help="put the RMSNorm in front of the router into the step (the layer input is "
                         "then the un-normalised residual stream, which the combine adds back)")
    ap.add_argument("--operands", default="random", choices=["random", "zeros"],
                    help="zeros: activations, gradients and expert weights all zero, routing from random "
                         "logits: the same launches without data-dependent switching power (a "
                         "diagnostic, not the benchmark)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--blas-reference", action="store_true",
                    help="also time the BLAS library (torch.matmul) on one expert's share of each of "
                         "the six GEMM shapes, after the timed steps; adds 'blas_reference'")
    ap.add_argument("--cpu-tokens", type=int, default=2048,
                    help="tokens of the bounded CPU sample (same H, F, E, top-k)")
    return ap.parse_args()


class KernelTimer:
    """Wraps the package's launch wrappers with HIP event pairs on the launch stream."""

    def __init__(self, torch, ops):
        self.torch = torch
        self.ops = ops
        self.records = []  # (name, start_event, end_event, work)
        self.enabled = False
        self._orig = {}

    def _wrap(self, name, label_fn):
        orig = getattr(self.ops, name)
        self._orig[name] = orig
        torch = self.torch

        def wrapped(*a, **kw):
            if not self.enabled:
                return orig(*a, **kw)
            s = torch.cuda.Event(enable_timing=True)
            e = torch.cuda.Event(enable_timing=True)
            s.record()
            out = orig(*a, **kw)
            e.record()
            self.records.append((label_fn(*a, **kw), s, e))
            return out

        setattr(self.ops, name, wrapped)

    def install(self):
        def gmm_label(a, b, off, trans_a=False, trans_b=False, out_dtype=None):
            N, K = a.shape
            if trans_a:
                M, mode = b.shape[1], "TN"
            else:
                M, mode = (b.shape[1], "NT") if trans_b else (b.shape[2], "NN")
            return ("gmm_%s" % mode, 2.0 * N * K * M, (N, K, M))

        self._wrap("gmm", gmm_label)

        def glu_fwd_label(a, w1, off, act="silu"):
            N, K = a.shape
            return ("gmm_NN+glu", 2.0 * N * K * w1.shape[2], (N, K, w1.shape[2]))

        def glu_bwd_label(go, w2, fc1, off, act="silu"):
            N, K = go.shape
            return ("gmm_NT+glu_bwd", 2.0 * N * K * w2.shape[1], (N, K, w2.shape[1]))

        self._wrap("gmm_glu", glu_fwd_label)
        self._wrap("gmm_glu_bwd", glu_bwd_label)
        for nm in ("permute_rows", "unpermute_rows", "unpermute_rows_bwd", "glu_fwd", "glu_bwd",
                   "permute_plan", "route_topk", "route_topk_bwd", "rmsnorm_fwd", "rmsnorm_bwd", "gate_fwd",
                   "gate_bwd"):
            self._wrap(nm, (lambda n: (lambda *a, **kw: (n, 0.0, None)))(nm))

    def uninstall(self):
        for k, v in self._orig.items():
            setattr(self.ops, k, v)

    def summary(self):
        agg = {}
        for (name, work, shape), s, e in self.records:
            key = name if shape is None else "%s %s" % (name, "x".join(map(str, shape)))
            d = agg.setdefault(key, {"name": name, "ms": 0.0, "calls": 0, "work": work})
            d["ms"] += s.elapsed_time(e)
            d["calls"] += 1
        return agg


def blas_reference(torch, w, dev, reps=10, zeros=False):
    """The vendor BLAS library on one expert's share (N/E rows) of the layer's six GEMMs, same dtype,
    same kind of data: a yardstick for what this chip sustains on these shapes, not part of `value`."""
    n = w.routed_rows // w.experts
    H, F = w.hidden, w.ffn
    g = torch.Generator(device=dev).manual_seed(7)

    def rnd(*shape, scale=1.0):
        if zeros:
            return torch.zeros(*shape, device=dev, dtype=w.dtype)
        return (scale * torch.randn(*shape, generator=g, device=dev, dtype=torch.float32)).to(w.dtype)

    x, fc1, act, dy = rnd(n, H), rnd(n, 2 * F), rnd(n, F), rnd(n, H)
    w1, w2 = rnd(H, 2 * F, scale=0.02), rnd(F, H, scale=0.02)
    cases = {
        "NN fc1 %dx%dx%d" % (n, H, 2 * F): (lambda: torch.matmul(x, w1), 2.0 * n * H * 2 * F),
        "NN fc2 %dx%dx%d" % (n, F, H): (lambda: torch.matmul(act, w2), 2.0 * n * F * H),
        "NT dx %dx%dx%d" % (n, 2 * F, H): (lambda: torch.matmul(fc1, w1.t()), 2.0 * n * H * 2 * F),
        "NT dact %dx%dx%d" % (n, H, F): (lambda: torch.matmul(dy, w2.t()), 2.0 * n * F * H),
        "TN dW1 %dx%dx%d" % (n, H, 2 * F): (lambda: torch.matmul(x.t(), fc1), 2.0 * n * H * 2 * F),
        "TN dW2 %dx%dx%d" % (n, F, H): (lambda: torch.matmul(act.t(), dy), 2.0 * n * F * H),
    }
    out = {}
    for name, (fn, flops) in cases.items():
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e) / reps
        out[name] = {"avg_ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1)}
    return out


def cpu_baseline(w, tokens, dispatcher):
    """Oracle forward+backward of the layer on the host, `tokens` tokens of workload `w`."""
    import torch
    from oracle import moe_oracle as orc
    import __graft_entry__ as entry

    pkg = entry.load_package()
    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env:
        cores = min(cores, int(env))
    torch.set_num_threads(cores)
    ws = pkg.configs.scaled(w, tokens=tokens)
    inp = pkg.configs.make_inputs(ws, seed=1234)
    x = inp["x"].float().requires_grad_(True)
    w_r = inp["w_r"].float().requires_grad_(True)
    w1 = inp["w1"].requires_grad_(True)  # kept in the storage dtype; the oracle computes in fp32
    w2 = inp["w2"].requires_grad_(True)
    dy = inp["dy"].float()
    t0 = time.perf_counter()
    out, aux, info = orc.moe_layer(x, w_r, w1, w2, ws.topk, dispatcher=dispatcher)
    out.backward(dy)
    dt = time.perf_counter() - t0
    flops = ws.gemm_flops()
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "seconds": dt,
        "sample": "oracle (torch CPU, fp32 math) layer fwd+bwd on T=%d of %d tokens, same H=%d F=%d "
                  "E=%d top-%d; 1 repetition" % (tokens, w.tokens, w.hidden, w.ffn, w.experts, w.topk),
    }


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU's share of the MoE layer; this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__ as entry

    entry.ensure_built()
    pkg = entry.load_package()
    configs = pkg.configs
    w = configs.WORKLOADS[args.workload]
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---- inputs resident in HBM: seeded, generated on the device for speed ---------------------
    g = torch.Generator(device=dev).manual_seed(1234)
    S = w.tokens // w.batch
    E, H, F = w.experts, w.hidden, w.ffn
    x = torch.randn(S, w.batch, H, generator=g, device=dev, dtype=torch.float32).to(w.dtype)
    dy = torch.randn(S, w.batch, H, generator=g, device=dev, dtype=torch.float32).to(w.dtype)
    cfg = pkg.MoEConfig(hidden_size=H, num_moe_experts=E, moe_ffn_hidden_size=F,
                        moe_router_topk=w.topk, moe_router_load_balancing_type="aux_loss",
                        moe_aux_loss_coeff=0.01, moe_token_dispatcher_type=args.dispatcher,
                        params_dtype=w.dtype, moe_shared_expert_intermediate_size=w.shared_ffn)
    torch.manual_seed(1234)
    router = pkg.GalvatronMoERouter(cfg, device=dev).train()
    mlp = pkg.GalvatronMoEMLP(cfg, device=dev).train()
    logit_bias = None
    if w.zipf:
        logit_bias = configs.make_inputs(w, with_weights=False)["logit_bias"].to(dev).to(w.dtype)
    fixed_logits = None
    if args.operands == "zeros":
        fixed_logits = torch.randn(w.tokens, E, generator=g, device=dev, dtype=torch.float32).to(w.dtype)
        with torch.no_grad():
            x.zero_()
            dy.zero_()
            for prm in mlp.parameters():
                prm.zero_()
    params = list(router.parameters()) + list(mlp.parameters())
    pre_norm = None
    if args.pre_router_norm:
        pre_norm = pkg.PreRouterNorm(cfg, device=dev).train()
        params += list(pre_norm.parameters())
    x.requires_grad_(True)

    def step():
        for p in params:
            p.grad = None
        x.grad = None
        h, residual = (x, None) if pre_norm is None else pre_norm(x)
        if fixed_logits is not None:
            probs, rmap, _ = pkg.topk_softmax_with_capacity(fixed_logits + 0 * router.router.gating(h).view(-1, E),
                                                            w.topk)
        elif logit_bias is None:
            probs, rmap = router(h)
        else:
            logits = router.router.gating(h).view(-1, E) + logit_bias
            probs, rmap, _ = pkg.topk_softmax_with_capacity(logits, w.topk)
        out = mlp(h, residual, probs, rmap)
        out.backward(dy)
        return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    timer = KernelTimer(torch, pkg.ops)
    timer.install()
    timer.enabled = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timer.enabled = False
    timer.uninstall()

    # One plain device copy of known size (1 GiB read + 1 GiB written), outside the timed region:
    # the reference point for scaling FETCH_SIZE / WRITE_SIZE counters of a profiled run.
    calib = torch.empty(1 << 28, dtype=torch.float32, device=dev)
    calib_dst = torch.empty_like(calib)
    calib_dst.copy_(calib)
    torch.cuda.synchronize()
    del calib, calib_dst

    ms_per_step = dt * 1e3 / args.steps
    flops = w.gemm_flops()
    value = flops / (dt / args.steps) / 1e12
    dkey = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[w.dtype]
    peak = MFMA_PEAK[dkey]

    agg = timer.summary()
    gemm = {k: v for k, v in agg.items() if v["name"].startswith("gmm_")}
    gemm_ms = sum(v["ms"] for v in gemm.values()) / args.steps
    gemm_flops = sum(v["work"] * v["calls"] for v in gemm.values()) / args.steps
    kernels = {}
    for k, v in sorted(agg.items()):
        avg = v["ms"] / v["calls"]
        ent = {"calls_per_step": v["calls"] / args.steps, "avg_ms": round(avg, 4)}
        if v["work"]:
            ent["tflops"] = round(v["work"] / (avg * 1e-3) / 1e12, 1)
        kernels[k] = ent
    # dominant kernel: the forward fc1 grouped GEMM (NN), the largest single launch
    # HBM-side bytes per launch of that kernel from rocprofv3 counters (FETCH_SIZE x 2.0 + WRITE_SIZE
    # x 1.0, the factors a 1 GiB device copy reads back); measured once per workload with the
    # commands kept in profiles/bench_mixtral_hbm_traffic.md, not in this run.
    measured_traffic = {("mixtral", "gmm_NN+glu 32768x4096x28672"): 21.2e9}
    dom_key = max(gemm, key=lambda k: gemm[k]["work"] * (1 if k.startswith("gmm_NN") else 0.5)) if gemm else None
    roofline = None
    if dom_key:
        d = gemm[dom_key]
        ach = d["work"] / (d["ms"] / d["calls"] * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": "gmm_kernel " + dom_key, "achieved": round(ach, 1),
                    "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4),
                    "traffic": measured_traffic.get((w.name, dom_key)),
                    "all_gmm_launches": {"achieved": round(gemm_flops / (gemm_ms * 1e-3) / 1e12, 1),
                                         "frac": round(gemm_flops / (gemm_ms * 1e-3) / 1e12 / peak, 4),
                                         "ms_per_step": round(gemm_ms, 3)}}

    def hbm(name, nbytes):
        v = agg.get(name)
        if not v:
            return None
        avg = v["ms"] / v["calls"]
        gbps = nbytes / (avg * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": name, "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "avg_ms": round(avg, 4),
                "bytes": nbytes}

    permute = {"permute_rows": hbm("permute_rows", w.permute_bytes()),
               "unpermute_rows": hbm("unpermute_rows", w.unpermute_bytes())}
    if pre_norm is not None:
        row_bytes = w.tokens * H * torch.finfo(w.dtype).bits // 8
        # two launches per step share the label: the combine, which now also reads the residual,
        # and the backward of the permute
        permute["unpermute_rows"] = hbm("unpermute_rows", w.unpermute_bytes() + row_bytes / 2)
        permute["rmsnorm_fwd"] = hbm("rmsnorm_fwd", 2 * row_bytes)   # x read, y written
        # dy, x and the residual branch's gradient read, dx written
        permute["rmsnorm_bwd"] = hbm("rmsnorm_bwd", 4 * row_bytes)

    result = {
        "metric": "MoE layer fwd+bwd TFLOP/s (1 GPU, % MFMA peak); permute GB/s (% HBM)",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dkey,
        "data": "synthetic" if args.operands == "random" else "synthetic, all-zero operands (diagnostic)",
        "config": {"workload": "%s: MoE layer fwd+bwd, T=%d (batch %d) H=%d F=%d E=%d top-%d, %s "
                               "dispatcher, aux-loss router" % (w.name, w.tokens, w.batch, H, F, E,
                                                                w.topk, args.dispatcher) +
                               (", pre-router RMSNorm and residual add included" if pre_norm else ""),
                   "flops_per_step": flops},
        "pct_mfma_peak": round(100 * value / peak, 2),
        "roofline": roofline,
        "permute": permute,
        "kernels": kernels,
    }
    if args.blas_reference:
        result["blas_reference"] = blas_reference(torch, w, dev, zeros=args.operands == "zeros")
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, min(args.cpu_tokens, w.tokens), args.dispatcher)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
