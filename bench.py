"""Headline benchmark: Mixtral-shape bf16 MoE MLP forward+backward on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c1] [--no-cpu]

One step = routing prep + GLUMLP forward + backward (dX, d gates, dW1, dW2) on synthetic inputs that
are resident in HBM before the timed region.  Prints ONE JSON line.  The CPU figure next to it is the
naive per-expert PyTorch path (the oracle) timed on the host cores on a reduced token count.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
os.environ.setdefault("SCATTERMOE_NO_HF_PATCH", "1")

PEAK_BF16_TFLOPS = 2500.0        # MI355X dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0

# HBM bytes moved per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (KiB per dispatch, scaled by a copy kernel of known size); None until measured for a workload.
# c2: average over the two products of the dominant kernel in a step (layer-1 forward with the gated linear unit
# in its epilogue 21.33 GB, layer-2 forward 7.49 GB; see profiles/s2s_mfma_c2_l1fwd_counters.md for the commands
# and raw counter values).
MEASURED_TRAFFIC = {"c2": 14.41e9}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-tokens", type=int, default=0, help="token count of the CPU sample (default T/16)")
    ap.add_argument("--decode", type=int, default=0, metavar="T",
                    help="forward-only latency of one layer at T tokens (decode regime of the workload's expert "
                         "shape); prints its own JSON line with an HBM roofline")
    ap.add_argument("--profile-kernel", default="",
                    help="run ONLY one kernel of the workload `steps` times (for rocprofv3 --pmc): "
                         "l1fwd | l2fwd | l1dx | l2dx | l1dw | l2dw | copy (a 256 MiB device copy of known size)")
    return ap.parse_args()


class TimedBackend:
    """Wraps the launch layer and brackets every scatter2scatter launch with events on the launch stream."""

    def __init__(self, inner, torch):
        self.inner, self.torch, self.records, self.on = inner, torch, [], False

    def __getattr__(self, name):
        return getattr(self.inner, name)

    def s2s(self, X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped):
        if not self.on:
            return self.inner.s2s(X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped)
        a, c = self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)
        a.record()
        self.inner.s2s(X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped)
        c.record()
        self.records.append((a, c, 2.0 * eid.numel() * X.size(1) * Y.size(1), W.stride(1) == 1))

    def _timed(self, fn, flops, k_contig):
        if not self.on:
            return fn()
        a, c = self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)
        a.record()
        ok = fn()
        c.record()
        if ok:
            self.records.append((a, c, flops, k_contig))
        return ok

    # the fused GEMM + gated-linear-unit launches are launches of the same kernel (scatter2scatter FLOPs only)
    def s2s_glu(self, X, W, b, pre, h, eid, idx, off, k, x_grouped, act):
        return self._timed(lambda: self.inner.s2s_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, act),
                           2.0 * eid.numel() * X.size(1) * W.size(2), W.stride(1) == 1)

    def s2s_glu_bwd(self, DY, W, pre, dpre, eid, idx, off, act):
        return self._timed(lambda: self.inner.s2s_glu_bwd(DY, W, pre, dpre, eid, idx, off, act),
                           2.0 * eid.numel() * DY.size(1) * W.size(2), W.stride(1) == 1)


def cpu_baseline(cfg, tokens, torch):
    """Naive per-expert PyTorch path (oracle), fp32, forward + autograd backward, on `tokens` tokens."""
    import oracle
    from _inputs import make_inputs, scaled
    small = scaled(cfg, T=tokens)
    n1 = (2 if cfg.glu else 1) * cfg.f
    t = make_inputs(small, weights=False)
    g = torch.Generator().manual_seed(1)
    W1 = torch.empty(cfg.E, n1, cfg.d).normal_(0, 0.02, generator=g).requires_grad_()
    W2 = torch.empty(cfg.E, cfg.d, cfg.f).normal_(0, 0.02, generator=g).requires_grad_()
    b1 = b2 = None
    if cfg.bias:
        b1 = torch.zeros(cfg.E, n1).requires_grad_()
        b2 = torch.zeros(cfg.E, cfg.d).requires_grad_()
    act = torch.nn.SiLU() if cfg.glu else torch.nn.GELU()
    hidden = oracle.glu(act) if cfg.glu else act
    x = t["x"].requires_grad_()
    p = t["p"].requires_grad_()
    t0 = time.perf_counter()
    y = oracle.naive_expert_forward(x, p, t["experts"], W1, W2, hidden, b1, b2)
    y.backward(t["dy"])
    dt = time.perf_counter() - t0
    return {"value": tokens / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%s at T=%d of %d tokens (same d, f, E, k), fp32, 1 forward+backward, %.1f s; host has %d cpus"
                      % (cfg.name, tokens, cfg.T, dt, os.cpu_count())}


def profile_one_kernel(args, cfg, torch, ops):
    """Launch one kernel of the workload `steps` times on synthetic operands (no timing, no JSON)."""
    import scattermoe_amd as sm
    dev, dt = "cuda:0", cfg.dtype
    L, d, f, E, k = cfg.T * cfg.k, cfg.d, cfg.f, cfg.E, cfg.k
    n1 = (2 if cfg.glu else 1) * f
    g = torch.Generator(device=dev).manual_seed(0)
    experts = torch.topk(torch.randn(cfg.T, E, generator=g, device=dev), k).indices
    eid, idx, off = sm.flatten_sort_count(experts, E)
    r = lambda *shape: torch.randn(*shape, generator=g, device=dev).to(dt)
    which = args.profile_kernel
    if which == "l1fwd":
        X, W = r(cfg.T, d), r(E, n1, d) * 0.02
        if cfg.glu:   # what GLUMLP launches: layer 1 with the gated linear unit in its epilogue
            fn = lambda: ops.scatter2scatter_glu(X, W.permute(0, 2, 1), eid, idx, k, expert_offsets=off)
        else:
            fn = lambda: ops.scatter2scatter(X, W.permute(0, 2, 1), eid, idx, k, y_grouped=True, expert_offsets=off)
    elif which == "l2fwd":
        H, W = r(L, f), r(E, d, f) * 0.02
        fn = lambda: ops.scatter2scatter(H, W.permute(0, 2, 1), eid, idx, 1, x_grouped=True, expert_offsets=off)
    elif which == "l1dx":
        G, W = r(L, n1), r(E, n1, d) * 0.02
        fn = lambda: ops.scatter2scatter(G, W, eid, idx, 1, x_grouped=True, expert_offsets=off)
    elif which == "l2dx":
        G, W = r(L, d), r(E, d, f) * 0.02
        if cfg.glu:   # layer-2 input gradient with the gradient of the gated linear unit in its epilogue
            P = r(L, n1)
            fn = lambda: ops.scatter2scatter_glu_bwd(G, W, P, eid, idx, expert_offsets=off)
        else:
            fn = lambda: ops.scatter2scatter(G, W, eid, idx, 1, x_grouped=True, y_grouped=True, expert_offsets=off)
    elif which == "l1dw":
        G, X = r(L, n1), r(L, d)
        fn = lambda: ops.group_bwd_W(G, X, off, E)
    elif which == "l2dw":
        G, H = r(L, d), r(L, f)
        fn = lambda: ops.group_bwd_W(G, H, off, E)
    elif which == "copy":
        A = torch.empty(1 << 28, device=dev, dtype=torch.uint8)
        B = torch.empty_like(A)
        fn = lambda: B.copy_(A)
    else:
        raise SystemExit("unknown --profile-kernel " + which)
    for _ in range(max(1, args.steps)):
        fn()
    torch.cuda.synchronize()


def decode_line(args, cfg, torch):
    """One MoE layer forward at `--decode T` tokens under no_grad: a stream over the weights of the experts hit."""
    from torch import nn
    from scattermoe_amd.mlp import GLUMLP, MLP
    dev, dt, T = torch.device("cuda:0"), cfg.dtype, args.decode
    g = torch.Generator(device=dev).manual_seed(T)
    p, experts = torch.topk(torch.softmax(torch.randn(T, cfg.E, generator=g, device=dev), -1), cfg.k)
    p = (p / p.sum(-1, keepdim=True)).to(dt)
    x = torch.randn(T, cfg.d, generator=g, device=dev).to(dt)
    cls = GLUMLP if cfg.glu else MLP
    with torch.device(dev):
        m = cls(cfg.d, cfg.f, cfg.E, cfg.k, bias=cfg.bias, activation=nn.SiLU() if cfg.glu else nn.GELU()).to(dt)
    hit = int(experts.unique().numel())
    with torch.no_grad():
        for _ in range(args.warmup):
            m(x, p, experts)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            m(x, p, experts)
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    w_bytes = hit * (3 if cfg.glu else 2) * cfg.d * cfg.f * x.element_size()
    gbs = w_bytes / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "moe_mlp_decode_layer_ms", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False, "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[dt], "data": "synthetic",
        "config": {"workload": "%s expert shape, forward only, T=%d tokens (d_model=%d d_ff=%d E=%d top_k=%d)" % (
            cfg.name, T, cfg.d, cfg.f, cfg.E, cfg.k), "tokens": T, "experts_hit": hit},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(gbs / 8000.0, 4), "traffic": None,
                     "bytes": "weights of the experts hit: %d x %d matrices of d_model x d_ff" % (
                         hit, 3 if cfg.glu else 2)}}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU; --gpus %d is not supported "
              "(no collective or multi-GPU code exists in this path)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from torch import nn
    from _inputs import CONFIGS
    from scattermoe_amd import _C
    from scattermoe_amd.kernels import ops
    from scattermoe_amd.mlp import GLUMLP, MLP

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    assert os.path.exists(_C.lib_path()), "libscattermoe_amd.so missing: run __graft_entry__.build()"
    _C.load()
    cfg = CONFIGS[args.workload]
    dev = torch.device("cuda:0")
    dtype = cfg.dtype
    if args.profile_kernel:
        profile_one_kernel(args, cfg, torch, ops)
        return
    if args.decode:
        decode_line(args, cfg, torch)
        return

    # synthetic inputs, generated on the device with a fixed seed; resident before timing starts
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.randn(cfg.T, cfg.E, generator=g, device=dev)
    if cfg.zipf_beta:
        logits = logits - cfg.zipf_beta * 1.2 * torch.log(torch.arange(1, cfg.E + 1, device=dev).float())
    p, experts = torch.topk(torch.softmax(logits, -1), cfg.k)
    p = (p / p.sum(-1, keepdim=True)).to(dtype).requires_grad_()
    x = torch.randn(cfg.T, cfg.d, generator=g, device=dev).to(dtype).requires_grad_()
    dy = torch.randn(cfg.T, cfg.d, generator=g, device=dev).to(dtype)
    cls = GLUMLP if cfg.glu else MLP
    with torch.device(dev):
        m = cls(cfg.d, cfg.f, cfg.E, cfg.k, bias=cfg.bias, activation=nn.SiLU() if cfg.glu else nn.GELU()).to(dtype)
    if cfg.bias:
        nn.init.normal_(m.experts.bias, std=0.02)
        nn.init.normal_(m.output_experts.bias, std=0.02)
    leaves = [x, p] + list(m.parameters())

    timed = TimedBackend(ops._backend, torch)
    ops._backend = timed

    def step():
        for t in leaves:
            t.grad = None
        y = m(x, p, experts)
        y.backward(dy)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timed.on = True
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed.on = False

    L = cfg.T * cfg.k
    flops_step = (18.0 if cfg.glu else 12.0) * L * cfg.d * cfg.f
    ms = dt / args.steps * 1e3
    tflops = flops_step / (ms * 1e-3) / 1e12

    # dominant kernel: the MFMA scatter2scatter (forward flavour: weights with contiguous contraction axis)
    fwd = [(a.elapsed_time(c), fl) for a, c, fl, kc in timed.records if kc]
    allk = [(a.elapsed_time(c), fl) for a, c, fl, kc in timed.records]
    sel = fwd if fwd else allk
    k_ms = sum(t for t, _ in sel) / len(sel)
    k_fl = sum(fl for _, fl in sel) / len(sel)
    achieved = k_fl / (k_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": MEASURED_TRAFFIC.get(cfg.name),
                "kernel": "s2s_mfma_kernel (scatter2scatter products with K-contiguous weights; a product of a few "
                          "rounds of tiles plus a remainder runs as two launches and is timed as one)",
                "launches_per_step": len(sel) // args.steps, "avg_launch_ms": round(k_ms, 4),
                "avg_flop_per_launch": k_fl,
                "all_s2s_launches_avg_tflops": round(sum(fl for _, fl in allk) / sum(t for t, _ in allk) / 1e9, 1)}

    out = {
        "metric": "moe_mlp_fwd_bwd_tokens_per_s", "value": round(cfg.T * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[dtype], "data": "synthetic",
        "config": {"workload": "%s: MoE MLP fwd+bwd T=%d d_model=%d d_ff=%d E=%d top_k=%d %s%s" % (
            cfg.name, cfg.T, cfg.d, cfg.f, cfg.E, cfg.k, "SwiGLU" if cfg.glu else "GELU", " +bias" if cfg.bias else ""),
            "tokens": cfg.T, "rows": L},
        "tflops": round(tflops, 1), "frac_of_bf16_mfma_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "roofline": roofline,
    }
    if not args.no_cpu:
        tokens = args.cpu_tokens or max(64, cfg.T // 16)
        out["cpu_baseline"] = cpu_baseline(cfg, tokens, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
