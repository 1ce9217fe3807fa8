"""Headline benchmark: Mixtral-shape bf16 MoE MLP forward+backward on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c1] [--no-cpu] [--compile] [--forward-only]

One step = routing prep + GLUMLP forward + backward (dX, d gates, dW1, dW2) on synthetic inputs that
are resident in HBM before the timed region (with --forward-only: routing prep + forward under no_grad).  Prints ONE JSON line.  The CPU figure next to it is the
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



def measured_traffic(workload, source_hash):
    """HBM-side bytes per launch of the dominant kernel, from profiles/<workload>_traffic.json - the record a
    rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE session of this benchmark leaves (the record itself names the commands).
    The record names the kernel sources it was measured on; for any other sources the figure would be a guess,
    so None is returned."""
    path = os.path.join(ROOT, "profiles", "%s_traffic.json" % workload)
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, None
    if rec.get("source_hash") != source_hash:
        return None, "profiles/%s_traffic.json was measured on kernel sources %s, this library is %s" % (
            workload, rec.get("source_hash"), source_hash)
    return rec.get("bytes_per_launch"), "profiles/%s_traffic.json (%s)" % (workload, rec.get("command", ""))


def traffic_record(args):
    """HBM-side bytes per product of the dominant kernel from four rocprofv3 --pmc runs (one counter each):
    DIR/fetch, DIR/write = FETCH_SIZE / WRITE_SIZE over `bench.py --workload W --no-cpu`, DIR/fetch_copy, DIR/write_copy
    = the same counters over `bench.py --profile-kernel copy` (256 MiB read + 256 MiB written per launch), which give
    the factor from counter units to KiB.  The dominant kernel's products are the scatter2scatter launches with
    K-contiguous weights (kernel instantiations with B_TR = false); a product split over two launches counts once."""
    import csv
    import glob
    import subprocess

    def rows(sub):
        out = []
        for f in glob.glob(os.path.join(args.traffic_record, sub, "**", "*counter_collection.csv"), recursive=True):
            out += list(csv.DictReader(open(f)))
        return out

    def per_launch(sub, counter, want):
        v = [float(r["Counter_Value"]) for r in rows(sub) if r["Counter_Name"] == counter and want(r["Kernel_Name"])]
        return v

    copy_kib = 256.0 * 1024
    is_copy = lambda n: "copyBuffer" in n
    f_copy = per_launch("fetch_copy", "FETCH_SIZE", is_copy)
    w_copy = per_launch("write_copy", "WRITE_SIZE", is_copy)
    f_factor = copy_kib / (sum(f_copy) / len(f_copy))
    w_factor = copy_kib / (sum(w_copy) / len(w_copy))
    # B_TR = false instantiations of the scatter2scatter MFMA kernel, any tile class
    dominant = lambda n: "s2s_mfma_kernel" in n and ("Lb0EEEv" in n or "false>" in n)
    fetch = per_launch("fetch", "FETCH_SIZE", dominant)
    write = per_launch("write", "WRITE_SIZE", dominant)
    steps = args.steps + args.warmup
    products_per_step = 2
    n_products = steps * products_per_step
    fetch_b = sum(fetch) * f_factor * 1024 / n_products
    write_b = sum(write) * w_factor * 1024 / n_products
    sys.path.insert(0, ROOT)
    from scattermoe_amd import _build
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        commit = ""
    print(json.dumps({
        "workload": args.workload, "kernel": "s2s_mfma_kernel, products with K-contiguous weights (layer-1 and layer-2 forward)",
        "bytes_per_launch": round(fetch_b + write_b), "fetch_bytes": round(fetch_b), "write_bytes": round(write_b),
        "launches_counted": {"fetch": len(fetch), "write": len(write)}, "products": n_products,
        "factor_to_kib": {"FETCH_SIZE": round(f_factor, 4), "WRITE_SIZE": round(w_factor, 4)},
        "source_hash": _build.source_hash(), "commit": commit,
        "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -- python3 bench.py --workload %s --steps %d "
                   "--warmup %d --no-cpu; same counters over python3 bench.py --profile-kernel copy --steps 10"
                   % (args.workload, args.steps, args.warmup)}, indent=1))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--compile", action="store_true",
                    help="run the module through torch.compile(fullgraph=True): every launch is a registered operator, "
                         "so the compiled step issues the same kernels as the eager one")
    ap.add_argument("--forward-only", action="store_true",
                    help="time the forward pass alone under no_grad (inference: the pre-activation is not stored); the "
                         "metric becomes moe_mlp_fwd_tokens_per_s")
    ap.add_argument("--cpu-tokens", type=int, default=0, help="token count of the CPU sample (default T/3)")
    ap.add_argument("--decode", type=int, default=0, metavar="T",
                    help="forward-only latency of one layer at T tokens (decode regime of the workload's expert "
                         "shape); prints its own JSON line with an HBM roofline")
    ap.add_argument("--profile-kernel", default="",
                    help="run ONLY one kernel of the workload `steps` times (for rocprofv3 --pmc): "
                         "l1fwd | l2fwd | l1dx | l2dx | l1dw | l2dw | copy (a 256 MiB device copy of known size)")
    ap.add_argument("--traffic-record", default="", metavar="DIR",
                    help="no GPU work: read the rocprofv3 --pmc csv files under DIR/{fetch,write,fetch_copy,write_copy} "
                         "(FETCH_SIZE / WRITE_SIZE over a run of this benchmark and over `--profile-kernel copy`) and "
                         "print the traffic record that belongs into profiles/<workload>_traffic.json")
    return ap.parse_args()


class TimedBackend:
    """Wraps the launch layer and brackets every expert-GEMM launch (scatter2scatter, groupXtY) with events on the
    launch stream.  Records: (start, stop, algorithmic FLOP, weights K-contiguous? (None for groupXtY), product name)."""

    def __init__(self, inner, torch, cfg):
        self.inner, self.torch, self.records, self.on = inner, torch, [], False
        self.l1_dw_shape = ((2 if cfg.glu else 1) * cfg.f, cfg.d)     # (columns of dY, columns of X) of the layer-1 dW

    def __getattr__(self, name):
        return getattr(self.inner, name)

    def s2s(self, X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped):
        name = ("l1_fwd" if not x_grouped else "l2_fwd") if W.stride(1) == 1 else ("l1_dx" if not y_grouped else "l2_dx")
        return self._timed(lambda: self.inner.s2s(X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped) is None,
                           2.0 * eid.numel() * X.size(1) * Y.size(1), W.stride(1) == 1, name)

    def xty(self, DY, X, DW, Db, off, E):
        name = "l1_dw" if (DY.size(1), X.size(1)) == self.l1_dw_shape else "l2_dw"
        return self._timed(lambda: self.inner.xty(DY, X, DW, Db, off, E) is None,
                           2.0 * DY.size(0) * X.size(1) * DY.size(1), None, name)

    def xty_gathered(self, DY, X, idx, fan_out, DW, Db, off, E):
        # only the layer-1 weight gradient reads its X operand through the index vector; a declined launch
        # (False) is not recorded: the caller then runs group + xty, and that launch is
        return self._timed(lambda: self.inner.xty_gathered(DY, X, idx, fan_out, DW, Db, off, E),
                           2.0 * DY.size(0) * X.size(1) * DY.size(1), None, "l1_dw")

    def _timed(self, fn, flops, k_contig, name):
        if not self.on:
            return fn()
        a, c = self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)
        a.record()
        ok = fn()
        c.record()
        if ok:
            self.records.append((a, c, flops, k_contig, name))
        return ok

    # the fused GEMM + gated-linear-unit launches are launches of the same kernel (scatter2scatter FLOPs only)
    def s2s_glu(self, X, W, b, pre, h, eid, idx, off, k, x_grouped, act):
        return self._timed(lambda: self.inner.s2s_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, act),
                           2.0 * eid.numel() * X.size(1) * W.size(2), W.stride(1) == 1, "l1_fwd")

    def s2s_glu_bwd(self, DY, W, pre, dpre, eid, idx, off, act):
        return self._timed(lambda: self.inner.s2s_glu_bwd(DY, W, pre, dpre, eid, idx, off, act),
                           2.0 * eid.numel() * DY.size(1) * W.size(2), W.stride(1) == 1, "l2_dx")


def cpu_baseline(cfg, tokens, torch, forward_only=False):
    """Naive per-expert PyTorch path (oracle), fp32, forward + autograd backward (or the forward alone), on `tokens`
    tokens."""
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
    if forward_only:
        with torch.no_grad():
            oracle.naive_expert_forward(x, p, t["experts"], W1, W2, hidden, b1, b2)
    else:
        y = oracle.naive_expert_forward(x, p, t["experts"], W1, W2, hidden, b1, b2)
        y.backward(t["dy"])
    dt = time.perf_counter() - t0
    return {"value": tokens / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%s at T=%d of %d tokens (same d, f, E, k), fp32, 1 %s, %.1f s; host has %d cpus"
                      % (cfg.name, tokens, cfg.T, "forward" if forward_only else "forward+backward", dt, os.cpu_count())}


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


def mfma_sustained(torch):
    """What the matrix pipe sustains on its own (no memory traffic), for all-zero operands and for operands with
    random signs and mantissas: the shader clock follows the operand bits, so the nominal peak that `roofline.frac`
    is priced against is not reachable on data that is not trivial.  The kernel lives in a small library of its own
    (scattermoe_amd/csrc/bench/mfma_probe.hip), not in the product library."""
    import ctypes
    from scattermoe_amd import _build
    if not os.path.exists(_build.PROBE_LIB_PATH):
        return None
    lib = ctypes.CDLL(_build.PROBE_LIB_PATH)
    lib.smoe_bench_mfma_rate.restype = ctypes.c_int
    lib.smoe_bench_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                         ctypes.c_void_p]
    out = torch.empty(65536, dtype=torch.float32, device="cuda:0")
    flop = ctypes.c_double(0.0)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {}
    for name, kind in (("zero_operands", 0), ("random_operands", 1)):
        for iters in (2000, 16000):                  # a short launch to settle the clock, then about 15 ms
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            rc = lib.smoe_bench_mfma_rate(out.data_ptr(), iters, kind, ctypes.byref(flop), st)
            b.record()
            torch.cuda.synchronize()
            assert rc == 0, "smoe_bench_mfma_rate failed: %d" % rc
        res[name + "_tflops"] = round(flop.value / a.elapsed_time(b) / 1e9, 1)
    res["kernel"] = "independent 32x32x16 bf16 MFMAs, one wave per SIMD on every CU, operands in registers"
    return res


def main():
    args = parse()
    if args.traffic_record:
        traffic_record(args)
        return
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

    # synthetic inputs, resident in HBM before timing starts.  Router logits (hence routing and gates), X and dY are
    # drawn on the CPU (seed 0, the draw order of tests/_inputs.make_inputs: the tensors the full-shape parity tests
    # use); the weights are drawn on the device (seed 1, tests/_inputs.make_module)
    from _inputs import make_inputs, make_module
    t = make_inputs(cfg, weights=False)
    experts = t["experts"].to(dev)
    p = t["p"].to(dtype).to(dev).requires_grad_()
    x = t["x"].to(dtype).to(dev).requires_grad_()
    dy = t["dy"].to(dtype).to(dev)
    m = make_module(cfg, dev)
    leaves = [x, p] + list(m.parameters())

    timed = TimedBackend(ops._backend, torch, cfg)
    ops._backend = timed

    fwd = torch.compile(lambda x, p, e: m(x, p, e), fullgraph=True) if args.compile else m

    def step():
        if args.forward_only:
            with torch.no_grad():
                fwd(x, p, experts)
            return
        for t in leaves:
            t.grad = None
        y = fwd(x, p, experts)
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
    flops_step = (18.0 if cfg.glu else 12.0) * L * cfg.d * cfg.f          # forward + both gradients of both layers
    if args.forward_only:
        flops_step /= 3.0
    ms = dt / args.steps * 1e3
    tflops = flops_step / (ms * 1e-3) / 1e12

    # dominant kernel: the MFMA scatter2scatter (forward flavour: weights with contiguous contraction axis)
    fwd = [(a.elapsed_time(c), fl) for a, c, fl, kc, _ in timed.records if kc]
    allk = [(a.elapsed_time(c), fl) for a, c, fl, kc, _ in timed.records if kc is not None]
    sel = fwd if fwd else allk
    # every product of the step by itself: TFLOP/s over its algorithmic 2 L K N, averaged over the timed steps
    products = {}
    for a, c, fl, _, name in timed.records:
        ms_, fl_ = products.get(name, (0.0, 0.0))
        products[name] = (ms_ + a.elapsed_time(c), fl_ + fl)
    products = {n: {"ms": round(v[0] / args.steps, 4), "tflops": round(v[1] / v[0] / 1e9, 1),
                    "frac": round(v[1] / v[0] / 1e9 / PEAK_BF16_TFLOPS, 4)} for n, v in sorted(products.items())}
    k_ms = sum(t for t, _ in sel) / len(sel)
    k_fl = sum(fl for _, fl in sel) / len(sel)
    achieved = k_fl / (k_ms * 1e-3) / 1e12
    traffic, traffic_src = measured_traffic(cfg.name, _C.source_hash())
    sustained = mfma_sustained(torch)
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": traffic, "traffic_source": traffic_src,
                "kernel": "s2s_mfma_kernel (scatter2scatter products with K-contiguous weights; a product may run as "
                          "several launches - whole rounds of tiles, remainder, the experts' last tiles in contraction "
                          "parts and their sum - and is timed as one)",
                "launches_per_step": len(sel) // args.steps, "avg_launch_ms": round(k_ms, 4),
                "avg_flop_per_launch": k_fl,
                "all_s2s_launches_avg_tflops": round(sum(fl for _, fl in allk) / sum(t for t, _ in allk) / 1e9, 1)}

    out = {
        "metric": "moe_mlp_fwd_tokens_per_s" if args.forward_only else "moe_mlp_fwd_bwd_tokens_per_s", "value": round(cfg.T * args.steps / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[dtype], "data": "synthetic",
        "config": {"workload": "%s: MoE MLP %s T=%d d_model=%d d_ff=%d E=%d top_k=%d %s%s" % (
            cfg.name, "forward (inference)" if args.forward_only else "fwd+bwd", cfg.T, cfg.d, cfg.f, cfg.E, cfg.k, "SwiGLU" if cfg.glu else "GELU", " +bias" if cfg.bias else ""),
            "tokens": cfg.T, "rows": L},
        "tflops": round(tflops, 1), "frac_of_bf16_mfma_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "roofline": roofline,
        "mfma_sustained": sustained,
        "products": products,
        "inputs": "router logits, X, dY: CPU generator seed 0 (tests/_inputs.make_inputs order); weights: device "
                  "generator seed 1, N(0, 0.02) (tests/_inputs.make_module)",
        "library_sources": _C.source_hash(),
        "torch_compile": bool(args.compile),
    }
    if not args.no_cpu:
        tokens = args.cpu_tokens or max(64, cfg.T // 3)            # c2: about 12 s on 16 cores
        out["cpu_baseline"] = cpu_baseline(cfg, tokens, torch, args.forward_only)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
