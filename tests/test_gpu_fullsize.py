"""Full-size checks at the Mixtral-shape workload (T=16384, d=4096, f=14336, E=8, k=2, bf16), where the CPU
oracle cannot run the whole computation in seconds: the routing triple is compared bit-exactly (it is cheap on
the CPU), the GEMM kernels are checked (a) on randomly sampled output rows / entries recomputed by the oracle in
fp32 from the same bf16 operands and (b) through size-independent properties that hold exactly in floating
point - scaling an operand by a power of two, permuting the tokens - and the whole module on sampled tokens
through the oracle's literal per-token form.  Tolerance for sampled values: rel 2e-2 / abs 1e-2 scaled by the
magnitude a dot product of that length reaches."""
import math

import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops
from scattermoe_amd.mlp import GLUMLP
from scattermoe_amd.parallel_experts import flatten_sort_count

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
T, D, F, E, K = 16384, 4096, 14336, 8, 2
BF = torch.bfloat16


@pytest.fixture(scope="module")
def big():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(T, E, generator=g)
    p, experts = torch.topk(torch.softmax(logits, -1), K)
    p = (p / p.sum(-1, keepdim=True)).to(BF)
    gd = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(T, D, generator=gd, device=DEV).to(BF)
    w1 = (torch.randn(E, 2 * F, D, generator=gd, device=DEV) * 0.02).to(BF)
    w2 = (torch.randn(E, D, F, generator=gd, device=DEV) * 0.02).to(BF)
    eid, idx, off = flatten_sort_count(experts.to(DEV), E)
    return dict(p=p.to(DEV), experts=experts.to(DEV), x=x, w1=w1, w2=w2, eid=eid, idx=idx, off=off)


def _close(got, want, klen):
    scale = math.sqrt(klen) * 0.02 * 1.0          # |x| ~ 1, |w| ~ 0.02
    err = (got.float().cpu() - want.float().cpu()).abs()
    bound = 1e-2 * scale + 2e-2 * want.float().cpu().abs()
    assert bool((err <= bound).all()), "max err %g" % float(err.max())


def test_routing_full_size_bit_exact(big):
    e, i, o = oracle.route_ref(big["experts"].cpu(), E)
    assert torch.equal(big["eid"].cpu(), e) and torch.equal(big["idx"].cpu(), i) and torch.equal(big["off"].cpu(), o)


def test_layer1_sampled_rows_and_exact_properties(big):
    x, w1, eid, idx, off = big["x"], big["w1"], big["eid"], big["idx"], big["off"]
    W = w1.permute(0, 2, 1)
    y = ops.scatter2scatter(x, W, eid, idx, K, y_grouped=True, expert_offsets=off)
    g = torch.Generator().manual_seed(2)
    for n in torch.randint(0, T * K, (48,), generator=g).tolist():
        e, src = int(eid[n]), int(idx[n]) // K
        want = x[src].float().cpu() @ w1[e].float().cpu().t()
        _close(y[n], want, D)
    # scaling the input by a power of two scales every output exactly
    y4 = ops.scatter2scatter(x * 4, W, eid, idx, K, y_grouped=True, expert_offsets=off)
    assert torch.equal(y4, y * 4)
    # the same tokens in another order: every (token, slot) row is the same dot product, bit for bit
    perm = torch.randperm(T, generator=g).to(DEV)
    eid2, idx2, off2 = flatten_sort_count(big["experts"][perm], E)
    y2 = ops.scatter2scatter(x[perm], W, eid2, idx2, K, y_grouped=False, expert_offsets=off2)   # slot order
    y_slot = torch.empty_like(y)
    y_slot[idx] = y                                                                             # grouped -> slot order
    assert torch.equal(y2.view(T, K, -1), y_slot.view(T, K, -1)[perm])


def test_layer2_and_input_gradient_sampled_rows(big):
    w2, eid, idx, off = big["w2"], big["eid"], big["idx"], big["off"]
    gd = torch.Generator(device=DEV).manual_seed(3)
    h = torch.randn(T * K, F, generator=gd, device=DEV).to(BF)
    y = ops.scatter2scatter(h, w2.permute(0, 2, 1), eid, idx, 1, x_grouped=True, y_grouped=False, expert_offsets=off)
    dy = torch.randn(T * K, D, generator=gd, device=DEV).to(BF)
    dh = ops.scatter2scatter(dy, w2, eid, idx, 1, x_grouped=True, y_grouped=True, expert_offsets=off)
    g = torch.Generator().manual_seed(4)
    for n in torch.randint(0, T * K, (32,), generator=g).tolist():
        e = int(eid[n])
        _close(y[int(idx[n])], h[n].float().cpu() @ w2[e].float().cpu().t(), F)
        _close(dh[n], dy[n].float().cpu() @ w2[e].float().cpu(), D)


def test_weight_gradient_sampled_entries_and_scaling(big):
    eid, off = big["eid"], big["off"]
    gd = torch.Generator(device=DEV).manual_seed(5)
    dy = torch.randn(T * K, D, generator=gd, device=DEV).to(BF)
    h = torch.randn(T * K, F, generator=gd, device=DEV).to(BF)
    dw, _ = ops.group_bwd_W(dy, h, off, E)                     # (E, K=F, N=D) view
    assert dw.shape == (E, F, D) and dw.permute(0, 2, 1).is_contiguous()
    offs = [0] + off.cpu().tolist()
    g = torch.Generator().manual_seed(6)
    for _ in range(64):
        e = int(torch.randint(0, E, (1,), generator=g))
        kk = int(torch.randint(0, F, (1,), generator=g))
        nn = int(torch.randint(0, D, (1,), generator=g))
        lo, hi = offs[e], offs[e + 1]
        want = (h[lo:hi, kk].float() * dy[lo:hi, nn].float()).sum().cpu()
        got = dw[e, kk, nn].float().cpu()
        rows = hi - lo
        assert abs(float(got - want)) <= 1e-2 * math.sqrt(rows) + 2e-2 * abs(float(want))
    dw2, _ = ops.group_bwd_W(dy * 2, h, off, E)
    assert torch.equal(dw2, dw * 2)


def test_module_sampled_tokens_against_per_token_oracle(big):
    with torch.device(DEV):
        m = GLUMLP(D, F, E, K).to(BF)
    with torch.no_grad():
        m.experts.weight.copy_(big["w1"])
        m.output_experts.weight.copy_(big["w2"])
        y = m(big["x"], big["p"], big["experts"])
        # doubling the gates doubles the output exactly
        assert torch.equal(m(big["x"], big["p"] * 2, big["experts"]), y * 2)
    g = torch.Generator().manual_seed(7)
    toks = torch.randint(0, T, (24,), generator=g)
    used = torch.unique(big["experts"][toks.to(DEV)]).cpu().tolist()
    w1 = {e: big["w1"][e].float().cpu() for e in used}
    w2 = {e: big["w2"][e].float().cpu() for e in used}
    for t in toks.tolist():
        xt = big["x"][t].float().cpu()
        want = torch.zeros(D)
        for j in range(K):
            e = int(big["experts"][t, j])
            pre = (w1[e] @ xt).to(BF).float()                  # the kernels store the pre-activation in bf16
            hid = (torch.nn.functional.silu(pre[F:]) * pre[:F]).to(BF).float()
            want += float(big["p"][t, j]) * (w2[e] @ hid).to(BF).float()
        err = (y[t].float().cpu() - want).abs()
        # abs 1e-2 relative to the magnitude of the output vector, rel 2e-2
        scale = max(1.0, float(want.abs().max()))
        assert bool((err <= 1e-2 * scale + 2e-2 * want.abs()).all()), "token %d max err %g" % (t, float(err.max()))


def test_grouped_input_larger_than_4_gib():
    """An expert-grouped activation matrix beyond 4 GiB (lane offsets inside the MFMA kernels are 32-bit and taken
    relative to each tile's first row): rows on both sides of the 4 GiB mark against the oracle's row products, and
    the launch must be fast enough to have been the MFMA kernel (the any-layout path takes seconds here)."""
    L, Fh, N, En = 160000, 14336, 512, 4                     # 4.59 GB of bf16 hidden rows
    gd = torch.Generator(device=DEV).manual_seed(5)
    h = torch.empty(L, Fh, device=DEV, dtype=BF).normal_(generator=gd)
    w = (torch.randn(En, N, Fh, generator=gd, device=DEV) * 0.02).to(BF)
    eid = torch.arange(L, device=DEV) * En // L              # already sorted: L / En rows per expert
    idx = torch.arange(L, device=DEV)
    off = torch.tensor([(e + 1) * L // En for e in range(En)], device=DEV)
    y = ops.scatter2scatter(h, w.permute(0, 2, 1), eid, idx, 1, x_grouped=True, y_grouped=True, expert_offsets=off)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    ops.scatter2scatter(h, w.permute(0, 2, 1), eid, idx, 1, x_grouped=True, y_grouped=True, expert_offsets=off, out=y)
    b.record()
    torch.cuda.synchronize()
    assert a.elapsed_time(b) < 60.0, "%.1f ms: not the MFMA path" % a.elapsed_time(b)     # 2.3e12 FLOP
    mark = (1 << 32) // (Fh * 2)                             # first row that starts beyond 4 GiB
    for n in [0, 39999, 40000, mark - 1, mark, mark + 1, 120000, L - 1]:
        e = int(eid[n])
        want = h[n].float().cpu() @ w[e].float().cpu().t()
        _close(y[n], want, Fh)
