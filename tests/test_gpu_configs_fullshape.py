"""Every benchmark configuration at its REAL shape, forward and backward, against the CPU oracle.

The oracle cannot run a whole c2 / c3 / c4 step in seconds, but two exact reductions of the problem can:

* tokens: the output row, the input gradient and the gate gradients of token t depend on nothing but token t, so
  `oracle.naive_token_forward` (the reference test's literal per-token form) + autograd on a sample of tokens
  gives Y[t], dX[t] and dgates[t] of the full problem;
* hidden units: the gradients of the layer-1 weight rows {n, f+n}, of the layer-2 weight column n and of the
  layer-1 bias entries of a hidden unit n depend on the other hidden units only through dY, which is given.
  `oracle.naive_expert_forward` + autograd on the model cut down to a sample S of hidden units (all tokens, all
  experts) therefore gives dW1[:, S u (f+S), :], dW2[:, :, S], db1[:, S u (f+S)] and db2 of the full problem.

Routing, tokens and dY come from `_inputs.make_inputs` (CPU generator, seed 0, the draw order of the benchmark
definition); the weights of these shapes are drawn on the device (seed 1) because drawing up to 5.6e9 normal
numbers on the host takes longer than everything else in this file together.
Bars: `_tol.check` (bf16 rel 2e-2 / abs 1e-2, absolute term scaled by the reference magnitude when that exceeds 1)
against the float32 oracle, and the literal bar (nothing scaled) against the oracle that rounds to the storage type
wherever the path stores a tensor (`oracle.rounded_glu_token_step`, `oracle.rounded_glu_hidden_unit_grads`): the
first bounds format error + kernel error, the second kernel error alone.
"""
import pytest
import torch
from torch import nn

import oracle
from _inputs import CONFIGS, make_inputs, make_module
from _tol import check
from scattermoe_amd.parallel_experts import flatten_sort_count

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF = torch.bfloat16


def _module(cfg):
    return make_module(cfg, DEV)


def _step(cfg):
    t = make_inputs(cfg, weights=False)
    m = _module(cfg)
    x = t["x"].to(cfg.dtype).to(DEV).requires_grad_()
    p = t["p"].to(cfg.dtype).to(DEV).requires_grad_()
    experts = t["experts"].to(DEV)
    y = m(x, p, experts)
    y.backward(t["dy"].to(cfg.dtype).to(DEV))
    torch.cuda.synchronize()
    return t, m, x, p, y


def _check_tokens(cfg, t, m, x, p, y, n_tokens, seed):
    """Y, dX, dgates of sampled tokens through the literal per-token form."""
    g = torch.Generator().manual_seed(seed)
    toks = torch.randperm(cfg.T, generator=g)[:n_tokens]
    W1, W2 = m.experts.weight.detach().float().cpu(), m.output_experts.weight.detach().float().cpu()
    b1 = m.experts.bias.detach().float().cpu() if cfg.bias else None
    b2 = m.output_experts.bias.detach().float().cpu() if cfg.bias else None
    xs = x.detach()[toks.to(DEV)].float().cpu().requires_grad_()
    ps = p.detach()[toks.to(DEV)].float().cpu().requires_grad_()
    dys = t["dy"][toks].to(cfg.dtype).float()
    want = oracle.naive_token_forward(xs, ps, t["experts"][toks], W1, W2, oracle.glu(nn.SiLU()), b1, b2)
    want.backward(dys)
    check("%s Y (sampled tokens)" % cfg.name, y.detach()[toks.to(DEV)], want, cfg.dtype)
    check("%s dX (sampled tokens)" % cfg.name, x.grad[toks.to(DEV)], xs.grad, cfg.dtype)
    check("%s dgates (sampled tokens)" % cfg.name, p.grad[toks.to(DEV)], ps.grad, cfg.dtype)
    # the same step with every tensor the path stores rounded to the storage type: what is left to differ is the
    # order of the float32 sums, so the bar is the literal one (abs 1e-2, rel 2e-2, nothing scaled)
    ry, rdx, rdp = oracle.rounded_glu_token_step(xs.detach(), ps.detach(), t["experts"][toks], W1, W2, dys, cfg.dtype, b1, b2)
    check("%s Y vs rounded oracle" % cfg.name, y.detach()[toks.to(DEV)], ry, cfg.dtype, literal=True)
    check("%s dX vs rounded oracle" % cfg.name, x.grad[toks.to(DEV)], rdx, cfg.dtype, literal=True)
    check("%s dgates vs rounded oracle" % cfg.name, p.grad[toks.to(DEV)], rdp, cfg.dtype, literal=True)


def _check_hidden_units(cfg, t, m, x, p, n_units, seed):
    """dW1, dW2, db1, db2 restricted to sampled hidden units, all experts, through the per-expert form."""
    g = torch.Generator().manual_seed(seed)
    S = torch.sort(torch.randperm(cfg.f, generator=g)[:n_units]).values
    S2 = torch.cat([S, cfg.f + S])
    W1 = m.experts.weight.detach()[:, S2.to(DEV)].float().cpu().requires_grad_()              # (E, 2|S|, d)
    W2 = m.output_experts.weight.detach()[:, :, S.to(DEV)].float().cpu().requires_grad_()     # (E, d, |S|)
    b1 = b2 = None
    if cfg.bias:
        b1 = m.experts.bias.detach()[:, S2.to(DEV)].float().cpu().requires_grad_()
        b2 = m.output_experts.bias.detach().float().cpu().requires_grad_()
    xc, pc = x.detach().float().cpu(), p.detach().float().cpu()
    want = oracle.naive_expert_forward(xc, pc, t["experts"], W1, W2, oracle.glu(nn.SiLU()), b1, b2)
    want.backward(t["dy"].to(cfg.dtype).float())
    check("%s dW1 (sampled hidden units)" % cfg.name, m.experts.weight.grad[:, S2.to(DEV)], W1.grad, cfg.dtype)
    check("%s dW2 (sampled hidden units)" % cfg.name, m.output_experts.weight.grad[:, :, S.to(DEV)], W2.grad, cfg.dtype)
    if cfg.bias:
        check("%s db1 (sampled hidden units)" % cfg.name, m.experts.bias.grad[:, S2.to(DEV)], b1.grad, cfg.dtype)
        check("%s db2" % cfg.name, m.output_experts.bias.grad, b2.grad, cfg.dtype)
    r1, r2, rb1, rb2 = oracle.rounded_glu_hidden_unit_grads(
        xc, pc, t["experts"], W1.detach(), W2.detach(), t["dy"].to(cfg.dtype).float(), cfg.dtype,
        b1.detach() if cfg.bias else None, with_b2=cfg.bias)
    check("%s dW1 vs rounded oracle" % cfg.name, m.experts.weight.grad[:, S2.to(DEV)], r1, cfg.dtype, literal=True)
    check("%s dW2 vs rounded oracle" % cfg.name, m.output_experts.weight.grad[:, :, S.to(DEV)], r2, cfg.dtype, literal=True)
    if cfg.bias:
        check("%s db1 vs rounded oracle" % cfg.name, m.experts.bias.grad[:, S2.to(DEV)], rb1, cfg.dtype, literal=True)
        check("%s db2 vs rounded oracle" % cfg.name, m.output_experts.bias.grad, rb2, cfg.dtype, literal=True)


def _check_routing(cfg, t):
    eid, idx, off = flatten_sort_count(t["experts"].to(DEV), cfg.E)
    e, i, o = oracle.route_ref(t["experts"], cfg.E)
    assert torch.equal(eid.cpu(), e) and torch.equal(idx.cpu(), i) and torch.equal(off.cpu(), o)
    return torch.diff(o, prepend=o.new_zeros(1))


def test_c2_full_backward():
    """Mixtral shape: the step the benchmark times (fused layer-1 + gated unit, fused layer-2 input gradient +
    gated-unit gradient, both weight gradients, the input gradient with its sum over the two slots)."""
    cfg = CONFIGS["c2"]
    t, m, x, p, y = _step(cfg)
    counts = _check_routing(cfg, t)
    assert int(counts.min()) > 3500 and int(counts.max()) < 4700          # near-uniform load
    _check_tokens(cfg, t, m, x, p, y, n_tokens=24, seed=11)
    _check_hidden_units(cfg, t, m, x, p, n_units=12, seed=12)


def test_c3_real_shape_forward_then_forward_backward():
    """gpt-oss-20b shape: d = f = 2880 (45 x 64: partial tiles in both directions), 5760 output columns with bias,
    Zipf-skewed load with an empty expert and experts of fewer than 16 rows."""
    cfg = CONFIGS["c3"]
    t = make_inputs(cfg, weights=False)
    counts = _check_routing(cfg, t)
    assert int((counts == 0).sum()) >= 1 and int(((counts > 0) & (counts < 16)).sum()) >= 1 and int(counts.max()) > 4096
    # forward only (inference), the launches without the saved pre-activation
    m = _module(cfg)
    with torch.no_grad():
        y_inf = m(t["x"].to(cfg.dtype).to(DEV), t["p"].to(cfg.dtype).to(DEV), t["experts"].to(DEV))
    # forward + backward
    t, m, x, p, y = _step(cfg)
    assert torch.equal(y_inf, y.detach()), "inference and training forward differ"
    _check_tokens(cfg, t, m, x, p, y, n_tokens=48, seed=21)
    # tokens routed to the least-loaded experts: their tiles are the ragged ones
    rare = torch.nonzero((counts > 0) & (counts < 16)).flatten()
    hit = torch.isin(t["experts"], rare).any(-1).nonzero().flatten()[:16]
    if hit.numel():
        W1, W2 = m.experts.weight.detach().float().cpu(), m.output_experts.weight.detach().float().cpu()
        b1, b2 = m.experts.bias.detach().float().cpu(), m.output_experts.bias.detach().float().cpu()
        xs = x.detach()[hit.to(DEV)].float().cpu()
        want = oracle.naive_token_forward(xs, p.detach()[hit.to(DEV)].float().cpu(), t["experts"][hit], W1, W2,
                                          oracle.glu(nn.SiLU()), b1, b2)
        check("c3 Y (tokens of experts with < 16 rows)", y.detach()[hit.to(DEV)], want, cfg.dtype)
    _check_hidden_units(cfg, t, m, x, p, n_units=16, seed=22)
    empty = torch.nonzero(counts == 0).flatten().to(DEV)
    for g_ in (m.experts.weight.grad, m.output_experts.weight.grad, m.experts.bias.grad, m.output_experts.bias.grad):
        assert float(g_[empty].abs().max()) == 0.0, "an expert without rows must get an all-zero gradient"


def test_c4_real_shape_forward_backward():
    """Fine-grained shape: L = 262144 rows over 128 experts, top-8, short contractions (768 / 2048)."""
    cfg = CONFIGS["c4"]
    t, m, x, p, y = _step(cfg)
    counts = _check_routing(cfg, t)
    assert int(counts.sum()) == cfg.T * cfg.k and int(counts.min()) > 1500
    _check_tokens(cfg, t, m, x, p, y, n_tokens=32, seed=31)
    _check_hidden_units(cfg, t, m, x, p, n_units=8, seed=32)


@pytest.mark.parametrize("T", [1, 8, 64, 256])
def test_c5_decode_real_width(T):
    """Decode regime at the Mixtral width (d = 4096, f = 14336: both layers, gated unit, the 14336-long
    contraction), uniform random routing, forward only under no_grad."""
    cfg = CONFIGS["c2"]
    m = _module(cfg)
    g = torch.Generator().manual_seed(100 + T)
    experts = torch.stack([torch.randperm(cfg.E, generator=g)[:cfg.k] for _ in range(T)])
    p = torch.softmax(torch.randn(T, cfg.k, generator=g), -1).to(BF)
    x = torch.randn(T, cfg.d, generator=g).to(BF)
    with torch.no_grad():
        y = m(x.to(DEV), p.to(DEV), experts.to(DEV))
    toks = torch.arange(T) if T <= 8 else torch.randperm(T, generator=g)[:12]
    W1, W2 = m.experts.weight.detach().float().cpu(), m.output_experts.weight.detach().float().cpu()
    want = oracle.naive_token_forward(x[toks].float(), p[toks].float(), experts[toks], W1, W2, oracle.glu(nn.SiLU()))
    check("c5 Y (T=%d)" % T, y[toks.to(DEV)], want, BF)
