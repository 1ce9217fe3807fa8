"""End-to-end GPU parity of MLP / GLUMLP forward + backward with the naive per-expert path.
The first test is the reference's own grid (tests/test_mlp.py:36-87): fp32, E = 8, odd sizes,
max-abs-diff < 1e-4 on Y, dX, dg, dW1, dW2, db1, db2."""
import pytest
import torch
from torch import nn

import oracle
from _inputs import CONFIGS, make_inputs, scaled
from scattermoe_amd.mlp import MLP, GLUMLP

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run_pair(m_cpu, x, p, experts, dy, dtype, per_token=False):
    """Run module on GPU (dtype) and oracle on CPU (fp32 master copy of the same rounded values)."""
    names = ["dX", "dg", "dW1", "dW2"] + (["db1", "db2"] if m_cpu.experts.bias is not None else [])
    m_gpu = type(m_cpu)(m_cpu.input_size, m_cpu.hidden_size, m_cpu.num_experts, m_cpu.top_k,
                        bias=m_cpu.experts.bias is not None, activation=m_cpu.activation).to(DEV).to(dtype)
    m_gpu.load_state_dict({k: v.to(dtype) for k, v in m_cpu.state_dict().items()})
    with torch.no_grad():                                    # oracle computes in fp32 on the rounded values
        for q, v in zip(m_cpu.parameters(), m_gpu.parameters()):
            q.copy_(v.float().cpu())
    xg = x.to(dtype).to(DEV).detach().clone().requires_grad_()
    pg = p.to(dtype).to(DEV).detach().clone().requires_grad_()
    params_g = [xg, pg, m_gpu.experts.weight, m_gpu.output_experts.weight]
    if m_gpu.experts.bias is not None:
        params_g += [m_gpu.experts.bias, m_gpu.output_experts.bias]
    y = m_gpu(xg, pg, experts.to(DEV))
    got = torch.autograd.grad(y, params_g, dy.to(dtype).to(DEV))

    xc = x.to(dtype).float().detach().clone().requires_grad_()
    pc = p.to(dtype).float().detach().clone().requires_grad_()
    params_c = [xc, pc, m_cpu.experts.weight, m_cpu.output_experts.weight]
    if m_cpu.experts.bias is not None:
        params_c += [m_cpu.experts.bias, m_cpu.output_experts.bias]
    y_ref = oracle.naive_module_forward(m_cpu, xc, pc, experts, per_token=per_token)
    want = torch.autograd.grad(y_ref, params_c, dy.to(dtype).float())
    return [("Y", y, y_ref)] + [(n, a, b) for n, a, b in zip(names, got, want)]


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("length", [1, 256, 512])
@pytest.mark.parametrize("x_dim,k", [(xd, k) for xd in [128, 256, 512, 600, 100] for k in [2, 3, 4]])
def test_mlp_correctness_reference_grid(length, x_dim, k, bias):
    E, h_dim = 8, (4 * x_dim) // k
    g = torch.Generator().manual_seed(length * 1000 + x_dim * 10 + k)
    weights = torch.softmax(torch.randn(length, E, generator=g), -1)
    p, experts = torch.topk(weights, k)                      # not renormalised, as in the reference test
    x = torch.randn(length, x_dim, generator=g)
    dy = torch.randn(length, x_dim, generator=g)
    torch.manual_seed(x_dim + k)
    m = MLP(x_dim, h_dim, E, k, bias=bias, activation=nn.GELU())
    if bias:
        nn.init.normal_(m.experts.bias, std=0.02)
        nn.init.normal_(m.output_experts.bias, std=0.02)
    for name, a, b in _run_pair(m, x, p, experts, dy, torch.float32, per_token=(length == 1)):
        diff = (a.detach().cpu() - b.detach()).abs().max().item()
        assert diff < 1e-4, "%s diff %g" % (name, diff)


def _rel_check(name, a, b, rtol, atol):
    a, b = a.detach().float().cpu(), b.detach().float()
    err = (a - b).abs()
    # tolerance relative to the tensor's scale: bf16 rounding acts on the value a row/column sum reaches
    bound = atol * max(1.0, b.abs().max().item()) + rtol * b.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, "%s: max err %g, rms ref %g" % (name, err.max().item(), b.pow(2).mean().sqrt().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name,T", [("c1", 256), ("c2", 512), ("c3", 1024), ("c4", 2048)])
def test_config_shapes_reduced(name, T, dtype):
    """The benchmark configurations at reduced T/d/f (same E, k, GLU/bias/skew), sized so the CPU oracle
    finishes in seconds."""
    cfg = CONFIGS[name]
    small = scaled(cfg, T=T, d=min(cfg.d, 512), f=min(cfg.f, 768))
    t = make_inputs(small)
    cls = GLUMLP if cfg.glu else MLP
    m = cls(small.d, small.f, small.E, small.k, bias=small.bias, activation=nn.SiLU() if cfg.glu else nn.GELU())
    with torch.no_grad():
        m.experts.weight.copy_(t["W1"]); m.output_experts.weight.copy_(t["W2"])
        if small.bias:
            m.experts.bias.copy_(t["b1"]); m.output_experts.bias.copy_(t["b2"])
    rtol, atol = (1e-4, 1e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    for n, a, b in _run_pair(m, t["x"], t["p"], t["experts"], t["dy"], dtype):
        _rel_check(n, a, b, rtol, atol)


def test_leading_dims_and_determinism():
    torch.manual_seed(0)
    m = GLUMLP(64, 96, 8, 2).to(DEV)
    x = torch.randn(3, 17, 64, device=DEV)
    p, e = torch.topk(torch.softmax(torch.randn(51, 8, device=DEV), -1), 2)
    y1, y2 = m(x, p, e), m(x, p, e)
    assert y1.shape == (3, 17, 64) and torch.equal(y1, y2)


@pytest.mark.parametrize("cls,dtype", [(GLUMLP, torch.bfloat16), (GLUMLP, torch.float32), (MLP, torch.float32)])
def test_empty_batch(cls, dtype):
    """No tokens: empty output, empty input gradients, zero weight gradients (every expert is empty)."""
    kw = {} if cls is GLUMLP else {"activation": nn.GELU()}
    with torch.device(DEV):
        m = cls(64, 96, 8, 2, **kw).to(dtype)
    x = torch.empty(0, 64, device=DEV, dtype=dtype, requires_grad=True)
    p = torch.empty(0, 2, device=DEV, dtype=dtype, requires_grad=True)
    experts = torch.empty(0, 2, device=DEV, dtype=torch.int64)
    y = m(x, p, experts)
    assert y.shape == (0, 64)
    y.sum().backward()
    assert x.grad.shape == (0, 64) and p.grad.shape == (0, 2)
    for prm in m.parameters():
        assert prm.grad is not None and not prm.grad.isnan().any() and float(prm.grad.abs().max()) == 0.0


def _random_module_cases():
    import random
    rnd = random.Random(7)
    out = []
    for rows_per_expert in (0.5, 3, 20, 30, 60, 100, 150, 260, 400):
        E = rnd.choice((4, 8, 8, 24))
        k = min(rnd.choice((1, 2, 2, 4)), E)
        T = max(1, round(rows_per_expert * E / k))
        d = rnd.choice((64, 136, 256, 520))
        f = rnd.choice((40, 128, 264, 512))
        out.append((T, E, k, d, f, rnd.choice(("glu", "mlp")), rnd.random() < 0.5,
                    rnd.choice((torch.bfloat16, torch.float16, torch.float32)), rnd.random() < 0.4))
    return out


@pytest.mark.parametrize("T,E,k,d,f,kind,bias,dtype,skew", _random_module_cases())
def test_module_random_shapes(T, E, k, d, f, kind, bias, dtype, skew):
    """Forward and every gradient of MLP / GLUMLP at seeded random sizes that cross the tile-class thresholds,
    against the oracle's per-expert form differentiated by autograd."""
    g = torch.Generator().manual_seed(T * 31 + d)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - 1.5 * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    p, experts = torch.topk(torch.softmax(logits, -1), k)
    x = torch.randn(T, d, generator=g)
    dy = torch.randn(T, d, generator=g)
    torch.manual_seed(d + f)
    m = (GLUMLP(d, f, E, k, bias=bias) if kind == "glu" else MLP(d, f, E, k, bias=bias, activation=nn.GELU()))
    with torch.no_grad():
        for prm in m.parameters():
            prm.normal_(0, 0.05)
    rtol, atol = (1e-4, 1e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    for n, a, b in _run_pair(m, x, p, experts, dy, dtype):
        _rel_check(n, a, b, rtol, atol)


@pytest.mark.parametrize("dtype,T", [(torch.float32, 300), (torch.bfloat16, 300), (torch.bfloat16, 3)])
def test_mixture_of_lora_shape(dtype, T):
    """The module of the reference's example (examples/molora.py:5-17): 16 rank-128 adapters over d = 1024 with
    an identity between the two layers, forward and every gradient."""
    d, rank, E, k = 1024, 128, 16, 2
    g = torch.Generator().manual_seed(T)
    p, experts = torch.topk(torch.softmax(torch.randn(T, E, generator=g), -1), k)
    x = torch.randn(T, d, generator=g)
    dy = torch.randn(T, d, generator=g)
    torch.manual_seed(5)
    m = MLP(d, rank, E, k, activation=nn.Identity())
    with torch.no_grad():
        for prm in m.parameters():
            prm.normal_(0, 0.05)
    rtol, atol = (1e-4, 1e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    for n, a, b in _run_pair(m, x, p, experts, dy, dtype, per_token=(T < 8)):
        _rel_check(n, a, b, rtol, atol)
