"""torch.compile(fullgraph=True) traces through every launch: each one is a registered operator
(the reference registers its three kernels and the bincount the same way, scattermoe/kernels/ops.py:140, :202,
:389 and parallel_experts.py:6).  The CPU test traces with the `aot_eager` backend over the oracle test double;
the GPU test compiles with the default backend and compares with eager."""
import pytest
import torch
from torch import nn


def _make(cls, dtype, device):
    from scattermoe_amd.mlp import MLP, GLUMLP
    kind = GLUMLP if cls == "glu" else MLP
    kw = {} if cls == "glu" else {"activation": nn.GELU()}
    torch.manual_seed(0)
    with torch.device(device):
        return kind(64, 96, 8, 2, **kw).to(dtype)


def _run(m, x, logits, compiled, backend):
    from scattermoe_amd.kernels import ops

    def f(x, logits):
        p, e = ops.topk_softmax(logits, 2)
        return m(x, p.to(x.dtype), e)

    torch._dynamo.reset()
    fn = torch.compile(f, fullgraph=True, backend=backend) if compiled else f
    y = fn(x, logits)
    grads = torch.autograd.grad(y.sum(), [x, logits] + list(m.parameters()))
    return [y.detach()] + [g.detach() for g in grads]


@pytest.mark.parametrize("cls", ["mlp", "glu"])
def test_fullgraph_trace_cpu(cls, cpu_backend):
    m = _make(cls, torch.float32, "cpu")
    g = torch.Generator().manual_seed(1)
    x = torch.randn(30, 64, generator=g, requires_grad=True)
    logits = torch.randn(30, 8, generator=g, requires_grad=True)
    want = _run(m, x, logits, False, None)
    got = _run(m, x, logits, True, "aot_eager")
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("cls,dtype", [("mlp", torch.float32), ("glu", torch.float32), ("glu", torch.bfloat16)])
def test_fullgraph_compile_gpu(cls, dtype):
    m = _make(cls, dtype, "cuda:0")
    g = torch.Generator().manual_seed(1)
    x = torch.randn(50, 64, generator=g).to(dtype).to("cuda:0").requires_grad_()
    logits = torch.randn(50, 8, generator=g).to("cuda:0").requires_grad_()
    want = _run(m, x, logits, False, None)
    got = _run(m, x, logits, True, "inductor")
    # the launches are the same ones; what the compiler generates itself (activation, softmax gradient) may round
    # differently from eager
    tol = dict(rtol=1e-4, atol=1e-5) if dtype is torch.float32 else dict(rtol=2e-2, atol=1e-2)
    for a, b in zip(got, want):
        torch.testing.assert_close(a.float(), b.float(), **tol)


@pytest.mark.gpu
def test_compiled_step_issues_the_same_launches_as_eager():
    """The benchmark's layer in small (GLUMLP, bf16, 8 experts, top-2; wide enough for the fused gated launches, the
    weight gradient that reads tokens through the index vector and the one-pass gate gradient): compiled with
    fullgraph=True, the forward + backward step must equal the eager one BIT FOR BIT - every launch is a registered
    operator that runs the same kernel on the same operands, and nothing is left for the compiler to generate."""
    from scattermoe_amd.mlp import GLUMLP
    from scattermoe_amd.kernels import ops
    dev, bf = "cuda:0", torch.bfloat16
    T, d, f, E, k = 4096, 512, 1024, 8, 2
    torch.manual_seed(0)
    with torch.device(dev):
        m = GLUMLP(d, f, E, k, bias=True).to(bf)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, d, generator=g).to(bf).to(dev).requires_grad_()
    probs = torch.softmax(torch.randn(T, E, generator=g), -1)
    p, experts = torch.topk(probs, k)
    p = p.to(bf).to(dev).requires_grad_()
    experts = experts.to(dev)
    dy = torch.randn(T, d, generator=g).to(bf).to(dev)
    leaves = [x, p] + list(m.parameters())

    def run(fn):
        y = fn(x, p, experts)
        return [y.detach()] + [t.detach() for t in torch.autograd.grad(y, leaves, dy)]

    seen = []
    real = ops._backend

    class Spy:
        def __getattr__(self, name):
            fn = getattr(real, name)

            def call(*a, **kw):
                seen.append(name)
                return fn(*a, **kw)
            return call

    want = run(m)
    ops._backend = Spy()
    try:
        eager_launches = (run(m), list(seen))[1]
        seen.clear()
        torch._dynamo.reset()
        got = run(torch.compile(lambda x, p, e: m(x, p, e), fullgraph=True))
        compiled_launches = list(seen)
    finally:
        ops._backend = real
    assert compiled_launches == eager_launches, (compiled_launches, eager_launches)
    assert "s2s_glu" in eager_launches and "xty_gathered" in eager_launches and "gate_grad_group" in eager_launches
    for a, b in zip(got, want):
        assert torch.equal(a, b)
