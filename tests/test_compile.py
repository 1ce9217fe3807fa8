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
