"""The two-launch decode step (smoe_decode_glu_mlp: layer 1 + GLU, layer 2 + gate combine, routing done inside the
kernels) against the general path it stands in for (routing, two scatter2scatter launches, combine): bit-identical;
and against the CPU oracle's literal per-token form (rel 2e-2 / abs 1e-2 scaled)."""
import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops
from scattermoe_amd.mlp import GLUMLP

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

ROUTINGS = {
    "one_token": [[1, 6]],
    "two_tokens_shared_expert": [[0, 3], [3, 5]],
    "seven_rows_one_expert": [[2], [2], [2], [2], [2], [2], [2]],
    "four_tokens": [[7, 0], [0, 1], [4, 0], [0, 2]],
    "top4": [[5, 1, 7, 2], [1, 5, 0, 3]],
    "single_row": [[5]],
}


def _general(x, p, experts, w1, b1, w2, b2, act, E):
    eid, idx, off = ops.route(experts, E)
    k = experts.size(1)
    _, h = ops.scatter2scatter_glu(x, w1.permute(0, 2, 1), eid, idx, k, b=b1, act=act, expert_offsets=off,
                                   need_pre=False)
    y = ops.scatter2scatter(h, w2.permute(0, 2, 1), eid, idx, 1, b=b2, x_grouped=True, y_grouped=False,
                            expert_offsets=off)
    return ops.combine(y.view(x.size(0), k, -1), p)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", [ops.ACT_SILU, ops.ACT_SILU_GATE_FIRST])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("d,F", [(64, 8), (200, 104), (1096, 264), (4096, 1032), (264, 6152)])
@pytest.mark.parametrize("routing", sorted(ROUTINGS))
def test_decode_step_equals_general_path_and_oracle(routing, d, F, bias, act, dtype):
    experts = torch.tensor(ROUTINGS[routing])
    T, k = experts.shape
    E = 8
    g = torch.Generator().manual_seed(d + F + T)
    x = torch.randn(T, d, generator=g).to(dtype)
    p = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    w1 = (torch.randn(E, 2 * F, d, generator=g) * 0.1).to(dtype)
    w2 = (torch.randn(E, d, F, generator=g) * 0.1).to(dtype)
    b1 = torch.randn(E, 2 * F, generator=g).to(dtype) if bias else None
    b2 = torch.randn(E, d, generator=g).to(dtype) if bias else None
    dev = lambda t: None if t is None else t.to(DEV)
    got = ops.decode_glu_mlp(dev(x), dev(p), dev(experts), dev(w1), dev(b1), dev(w2), dev(b2), act)
    assert got is not None and got.shape == (T, d)
    ref = _general(dev(x), dev(p), dev(experts), dev(w1), dev(b1), dev(w2), dev(b2), act, E)
    assert torch.equal(got, ref)

    def hidden(pre):
        first, second = pre.chunk(2, dim=-1)
        lin, gat = (second, first) if act == ops.ACT_SILU_GATE_FIRST else (first, second)
        return torch.nn.functional.silu(gat) * lin
    f32 = lambda t: None if t is None else t.float()
    want = oracle.naive_token_forward(x.float(), p.float(), experts, w1.float(), w2.float(), hidden, f32(b1), f32(b2))
    scale = max(1.0, float(want.abs().max()))
    err = (got.float().cpu() - want).abs()
    assert bool((err <= 1e-2 * scale + 2e-2 * want.abs()).all()), "max err %g (scale %g)" % (err.max(), scale)


def test_module_takes_the_decode_step_only_without_grad():
    torch.manual_seed(4)
    with torch.device(DEV):
        m = GLUMLP(256, 384, 8, 2, bias=True).to(torch.bfloat16)
        torch.nn.init.normal_(m.experts.bias, std=0.1)
        torch.nn.init.normal_(m.output_experts.bias, std=0.1)
    x = torch.randn(2, 3, 256, device=DEV, dtype=torch.bfloat16)[:, :2]        # (2, 2, 256) tokens with a leading dim
    x = x.contiguous()
    logits = torch.randn(4, 8, device=DEV)
    w, i = ops.topk_softmax(logits, 2)
    w = w.to(torch.bfloat16)
    with_grad = m(x, w, i)                      # general path (autograd node)
    with torch.no_grad():
        without = m(x, w, i)                    # decode step
    assert without.shape == with_grad.shape == (2, 2, 256)
    assert torch.equal(without, with_grad.detach())


def test_calls_outside_the_decode_step_are_declined():
    x = torch.randn(2, 64, device=DEV)
    e = torch.tensor([[0, 1], [2, 3]], device=DEV)
    p = torch.full((2, 2), 0.5, device=DEV)
    w1, w2 = torch.randn(4, 32, 64, device=DEV), torch.randn(4, 64, 16, device=DEV)
    assert ops.decode_glu_mlp(x, p, e, w1, None, w2, None) is None                             # float32
    h = torch.bfloat16
    e10 = torch.zeros(5, 2, dtype=torch.int64, device=DEV)
    assert ops.decode_glu_mlp(torch.randn(5, 64, device=DEV, dtype=h), torch.ones(5, 2, device=DEV, dtype=h), e10,
                              w1.to(h), None, w2.to(h), None) is None                          # ten rows
    w1o = torch.randn(4, 32, 68, device=DEV, dtype=h)[:, :, :60]                               # d = 60: rows not 16-byte multiples
    assert ops.decode_glu_mlp(torch.randn(2, 60, device=DEV, dtype=h), p.to(h), e, w1o,
                              None, torch.randn(4, 60, 16, device=DEV, dtype=h), None) is None
