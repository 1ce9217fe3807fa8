"""Few-row launches (at most 8 expert rows, K-contiguous bf16 / fp16 weights) run on the row-dot kernel instead
of the MFMA tiles: parity against the CPU oracle for plain and GLU-fused forms, every scatter/gather mode, bias,
contraction lengths that are not multiples of what a wave or a workgroup covers per step, ragged column counts,
several rows per expert (one tile holds four) and experts with more rows than one tile.
Tolerance: rel 2e-2 / abs 1e-2 scaled by the magnitude a dot product of that length reaches."""
import itertools

import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _close(got, want, scale):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = 1e-2 * scale + 2e-2 * want.abs()
    assert bool((err <= bound).all()), "max err %g at bound %g" % (err.max(), bound.flatten()[err.argmax()])


# expert ids per token (T, k): L = T*k <= 8
ROUTINGS = {
    "one_token": [[1, 6]],
    "two_tokens": [[0, 3], [3, 5]],
    "same_expert": [[2], [2], [2], [2], [2], [2], [2]],          # 7 rows of one expert: two tiles
    "four_tokens": [[7, 0], [0, 1], [4, 0], [0, 2]],               # expert 0 has four rows
    "single_row": [[5]],
}
# K, N
DIMS = [(64, 8), (200, 13), (1096, 136), (4096, 264), (2568, 24)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K,N", DIMS)
@pytest.mark.parametrize("routing", sorted(ROUTINGS))
def test_rowdot_gather_to_grouped(routing, K, N, dtype):
    experts = torch.tensor(ROUTINGS[routing])
    T, k = experts.shape
    E = 8
    eid, idx, off = oracle.route_ref(experts, E)
    g = torch.Generator().manual_seed(K + N + T)
    X = torch.randn(T, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    b = torch.randn(E, N, generator=g).to(dtype)
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, k, b.float(), False, True)
    out = torch.full((T * k, N), float("nan"), dtype=dtype, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wp.to(DEV).permute(0, 2, 1), eid.to(DEV), idx.to(DEV), k, b=b.to(DEV),
                              y_grouped=True, expert_offsets=off.to(DEV), out=out)
    _close(got, want, scale=0.1 * K ** 0.5)


@pytest.mark.parametrize("x_grouped,y_grouped", list(itertools.product([False, True], repeat=2)))
@pytest.mark.parametrize("routing", ["four_tokens", "same_expert"])
def test_rowdot_modes(routing, x_grouped, y_grouped):
    experts = torch.tensor(ROUTINGS[routing])
    T, k = experts.shape
    E, K, N = 8, 520, 40
    eid, idx, off = oracle.route_ref(experts, E)
    fan = 1 if x_grouped else k
    g = torch.Generator().manual_seed(17)
    X = torch.randn(T * k // fan, K, generator=g).bfloat16()
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).bfloat16()
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, None, x_grouped, y_grouped)
    out = torch.full((T * k, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wp.to(DEV).permute(0, 2, 1), eid.to(DEV), idx.to(DEV), fan,
                              x_grouped=x_grouped, y_grouped=y_grouped, expert_offsets=off.to(DEV), out=out)
    assert not torch.isnan(got.float()).any()
    _close(got, want, scale=0.1 * K ** 0.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", [ops.ACT_SILU, ops.ACT_SILU_GATE_FIRST])
@pytest.mark.parametrize("bias,need_pre", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("K,F", [(64, 4), (1096, 13), (4096, 130)])
@pytest.mark.parametrize("routing", ["one_token", "four_tokens", "same_expert"])
def test_rowdot_fused_glu(routing, K, F, bias, need_pre, act, dtype):
    experts = torch.tensor(ROUTINGS[routing])
    T, k = experts.shape
    E = 8
    eid, idx, off = oracle.route_ref(experts, E)
    g = torch.Generator().manual_seed(K + F)
    X = torch.randn(T, K, generator=g).to(dtype)
    Wp = (torch.randn(E, 2 * F, K, generator=g) * 0.1).to(dtype)
    b = torch.randn(E, 2 * F, generator=g).to(dtype) if bias else None
    pre_want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, k,
                                          None if b is None else b.float(), False, True)
    pre_r = pre_want.to(dtype).float()                 # the hidden value is computed from the rounded halves
    first, second = pre_r.chunk(2, dim=-1)
    lin, gat = (second, first) if act == ops.ACT_SILU_GATE_FIRST else (first, second)
    h_want = torch.nn.functional.silu(gat) * lin
    pre, h = ops.scatter2scatter_glu(X.to(DEV), Wp.to(DEV).permute(0, 2, 1), eid.to(DEV), idx.to(DEV), k,
                                     b=None if b is None else b.to(DEV), act=act, expert_offsets=off.to(DEV),
                                     need_pre=need_pre)
    scale = 0.1 * K ** 0.5
    if need_pre:
        _close(pre, pre_want, scale)
    else:
        assert pre is None
    _close(h, h_want, scale * max(1.0, scale))


def test_rowdot_matches_the_tile_kernels_on_the_module():
    """One decode token through GLUMLP (row-dot kernels) against the same token among 64 (MFMA tiles)."""
    from scattermoe_amd.mlp import GLUMLP
    torch.manual_seed(3)
    m = GLUMLP(256, 384, 8, 2).to(DEV).to(torch.bfloat16)
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16)
    logits = torch.randn(64, 8, device=DEV)
    w, i = torch.topk(torch.softmax(logits, -1), 2)
    w = w.to(torch.bfloat16)
    with torch.no_grad():
        many = m(x, w, i)
        for t in (0, 17, 63):
            one = m(x[t:t + 1], w[t:t + 1], i[t:t + 1])
            torch.testing.assert_close(one.float(), many[t:t + 1].float(), rtol=2e-2, atol=2e-2)
