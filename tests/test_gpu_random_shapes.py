"""Seeded random shapes across every dispatch boundary of scatter2scatter / group_bwd_W (rows per expert around
8 rows in total, 24, 52, 112 and 224 per expert; contraction and column counts that are and are not multiples of
the tile sizes; both weight layouts; all gather / scatter modes; fan-out 1..4; skewed routing with empty experts)
against the CPU oracle.  Tolerance: rel 2e-2 / abs 1e-2 scaled by the magnitude a dot product of that length reaches."""
import random

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


def _cases():
    rnd = random.Random(1234)
    out = []
    # rows per expert targets straddling the class thresholds, in total rows L = T * k
    for target in (0.25, 1, 2, 7, 20, 23, 25, 40, 47, 51, 53, 80, 111, 113, 160, 223, 225, 300, 600):
        for _ in range(2):
            E = rnd.choice((2, 4, 8, 8, 16, 37))
            k = rnd.choice((1, 2, 2, 3, 4))
            k = min(k, E)
            T = max(1, round(target * E / k))
            K = rnd.choice((64, 72, 200, 256, 520, 1096))
            N = rnd.choice((8, 40, 136, 256, 264, 520, 1032))
            out.append((T, E, k, K, N, rnd.choice(("k_contig", "n_contig")), rnd.choice((torch.bfloat16, torch.float16)),
                        rnd.random() < 0.5, rnd.random() < 0.5, rnd.random() < 0.5, rnd.randrange(1 << 30)))
    return out


@pytest.mark.parametrize("T,E,k,K,N,layout,dtype,x_grouped,y_grouped,skew,seed", _cases())
def test_scatter2scatter_random(T, E, k, K, N, layout, dtype, x_grouped, y_grouped, skew, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - 2.0 * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    experts = torch.topk(logits, k).indices
    eid, idx, off = oracle.route_ref(experts, E)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    b = torch.randn(E, N, generator=g).to(dtype)
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if layout == "n_contig":
        Wd = Wd.contiguous()
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, b.float(), x_grouped, y_grouped)
    out = torch.full((T * k, N), float("nan"), dtype=dtype, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), fan, b=b.to(DEV), x_grouped=x_grouped,
                              y_grouped=y_grouped, expert_offsets=off.to(DEV), out=out)
    assert not torch.isnan(got.float()).any()
    _close(got, want, scale=0.1 * K ** 0.5 + 1.0)


@pytest.mark.parametrize("T,E,k,K,N,layout,dtype,x_grouped,y_grouped,skew,seed", _cases()[::3])
def test_group_bwd_W_random(T, E, k, K, N, layout, dtype, x_grouped, y_grouped, skew, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - 2.0 * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    experts = torch.topk(logits, k).indices
    eid, idx, off = oracle.route_ref(experts, E)
    L = T * k
    X = torch.randn(L, K, generator=g).to(dtype)
    DY = (torch.randn(L, N, generator=g) * 0.1).to(dtype)
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.float(), X.float(), off, E, has_bias=True)
    like = torch.empty(E, K, N, device=DEV, dtype=dtype) if layout == "n_contig" else None
    DW, Db = ops.group_bwd_W(DY.to(DEV), X.to(DEV), off.to(DEV), E, has_bias=True, like=like)
    assert DW.shape == (E, K, N) and (DW.is_contiguous() if like is not None else DW.permute(0, 2, 1).is_contiguous())
    rows = max(1, int(torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)).max()))
    _close(DW, DW_ref, scale=0.1 * rows ** 0.5)
    _close(Db, Db_ref, scale=0.1 * rows ** 0.5)


# ---------------------------------------------------------------------------------------------------
# float32: rows that are 16-byte multiples run on the fp32 MFMA kernels, everything else on the any-layout kernels;
# both to rel 1e-4 (scaled by the magnitude of the dot products)
# ---------------------------------------------------------------------------------------------------
def _close32(got, want, scale):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = 1e-5 * scale + 1e-4 * want.abs()
    assert bool((err <= bound).all()), "max err %g at bound %g" % (err.max(), bound.flatten()[err.argmax()])


def _cases32():
    rnd = random.Random(99)
    out = []
    for target in (0.5, 3, 30, 100, 129, 300):
        for K, N in ((64, 128), (200, 264), (36, 4), (516, 388), (130, 75)):        # the last one: not 16-byte rows
            E = rnd.choice((2, 8, 19))
            k = min(rnd.choice((1, 2, 3)), E)
            T = max(1, round(target * E / k))
            out.append((T, E, k, K, N, rnd.choice(("k_contig", "n_contig")), rnd.random() < 0.5, rnd.random() < 0.5,
                        rnd.random() < 0.5, rnd.randrange(1 << 30)))
    return out


@pytest.mark.parametrize("T,E,k,K,N,layout,x_grouped,y_grouped,skew,seed", _cases32())
def test_float32_random(T, E, k, K, N, layout, x_grouped, y_grouped, skew, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - 2.0 * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    experts = torch.topk(logits, k).indices
    eid, idx, off = oracle.route_ref(experts, E)
    fan = 1 if x_grouped else k
    L = T * k
    X = torch.randn(L // fan, K, generator=g)
    Wp = torch.randn(E, N, K, generator=g) * 0.1
    b = torch.randn(E, N, generator=g)
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if layout == "n_contig":
        Wd = Wd.contiguous()
    want = oracle.scatter2scatter_ref(X.double(), Wp.permute(0, 2, 1).double(), eid, idx, fan, b.double(), x_grouped,
                                      y_grouped, acc=torch.float64)
    out = torch.full((L, N), float("nan"), device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), fan, b=b.to(DEV), x_grouped=x_grouped,
                              y_grouped=y_grouped, expert_offsets=off.to(DEV), out=out)
    assert not torch.isnan(got).any()
    _close32(got, want, scale=0.1 * K ** 0.5 + 1.0)

    Xg = torch.randn(L, K, generator=g)
    DY = torch.randn(L, N, generator=g) * 0.1
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.double(), Xg.double(), off, E, has_bias=True, acc=torch.float64)
    like = torch.empty(E, K, N, device=DEV) if layout == "n_contig" else None
    DW, Db = ops.group_bwd_W(DY.to(DEV), Xg.to(DEV), off.to(DEV), E, has_bias=True, like=like)
    rows = max(1, int(torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)).max()))
    _close32(DW, DW_ref, scale=0.1 * rows ** 0.5)
    _close32(Db, Db_ref, scale=0.1 * rows ** 0.5)
