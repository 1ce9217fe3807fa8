"""bf16 / fp16 MFMA paths: shapes that exercise every tile class, contraction and column tails, both
weight layouts, scatter/gather modes, empty and tiny experts.  Oracle: CPU fp32 on the same rounded
inputs; tolerance rel 2e-2 / abs 1e-2 (scaled by the magnitude a dot product of that length reaches)."""
import itertools

import pytest
import torch

import oracle
import scattermoe_amd as sm
from scattermoe_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _close(got, want, scale):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = 1e-2 * scale + 2e-2 * want.abs()
    assert bool((err <= bound).all()), "max err %g at bound %g" % (err.max(), bound.flatten()[err.argmax()])


def _routing(T, E, k, seed, skew=0.0, empty=()):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - skew * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    for e in empty:
        logits[:, e] = -1e9
    experts = torch.topk(logits, k).indices
    return experts, oracle.route_ref(experts, E)


# T, E, k, K, N  — rows/expert select the tile class
SHAPES = [
    (4096, 8, 2, 512, 768),      # 1024 rows/expert: 256x256 tiles, exact multiples
    (1100, 8, 2, 200, 264),      # 275 rows/expert: ragged row tails, K % 64 != 0, N % 256 != 0
    (520, 8, 2, 320, 1000),      # 130 rows/expert: ring-buffered 256x128 tiles
    (160, 8, 3, 448, 72),        # 60 rows/expert: ring-buffered 128x128 tiles, N < one tile
    (300, 8, 2, 200, 328),       # 75 rows/expert: 128x128 ring tiles with contraction and column tails
    (130, 8, 2, 448, 200),       # ~32 rows/expert: 64-row ring tiles
    (3, 8, 2, 64, 256),          # decode-like: a handful of rows (ring-buffered 32-row tiles)
    (40, 8, 2, 200, 264),        # 10 rows/expert: 32-row tiles with contraction and column tails
    (9, 4, 2, 1096, 136),        # 32-row tiles, contraction longer than the ring (17 full slices + tail)
    (40, 8, 2, 200, 1288),       # enough 128-wide tiles to pick the 64-wide ring class for K-contiguous weights
    (2048, 32, 4, 192, 328),     # E = 32 with skew: tiny and empty experts
    (960, 8, 2, 64, 4096),       # 240 rows/expert, about half a round of 256x256 tiles: half-width tiles chosen
    (1600, 32, 2, 64, 4096),     # 100 rows/expert and 512 wide tiles: 128x256 ring tiles
    (2560, 32, 2, 64, 4096),     # 160 rows/expert and 512 wide tiles: 256x256 tiles below their usual threshold
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("T,E,k,K,N", SHAPES)
def test_s2s_gather_to_grouped(T, E, k, K, N, w_layout, dtype):
    experts, (eid, idx, off) = _routing(T, E, k, seed=K + N, skew=2.0 if E == 32 else 0.0,
                                        empty=(3,) if E == 32 else ())
    g = torch.Generator().manual_seed(T)
    X = torch.randn(T, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)          # parameter layout (E, out, in)
    b = (torch.randn(E, N, generator=g)).to(dtype)
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if w_layout == "n_contig":
        Wd = Wd.contiguous()
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, k, b.float(), False, True)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), k, b=b.to(DEV), y_grouped=True,
                              expert_offsets=off.to(DEV))
    _close(got, want, scale=0.1 * K ** 0.5)


@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("x_grouped,y_grouped", list(itertools.product([False, True], repeat=2)))
def test_s2s_modes(x_grouped, y_grouped, w_layout):
    T, E, k, K, N = 900, 8, 2, 256, 512
    experts, (eid, idx, off) = _routing(T, E, k, seed=5, skew=1.0, empty=(6,))
    g = torch.Generator().manual_seed(9)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g).bfloat16()
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).bfloat16()
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if w_layout == "n_contig":
        Wd = Wd.contiguous()
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, None, x_grouped, y_grouped)
    out = torch.full((T * k, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), fan, x_grouped=x_grouped,
                              y_grouped=y_grouped, out=out, expert_offsets=off.to(DEV))
    _close(got, want, scale=0.1 * K ** 0.5)
    again = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), fan, x_grouped=x_grouped,
                                y_grouped=y_grouped, expert_offsets=off.to(DEV))
    assert torch.equal(got, again)


@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("x_grouped,y_grouped", list(itertools.product([False, True], repeat=2)))
@pytest.mark.parametrize("T,skew", [(4000, 0.0), (4200, 0.0), (4000, 1.0)])
def test_s2s_launch_split_by_tile_rows(T, skew, x_grouped, y_grouped, w_layout):
    """Two whole rounds of 256 x 256 tiles plus a remainder of up to half a round (T = 4000: 32 expected remaining
    tiles, T = 4200: 96): the product is cut by tile rows and the remainder goes to a launch of 256 x 128 tiles;
    with skewed routing the host's expectation of the tile rows is off.  Every output row must be written exactly
    once, and each element must be the same bits as in the launches over the two column halves, which are not
    split."""
    E, k, K, N = 8, 2, 64, 4096
    experts, (eid, idx, off) = _routing(T, E, k, seed=T, skew=skew)
    g = torch.Generator().manual_seed(T + 1)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g).bfloat16()
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).bfloat16()
    b = torch.randn(E, N, generator=g).bfloat16()
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if w_layout == "n_contig":
        Wd = Wd.contiguous()
    args = (eid.to(DEV), idx.to(DEV), fan)
    kw = dict(x_grouped=x_grouped, y_grouped=y_grouped, expert_offsets=off.to(DEV))
    out = torch.full((T * k, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, *args, b=b.to(DEV), out=out, **kw)
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, b.float(), x_grouped, y_grouped)
    _close(got, want, scale=0.1 * K ** 0.5)
    halves = [ops.scatter2scatter(X.to(DEV), Wd[:, :, c:c + N // 2], *args, b=b.to(DEV)[:, c:c + N // 2], **kw)
              for c in (0, N // 2)]
    assert torch.equal(got, torch.cat(halves, 1))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("x_grouped,y_grouped", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("K", [1792, 1856])
def test_s2s_long_contraction(K, x_grouped, y_grouped, w_layout, dtype):
    """Contractions of 1792 and more run on the one-wave-per-SIMD form of the 256 x 256 class (operands through
    registers, 28 and 29 slices: the loop handles two slices per trip): ragged tile rows, an expert without rows,
    a partial tile column, bias."""
    T, E, k, N = 1500, 4, 2, 520
    experts, (eid, idx, off) = _routing(T, E, k, seed=K, skew=0.5, empty=(2,))
    g = torch.Generator().manual_seed(K + 1)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.05).to(dtype)
    b = torch.randn(E, N, generator=g).to(dtype)
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if w_layout == "n_contig":
        Wd = Wd.contiguous()
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, b.float(), x_grouped, y_grouped)
    out = torch.full((T * k, N), float("nan"), dtype=dtype, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), fan, b=b.to(DEV), x_grouped=x_grouped,
                              y_grouped=y_grouped, out=out, expert_offsets=off.to(DEV))
    _close(got, want, scale=0.05 * K ** 0.5)


def test_s2s_long_contraction_same_bits_as_column_halves():
    """The one-wave-per-SIMD form and the 8-wave form add up every output element in the same order: a product
    whose remainder of tile rows goes to a second launch of 256 x 128 tiles (8 waves) equals, bit for bit, the two
    launches over its column halves, which are not split."""
    T, E, k, K, N = 4200, 8, 2, 1792, 4096
    experts, (eid, idx, off) = _routing(T, E, k, seed=3)
    g = torch.Generator().manual_seed(4)
    X = torch.randn(T, K, generator=g).bfloat16().to(DEV)
    Wd = (torch.randn(E, N, K, generator=g) * 0.05).bfloat16().to(DEV).permute(0, 2, 1)
    args = (eid.to(DEV), idx.to(DEV), k)
    kw = dict(y_grouped=True, expert_offsets=off.to(DEV))
    got = ops.scatter2scatter(X, Wd, *args, **kw)
    halves = [ops.scatter2scatter(X, Wd[:, :, c:c + N // 2], *args, **kw) for c in (0, N // 2)]
    assert torch.equal(got, torch.cat(halves, 1))


LAST_TILE_COUNTS = [1380, 1224, 1024, 0, 60, 1408, 1409, 1281]


def _routing_with_counts(counts, k, seed):
    """Routing in which expert e receives exactly counts[e] of the T * k slots."""
    E, L = len(counts), sum(counts)
    g = torch.Generator().manual_seed(seed)
    experts = torch.repeat_interleave(torch.arange(E), torch.tensor(counts))[torch.randperm(L, generator=g)].view(L // k, k)
    eid, idx, off = oracle.route_ref(experts, E)
    assert off.tolist() == torch.tensor(counts).cumsum(0).tolist()
    return eid, idx, off, g


@pytest.mark.parametrize("x_grouped,y_grouped", [(False, True), (True, False), (True, True)])
def test_s2s_last_tiles_of_few_rows_in_their_own_launch(x_grouped, y_grouped):
    """A large product with fewer than 1536 rows per expert leaves every expert's last tile of at most 128 rows to a
    second launch of 128-row tiles.  Row counts chosen for each case of the tile lookup: a last tile of 100 rows
    (second launch), of 200 rows (stays), none (exact multiple of 256), an expert without rows, one of 60 rows
    (only the second launch sees it), last tiles of exactly 128 and of 129 rows, and one of 1 row.  Every row must
    be written once, to the oracle's values, and with the same bits as the launches over the column halves, which
    are too small to be split.  (30 tile columns: 3.75 rounds, so the product is not cut by whole rounds instead.)"""
    counts, k, K, N = LAST_TILE_COUNTS, 2, 2048, 7680
    E, L = len(counts), sum(counts)
    eid, idx, off, g = _routing_with_counts(counts, k, seed=11)
    fan = 1 if x_grouped else k
    X = torch.randn(L // fan, K, generator=g).bfloat16()
    Wp = (torch.randn(E, N, K, generator=g) * 0.05).bfloat16()
    b = torch.randn(E, N, generator=g).bfloat16()
    Wd = Wp.to(DEV).permute(0, 2, 1)
    args = (eid.to(DEV), idx.to(DEV), fan)
    kw = dict(x_grouped=x_grouped, y_grouped=y_grouped, expert_offsets=off.to(DEV))
    out = torch.full((L, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, *args, b=b.to(DEV), out=out, **kw)
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, fan, b.float(), x_grouped, y_grouped)
    _close(got, want, scale=0.05 * K ** 0.5)
    halves = [ops.scatter2scatter(X.to(DEV), Wd[:, :, c:c + N // 2], *args, b=b.to(DEV)[:, c:c + N // 2], **kw)
              for c in (0, N // 2)]
    assert torch.equal(got, torch.cat(halves, 1))


SPLIT_COUNTS = [1613, 1830, 1792, 2432, 60]      # last tiles of 77, 38, none, 128 rows; an expert of 60 rows only


def _s2s_through_the_c_abi(X, W, b, eid, idx, off, fan, x_grouped, y_grouped, workspace):
    """smoe_scatter2scatter_ws with the workspace the library asks for, or smoe_scatter2scatter (none)."""
    from scattermoe_amd import _C
    lib = _C.load()
    L, N = eid.numel(), W.size(2)
    Y = torch.full((L, N), float("nan"), dtype=X.dtype, device=DEV)
    common = (_C.ptr(X), X.stride(0), X.stride(1), _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
              _C.ptr(b), b.stride(0), b.stride(1), _C.ptr(Y), Y.stride(0), Y.stride(1), _C.ptr(eid), _C.ptr(idx),
              _C.ptr(off), L, X.size(1), N, W.size(0), fan, int(x_grouped), int(y_grouped), _C.float_code(X.dtype))
    if workspace:
        need = lib.smoe_scatter2scatter_workspace_bytes(L, X.size(1), N, W.size(0), _C.float_code(X.dtype))
        assert need > 0, "this product is meant to split the contraction of its last tiles"
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        rc = lib.smoe_scatter2scatter_ws(*common, _C.ptr(ws), need, _C.stream_ptr(X.device))
    else:
        rc = lib.smoe_scatter2scatter(*common, _C.stream_ptr(X.device))
    assert rc == 0, lib.smoe_last_error()
    torch.cuda.synchronize()
    return Y


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("x_grouped,y_grouped", [(False, True), (True, False), (True, True)])
def test_s2s_last_tiles_with_split_contraction(x_grouped, y_grouped, w_layout, dtype):
    """Many rows per expert, few tile columns and a long contraction (the Mixtral layer-2 forward and layer-1 input
    gradient in small): with a workspace the experts' last tiles of at most 128 rows are multiplied in contraction
    parts and added up by a second launch.  Against the oracle at the usual bar; the same bits on a second run (the
    parts are added in a fixed order); and against the product without workspace: the same bits in every row outside
    those tiles, within float32 regrouping of the sum (one unit in the last place of the 16-bit result) inside."""
    counts, k, K, N = SPLIT_COUNTS, 1, 4096, 4096
    E, L = len(counts), sum(counts)
    eid, idx, off, g = _routing_with_counts(counts, k, seed=21)
    X = torch.randn(L, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.03).to(dtype)
    b = torch.randn(E, N, generator=g).to(dtype)
    Wd = Wp.to(DEV).permute(0, 2, 1)
    if w_layout == "n_contig":
        Wd = Wd.contiguous()
    args = (X.to(DEV), Wd, b.to(DEV), eid.to(DEV), idx.to(DEV), off.to(DEV), 1, x_grouped, y_grouped)
    got = _s2s_through_the_c_abi(*args, workspace=True)
    want = oracle.scatter2scatter_ref(X.float(), Wp.permute(0, 2, 1).float(), eid, idx, 1, b.float(), x_grouped, y_grouped)
    _close(got, want, scale=0.03 * K ** 0.5)
    assert torch.equal(got, _s2s_through_the_c_abi(*args, workspace=True))
    plain = _s2s_through_the_c_abi(*args, workspace=False)
    in_tail = torch.zeros(L, dtype=torch.bool)
    lo = 0
    for c in counts:
        if 0 < c % 256 <= 128:
            in_tail[lo + c - c % 256:lo + c] = True
        lo += c
    rows = in_tail if y_grouped else torch.zeros(L, dtype=torch.bool).index_put_((idx,), in_tail)
    assert int(rows.sum()) == 77 + 38 + 128 + 60
    assert torch.equal(got[~rows.to(DEV)], plain[~rows.to(DEV)])
    a, p = got[rows.to(DEV)].float(), plain[rows.to(DEV)].float()
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    assert bool(((a - p).abs() <= ulp * p.abs() + 1e-4).all())      # float32 regrouping of a sum of 4096 terms of size 1
    # the module-level wrapper brings the workspace by itself
    via_ops = ops.scatter2scatter(args[0], Wd, args[3], args[4], 1, b=args[2], x_grouped=x_grouped, y_grouped=y_grouped,
                                  expert_offsets=args[5])
    assert torch.equal(via_ops, got)


def test_s2s_workspace_that_is_too_small_or_misaligned_is_not_used():
    """smoe_scatter2scatter_ws with less workspace than it asks for, or with a workspace that is not 16-byte aligned,
    is exactly smoe_scatter2scatter: same bits, nothing written to the workspace."""
    from scattermoe_amd import _C
    lib = _C.load()
    counts, K, N = SPLIT_COUNTS, 4096, 4096
    E, L = len(counts), sum(counts)
    eid, idx, off, g = _routing_with_counts(counts, 1, seed=22)
    X = torch.randn(L, K, generator=g).bfloat16().to(DEV)
    W = (torch.randn(E, N, K, generator=g) * 0.03).bfloat16().to(DEV).permute(0, 2, 1)
    b = torch.randn(E, N, generator=g).bfloat16().to(DEV)
    eid, idx, off = eid.to(DEV), idx.to(DEV), off.to(DEV)
    plain = _s2s_through_the_c_abi(X, W, b, eid, idx, off, 1, True, False, workspace=False)
    need = lib.smoe_scatter2scatter_workspace_bytes(L, K, N, E, _C.float_code(X.dtype))
    assert need == E * (N // 256) * 4 * 128 * 256 * 4                  # experts x tile columns x parts x one float32 tile
    ws = torch.full((need + 64,), 0x5a, dtype=torch.uint8, device=DEV)
    for ptr, size in ((ws.data_ptr(), need - 16), (ws.data_ptr() + 8, need)):
        Y = torch.full((L, N), float("nan"), dtype=X.dtype, device=DEV)
        rc = lib.smoe_scatter2scatter_ws(_C.ptr(X), X.stride(0), X.stride(1), _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                                         _C.ptr(b), b.stride(0), b.stride(1), _C.ptr(Y), Y.stride(0), Y.stride(1),
                                         _C.ptr(eid), _C.ptr(idx), _C.ptr(off), L, K, N, E, 1, 1, 0, _C.float_code(X.dtype),
                                         ptr, size, _C.stream_ptr(X.device))
        assert rc == 0, lib.smoe_last_error()
        torch.cuda.synchronize()
        assert torch.equal(Y, plain)
        assert bool((ws == 0x5a).all())
    # products that would not split ask for none
    assert lib.smoe_scatter2scatter_workspace_bytes(L, K, 28672, E, _C.float_code(X.dtype)) == 0      # enough tile columns
    assert lib.smoe_scatter2scatter_workspace_bytes(L, 64, N, E, _C.float_code(X.dtype)) == 0         # short contraction
    assert lib.smoe_scatter2scatter_workspace_bytes(L, K, N, E, _C.F32) == 0


@pytest.mark.parametrize("act", ["SILU", "GPT_OSS"])
def test_fused_gated_products_with_last_tiles_in_their_own_launch(act):
    """The same row counts through the products that carry the gated unit in their epilogue (forward: saved
    pre-activations and hidden rows; backward: gradient of the pre-activations), against the plain product followed
    by the elementwise pass, which is checked above."""
    counts, k, d, F = LAST_TILE_COUNTS, 2, 2048, 4096
    E, L = len(counts), sum(counts)
    eid, idx, off, g = _routing_with_counts(counts, k, seed=12)
    eid, idx, off = eid.to(DEV), idx.to(DEV), off.to(DEV)
    code = getattr(ops, "ACT_" + act)
    extra = dict(alpha=1.702, limit=7.0) if act == "GPT_OSS" else {}
    x = torch.randn(L // k, d, generator=g).bfloat16().to(DEV)
    W1 = (torch.randn(E, 2 * F, d, generator=g) * 0.05).bfloat16().to(DEV).permute(0, 2, 1)
    b1 = (torch.randn(E, 2 * F, generator=g) * 0.1).bfloat16().to(DEV)
    pre_ref = ops.scatter2scatter(x, W1, eid, idx, k, b=b1, y_grouped=True, expert_offsets=off)
    pre, h = ops.scatter2scatter_glu(x, W1, eid, idx, k, b=b1, act=code, expert_offsets=off, **extra)
    assert torch.equal(pre, pre_ref)
    h_ref = ops.gpt_oss_glu(pre_ref, 1.702, 7.0) if act == "GPT_OSS" else ops.glu_fwd(pre_ref, code)
    assert float((h.float() - h_ref.float()).abs().max()) <= 2 ** -7 * float(h_ref.float().abs().max())
    # backward through the second linear: (L, d) gradient rows times (E, d, F) weights, 2 * L * d * F flop
    dy = torch.randn(L, 2 * d, generator=g).bfloat16().to(DEV)
    W2 = (torch.randn(E, 2 * d, F, generator=g) * 0.05).bfloat16().to(DEV)
    dh = ops.scatter2scatter(dy, W2, eid, idx, 1, x_grouped=True, y_grouped=True, expert_offsets=off)
    ref = torch.empty_like(pre)
    if act == "GPT_OSS":
        ops._launch("oss_glu_bwd", pre, dh, ref, 1.702, 7.0)
    else:
        ref = ops.glu_bwd(pre, dh, code)
    got = ops.scatter2scatter_glu_bwd(dy, W2, pre, eid, idx, act=code, expert_offsets=off, **extra)
    err = (got.float() - ref.float()).abs()
    assert bool((err <= 2 ** -7 * ref.float().abs() + 1e-30).all())


@pytest.mark.parametrize("T,E,k,K,N", [(4000, 8, 2, 64, 4096),        # cut by tile rows: whole rounds + remainder
                                       (5000, 8, 2, 2048, 7680),      # experts' last tiles of few rows on their own
                                       (4100, 4, 2, 4096, 4096)])     # ... multiplied in contraction parts (workspace)
def test_split_product_replays_from_a_graph(T, E, k, K, N):
    """A product that runs as two launches (see the tests above), routing included, captured into a HIP graph and
    replayed on fresh inputs (the routing, hence which tiles go to which launch, changes from replay to replay), with
    eager work between the replays: every replay equals the eager result."""
    g = torch.Generator().manual_seed(3)
    W = (torch.randn(E, N, K, generator=g) * 0.1).bfloat16().to(DEV).permute(0, 2, 1)
    X = torch.randn(T, K, generator=g).bfloat16().to(DEV)
    experts = torch.topk(torch.randn(T, E, generator=g), k).indices.to(DEV)

    def step():
        eid, idx, off = sm.flatten_sort_count(experts, E)
        return ops.scatter2scatter(X, W, eid, idx, k, expert_offsets=off)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = step()
    for r in range(3):
        X.copy_(torch.randn(T, K, generator=g).bfloat16())
        experts.copy_(torch.topk(torch.randn(T, E, generator=g), k).indices)
        graph.replay()
        torch.cuda.synchronize()
        got = y_static.clone()
        want = step()
        torch.cuda.synchronize()
        assert torch.equal(got, want), "replay %d differs from the eager result" % r


def test_s2s_strided_rows():
    """X and Y that are column slices of wider buffers (row stride != width)."""
    T, E, k, K, N = 600, 8, 2, 128, 256
    experts, (eid, idx, off) = _routing(T, E, k, seed=1)
    g = torch.Generator().manual_seed(2)
    Xw = torch.randn(T, K + 64, generator=g).bfloat16()
    W = (torch.randn(E, K, N, generator=g) * 0.1).bfloat16()
    want = oracle.scatter2scatter_ref(Xw[:, 32:32 + K].float(), W.float(), eid, idx, k)
    Yw = torch.zeros(T * k, N + 16, dtype=torch.bfloat16, device=DEV)
    ops.scatter2scatter(Xw.to(DEV)[:, 32:32 + K], W.to(DEV), eid.to(DEV), idx.to(DEV), k, out=Yw[:, 8:8 + N])
    _close(Yw[:, 8:8 + N], want, scale=0.1 * K ** 0.5)
    assert not Yw[:, :8].any() and not Yw[:, 8 + N:].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("out_layout", ["param", "plain"])
@pytest.mark.parametrize("T,E,k,K,N", [(4096, 8, 2, 512, 256), (1100, 8, 2, 200, 264), (130, 8, 3, 448, 72),
                                       (2048, 32, 4, 192, 328), (700, 4, 1, 1024, 520)])
def test_xty(T, E, k, K, N, out_layout, dtype):
    experts, (eid, idx, off) = _routing(T, E, k, seed=N, skew=2.0 if E == 32 else 0.0, empty=(1,) if E == 32 else ())
    g = torch.Generator().manual_seed(K)
    L = T * k
    X = torch.randn(L, K, generator=g).to(dtype)
    DY = (torch.randn(L, N, generator=g) * 0.1).to(dtype)
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.float(), X.float(), off, E, has_bias=True)
    rows = torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)).max().item()
    if out_layout == "param":
        DW, Db = ops.group_bwd_W(DY.to(DEV), X.to(DEV), off.to(DEV), E, has_bias=True)
        assert DW.permute(0, 2, 1).is_contiguous()
    else:                                         # (E, K, N)-contiguous output through the raw op
        DW = torch.full((E, K, N), float("nan"), dtype=dtype, device=DEV)
        Db = torch.full((E, N), float("nan"), dtype=dtype, device=DEV)
        ops._xty_launch(E, DW, Db, DY.to(DEV), X.to(DEV), off.to(DEV))
    _close(DW, DW_ref, scale=0.1 * rows ** 0.5)
    _close(Db, Db_ref, scale=0.1 * rows ** 0.5)
    for e in (torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)) == 0).nonzero().flatten().tolist():
        assert not DW[e].any() and not Db[e].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("out_layout,has_bias", [("param", False), ("plain", False), ("plain", True)])
def test_xty_long_segments(out_layout, has_bias, dtype):
    """From 2048 rows per expert on average the weight gradient runs on the one-wave-per-SIMD form (unless the bias
    gradient rides along in the main loop): ragged segment lengths (the last slice of a segment is zero-filled by the
    loads themselves), an expert without rows, partial tiles in both output directions."""
    T, E, K, N = 13000, 4, 264, 520
    experts, (eid, idx, off) = _routing(T, E, 1, seed=17, skew=0.7, empty=(1,))
    g = torch.Generator().manual_seed(18)
    X = torch.randn(T, K, generator=g).to(dtype)
    DY = (torch.randn(T, N, generator=g) * 0.1).to(dtype)
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.float(), X.float(), off, E, has_bias=has_bias)
    counts = torch.diff(off, prepend=torch.zeros(1, dtype=torch.long))
    assert int(counts.min()) == 0 and int((counts % 64 != 0).sum()) >= 2
    if out_layout == "param":
        DW, Db = ops.group_bwd_W(DY.to(DEV), X.to(DEV), off.to(DEV), E, has_bias=has_bias)
    else:
        DW = torch.full((E, K, N), float("nan"), dtype=dtype, device=DEV)
        Db = torch.full((E, N), float("nan"), dtype=dtype, device=DEV) if has_bias else None
        ops._xty_launch(E, DW, Db, DY.to(DEV), X.to(DEV), off.to(DEV))
    _close(DW, DW_ref, scale=0.1 * int(counts.max()) ** 0.5)
    if has_bias:
        _close(Db, Db_ref, scale=0.1 * int(counts.max()) ** 0.5)
    assert not DW[1].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("out_layout", ["param", "plain"])
@pytest.mark.parametrize("T,E,k,K,N", [(4096, 8, 2, 512, 256), (1100, 8, 2, 200, 264), (130, 8, 3, 448, 72),
                                       (2048, 32, 4, 192, 328), (700, 4, 1, 1024, 520), (3, 4, 2, 64, 64)])
def test_xty_reads_tokens_through_the_index(T, E, k, K, N, out_layout, dtype):
    """`group_bwd_W(..., gather=(idx, k))` - the weight gradient that picks the rows of the token matrix itself -
    gives the bits of `group_bwd_W(DY, group(X, idx, fan_out=k), ...)`, the pair of the reference
    (parallel_experts.py:95-107), in both output layouts, with bias gradient, ragged and empty experts; float32
    (no gathering kernel) takes the grouped copy by itself.  And both agree with the oracle."""
    experts, (eid, idx, off) = _routing(T, E, k, seed=N + 1, skew=2.0 if E == 32 else 0.0, empty=(1,) if E == 32 else ())
    g = torch.Generator().manual_seed(K + 1)
    X = torch.randn(T, K, generator=g).to(dtype)
    DY = (torch.randn(T * k, N, generator=g) * 0.1).to(dtype)
    like = None if out_layout == "param" else torch.empty(E, K, N, dtype=dtype, device=DEV)
    Xd, DYd, idxd, offd = X.to(DEV), DY.to(DEV), idx.to(DEV), off.to(DEV)
    DW, Db = ops.group_bwd_W(DYd, Xd, offd, E, has_bias=True, like=like, gather=(idxd, k))
    DW2, Db2 = ops.group_bwd_W(DYd, ops.group(Xd, idxd, fan_out=k), offd, E, has_bias=True, like=like)
    assert DW.stride() == DW2.stride()
    assert torch.equal(DW, DW2) and torch.equal(Db, Db2)
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.float(), oracle.group_ref(X, idx, None, k).float(), off, E, has_bias=True)
    rows = torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)).max().item()
    if dtype is not torch.float32:
        _close(DW, DW_ref, scale=0.1 * rows ** 0.5)
        _close(Db, Db_ref, scale=0.1 * rows ** 0.5)
    else:
        torch.testing.assert_close(DW.cpu(), DW_ref, rtol=1e-4, atol=1e-4)
