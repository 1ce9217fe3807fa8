"""GPU parity of each C-ABI entry point against the CPU oracle on identical seeded inputs.
Integer outputs bit-exact; floating point: fp32 rel 1e-4, bf16/fp16 rel 2e-2 / abs 1e-2."""
import itertools

import pytest
import torch

import oracle
from scattermoe_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

TOL = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=2e-2, atol=1e-2),
       torch.float16: dict(rtol=2e-2, atol=1e-2)}


def _close(got, want, dtype, scale=1.0):
    t = TOL[dtype]
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = t["atol"] * scale + t["rtol"] * want.abs()
    assert bool((err <= bound).all()), "max err %g (bound %g)" % (err.max(), bound.flatten()[err.argmax()])


def _experts(T, E, k, seed, skew=False):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    if skew:
        logits = logits - 1.8 * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    return torch.topk(logits, k).indices


# ---------------------------------------------------------------------------------------------------
# routing: bit-exact
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (3, 1, 1), (256, 8, 2), (512, 8, 4), (2048, 8, 2), (2049, 8, 2),
                                   (8192, 32, 4), (32768, 128, 8), (16384, 8, 2), (5000, 300, 3), (70000, 64, 1),
                                   (4096, 512, 8), (2000, 700, 5), (16385, 8, 2), (40000, 2000, 1),
                                   (2048, 512, 8)])      # 16384 rows over 512 experts: the most one workgroup sorts
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_route_bit_exact(T, E, k, dtype):
    experts = _experts(T, E, k, seed=T + E, skew=(E >= 32)).to(dtype)
    eid, idx, off = ops.route(experts.to(DEV), E)
    r_eid, r_idx, r_off = oracle.route_ref(experts, E)
    assert eid.dtype == idx.dtype == off.dtype == torch.int64
    assert torch.equal(eid.cpu(), r_eid) and torch.equal(idx.cpu(), r_idx) and torch.equal(off.cpu(), r_off)
    s_eid, s_idx = torch.sort(experts.flatten().long(), stable=True)
    assert torch.equal(eid.cpu(), s_eid) and torch.equal(idx.cpu(), s_idx)


def test_route_edge_cases():
    flat = torch.full((5000,), 3, dtype=torch.int64)                      # one expert takes everything
    eid, idx, off = ops.route(flat.to(DEV), 6)
    assert torch.equal(idx.cpu(), torch.arange(5000)) and off.tolist() == [0, 0, 0, 5000, 5000, 5000]
    eid, idx, off = ops.route(torch.empty(0, 2, dtype=torch.int64, device=DEV), 4)   # no rows
    assert eid.numel() == 0 and off.tolist() == [0, 0, 0, 0]
    u8 = torch.tensor([[7, 0], [0, 7]], dtype=torch.uint8)
    eid, idx, off = ops.route(u8.to(DEV), 8)
    assert eid.tolist() == [0, 0, 7, 7] and idx.tolist() == [1, 2, 0, 3] and off.tolist() == [2] * 7 + [4]
    a = ops.route(_experts(4096, 16, 4, 1).to(DEV), 16)
    b = ops.route(_experts(4096, 16, 4, 1).to(DEV), 16)
    assert all(torch.equal(x, y) for x, y in zip(a, b))                   # run-to-run identical


def test_offsets_from_sorted():
    for E, L in [(8, 1000), (40, 77), (5, 0), (128, 9000)]:
        eid = torch.sort(torch.randint(0, E, (L,))).values
        if L:
            eid[eid == 1] = 0                                             # an empty expert
            eid = torch.sort(eid).values
        off = ops.offsets_from_sorted(eid.to(DEV), E)
        assert torch.equal(off.cpu(), torch.bincount(eid, minlength=E).cumsum(0))


# ---------------------------------------------------------------------------------------------------
# scatter2scatter
# ---------------------------------------------------------------------------------------------------
S2S_SHAPES = [  # T, E, k, K, N
    (1, 8, 2, 128, 128), (77, 8, 3, 100, 133), (256, 8, 2, 128, 256), (300, 8, 4, 600, 150),
    (512, 16, 2, 64, 72), (1024, 8, 2, 256, 512), (2048, 8, 2, 512, 384),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_layout", ["k_contig", "n_contig"])
@pytest.mark.parametrize("T,E,k,K,N", S2S_SHAPES)
def test_scatter2scatter_forward_layer(T, E, k, K, N, w_layout, dtype):
    g = torch.Generator().manual_seed(K * 7 + N)
    experts = _experts(T, E, k, seed=T)
    eid, idx, off = oracle.route_ref(experts, E)
    X = torch.randn(T, K, generator=g).to(dtype)
    Wp = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)
    W = Wp.permute(0, 2, 1) if w_layout == "k_contig" else Wp.permute(0, 2, 1).contiguous()
    b = torch.randn(E, N, generator=g).to(dtype)
    want = oracle.scatter2scatter_ref(X.float(), W.float(), eid, idx, k, b.float(), False, True)
    Wd = Wp.to(DEV).permute(0, 2, 1) if w_layout == "k_contig" else W.to(DEV)
    got = ops.scatter2scatter(X.to(DEV), Wd, eid.to(DEV), idx.to(DEV), k, b=b.to(DEV), y_grouped=True,
                              expert_offsets=off.to(DEV))
    assert got.dtype == dtype
    _close(got, want, dtype, scale=K ** 0.5 * 0.1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("x_grouped,y_grouped", list(itertools.product([False, True], repeat=2)))
def test_scatter2scatter_grouping_modes(x_grouped, y_grouped, dtype):
    T, E, k, K, N = 700, 8, 2, 256, 192
    g = torch.Generator().manual_seed(12)
    experts = _experts(T, E, k, seed=3, skew=True)
    experts[experts == 5] = 4                                             # expert 5 has no rows
    eid, idx, off = oracle.route_ref(experts, E)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g).to(dtype)
    W = (torch.randn(E, K, N, generator=g) * 0.1).to(dtype)
    want = oracle.scatter2scatter_ref(X.float(), W.float(), eid, idx, fan, None, x_grouped, y_grouped)
    # offsets omitted on purpose: the wrapper derives them from the sorted ids like the reference signature
    got = ops.scatter2scatter(X.to(DEV), W.to(DEV), eid.to(DEV), idx.to(DEV), fan,
                              x_grouped=x_grouped, y_grouped=y_grouped)
    _close(got, want, dtype, scale=K ** 0.5 * 0.1)
    out = torch.full((T * k, N), float("nan"), dtype=dtype, device=DEV)
    ret = ops.scatter2scatter(X.to(DEV), W.to(DEV), eid.to(DEV), idx.to(DEV), fan, x_grouped=x_grouped,
                              y_grouped=y_grouped, out=out)
    assert ret.data_ptr() == out.data_ptr() and torch.equal(ret, got)     # out= is filled completely, deterministically


def test_scatter2scatter_e1_is_plain_gemm():
    T, K, N = 1000, 384, 320
    g = torch.Generator().manual_seed(0)
    X = torch.randn(T, K, generator=g)
    W = torch.randn(1, K, N, generator=g) * 0.05
    eid, idx, off = oracle.route_ref(torch.zeros(T, 1, dtype=torch.long), 1)
    got = ops.scatter2scatter(X.to(DEV), W.to(DEV), eid.to(DEV), idx.to(DEV), 1)
    _close(got, X @ W[0], torch.float32, scale=K ** 0.5 * 0.05)


# ---------------------------------------------------------------------------------------------------
# group
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,K", [(1, 2, 128), (333, 3, 100), (1024, 2, 4096), (257, 4, 72)])
@pytest.mark.parametrize("with_coeff", [False, True])
def test_group_bit_exact(T, k, K, with_coeff, dtype):
    g = torch.Generator().manual_seed(T + K)
    experts = _experts(T, 8, k, seed=K)
    _, idx, _ = oracle.route_ref(experts, 8)
    A = torch.randn(T, K, generator=g).to(dtype)
    coeff = torch.rand(T, k, generator=g).to(dtype) if with_coeff else None
    want = oracle.group_ref(A, idx, None if coeff is None else coeff.flatten(), fan_out=k)
    got = ops.group(A.to(DEV), idx.to(DEV), coeff=None if coeff is None else coeff.flatten().to(DEV), fan_out=k)
    assert torch.equal(got.cpu(), want)          # a copy with one correctly rounded product: bit-exact
    sub = torch.randn(T, K + 8, generator=g).to(dtype)                    # strided source rows
    got2 = ops.group(sub.to(DEV)[:, 3:K + 3], idx.to(DEV), fan_out=k)
    assert torch.equal(got2.cpu(), oracle.group_ref(sub[:, 3:K + 3], idx, None, k))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,K", [(1, 2, 64), (300, 8, 2048), (777, 4, 2880), (64, 64, 520), (200, 2, 4096 + 64),
                                   (50, 3, 100)])
def test_group_walked_by_source_row(T, k, K, dtype):
    """`permutation=True` reads every source row once and writes its k scaled copies through the inverse
    permutation: the oracle's values and the same bits as the gather, for rows longer than one pass of a wave
    (more than 2048 16-bit columns), row lengths that are no multiple of a pass, k up to a whole wave, and row
    lengths the 16-byte path does not take (the call then falls back to the gather)."""
    g = torch.Generator().manual_seed(T * k + K)
    experts = torch.stack([torch.randperm(max(k, 8), generator=g)[:k] for _ in range(T)])
    _, idx, _ = oracle.route_ref(experts, max(k, 8))
    A = torch.randn(T, K, generator=g).to(dtype)
    coeff = torch.rand(T * k, generator=g).to(dtype)
    want = oracle.group_ref(A, idx, coeff, fan_out=k)
    out = torch.full((T * k + 2, K), float("nan"), dtype=dtype, device=DEV)      # a guard row on either side
    got = ops.group(A.to(DEV), idx.to(DEV), coeff=coeff.to(DEV), fan_out=k, out=out[1:-1], permutation=True)
    assert torch.equal(got.cpu(), want)
    assert bool(torch.isnan(out[0]).all()) and bool(torch.isnan(out[-1]).all())
    assert torch.equal(got, ops.group(A.to(DEV), idx.to(DEV), coeff=coeff.to(DEV), fan_out=k))


def test_group_walked_by_source_row_skips_what_is_not_a_permutation():
    """An index vector with a repeated and an out-of-range entry, and a workspace full of stale values: rows whose
    index entry is theirs alone get the gather's values, and nothing is written outside Y."""
    import ctypes
    from scattermoe_amd import _C
    T, k, K = 40, 4, 256
    L = T * k
    g = torch.Generator().manual_seed(5)
    idx = torch.randperm(L, generator=g)
    idx[7] = idx[3]                       # slot idx[3] claimed twice, the slot that row 7 had by nobody
    idx[11] = L + 5                       # out of range
    A = torch.randn(T, K, generator=g).bfloat16().to(DEV)
    coeff = torch.rand(L, generator=g).bfloat16().to(DEV)
    Y = torch.full((L + 2, K), float("nan"), dtype=torch.bfloat16, device=DEV)
    inv = torch.randint(-2 ** 31, 2 ** 31 - 1, (L,), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
    lib = _C.load()
    idx_d = idx.to(DEV)
    rc = lib.smoe_group_by_source(_C.ptr(A), A.stride(0), 1, _C.ptr(coeff), _C.ptr(Y[1:]), K, 1, _C.ptr(idx_d),
                                  _C.ptr(inv), L, K, k, _C.float_code(A.dtype), _C.stream_ptr(A.device))
    assert rc == 0
    torch.cuda.synchronize()
    got = Y[1:-1].cpu()
    sure = [r for r in range(L) if r not in (3, 7, 11)]
    want = (A.cpu().float()[idx[sure] // k] * coeff.cpu().float()[idx[sure]].unsqueeze(1)).bfloat16()
    assert torch.equal(got[sure], want)
    assert bool(torch.isnan(got[11]).all())                          # its slot does not exist
    assert bool(torch.isnan(got[3]).all()) != bool(torch.isnan(got[7]).all())      # one of the two claimants wins
    assert bool(torch.isnan(Y[0]).all()) and bool(torch.isnan(Y[-1]).all())


# ---------------------------------------------------------------------------------------------------
# groupXtY
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,K,N", [(1, 8, 2, 128, 128), (77, 8, 3, 100, 133), (512, 8, 2, 256, 128),
                                       (1500, 16, 2, 192, 320), (2048, 4, 2, 512, 256)])
def test_group_bwd_W(T, E, k, K, N, dtype):
    g = torch.Generator().manual_seed(N + 3 * K)
    experts = _experts(T, E, k, seed=T + 1, skew=True)
    eid, idx, off = oracle.route_ref(experts, E)
    L = T * k
    X = torch.randn(L, K, generator=g).to(dtype)
    DY = (torch.randn(L, N, generator=g) * 0.1).to(dtype)
    DW_ref, Db_ref = oracle.group_bwd_W_ref(DY.float(), X.float(), off, E, has_bias=True)
    DW, Db = ops.group_bwd_W(DY.to(DEV), X.to(DEV), off.to(DEV), E, has_bias=True)
    assert DW.shape == (E, K, N) and DW.permute(0, 2, 1).is_contiguous() and Db.shape == (E, N)
    rows = torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)).max().item()
    _close(DW, DW_ref, dtype, scale=rows ** 0.5 * 0.1)
    _close(Db, Db_ref, dtype, scale=rows ** 0.5 * 0.1)
    empty = (torch.diff(off, prepend=torch.zeros(1, dtype=torch.long)) == 0).nonzero().flatten()
    for e in empty.tolist():
        assert not DW[e].any() and not Db[e].any()                        # written as exact zeros
    DW2, _ = ops.group_bwd_W(DY.to(DEV), X.to(DEV), off.to(DEV), E, has_bias=False)
    assert torch.equal(DW2, DW)                                           # fixed summation order


# ---------------------------------------------------------------------------------------------------
# fused passes: combine, gate gradient, gated linear unit
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,N", [(1, 2, 128), (300, 3, 100), (1024, 2, 4096), (77, 8, 264), (50, 1, 64)])
def test_combine_and_gate_grad(T, k, N, dtype):
    g = torch.Generator().manual_seed(T + N)
    Y = torch.randn(T, k, N, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).to(dtype)
    dO = torch.randn(T, N, generator=g).to(dtype)
    want = (Y.float() * gates.float().unsqueeze(-1)).sum(1)
    got = ops.combine(Y.to(DEV), gates.to(DEV))
    _close(got, want, dtype, scale=k ** 0.5)
    want_g = (Y.float() * dO.float().unsqueeze(1)).sum(-1)
    got_g = ops.gate_grad(Y.to(DEV), dO.to(DEV))
    _close(got_g, want_g, dtype, scale=N ** 0.5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,N,E", [(1, 2, 128, 4), (300, 3, 104, 8), (1024, 2, 4096, 8), (77, 8, 264, 32),
                                     (50, 1, 64, 4), (513, 4, 2880, 32), (40, 2, 100, 4)])
def test_gate_grad_and_scaled_gather_in_one_pass(T, k, N, E, dtype):
    """`gate_grad_group` = `gate_grad` + `group(grad_out, idx, coeff=gates, fan_out=k)` over one read of grad_out:
    the gathered rows bit-exact against the oracle's group (one rounding of the product), the gate gradient against
    the float32 row dots; rows longer than one pass of a wave (4096, 2880), rows that are no whole 16-byte pieces
    (N = 100 with 16-bit types: the two separate passes run instead)."""
    g = torch.Generator().manual_seed(T + N + k)
    experts = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    _, idx, _ = oracle.route_ref(experts, E)
    Y = torch.randn(T, k, N, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).to(dtype)
    dO = torch.randn(T, N, generator=g).to(dtype)
    d_gates, dy = ops.gate_grad_group(Y.to(DEV), dO.to(DEV), gates.to(DEV), idx.to(DEV))
    want_dy = oracle.group_ref(dO, idx, gates.reshape(-1), k)
    assert torch.equal(dy.cpu(), want_dy)
    want_g = (Y.float() * dO.float().unsqueeze(1)).sum(-1)
    _close(d_gates, want_g, dtype, scale=N ** 0.5)
    again = ops.gate_grad_group(Y.to(DEV), dO.to(DEV), gates.to(DEV), idx.to(DEV))
    assert torch.equal(again[0], d_gates) and torch.equal(again[1], dy)           # fixed summation order


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,f", [(1, 128), (333, 100), (4096, 768), (64, 2880)])
def test_glu_fwd_bwd(rows, f, dtype):
    g = torch.Generator().manual_seed(rows + f)
    pre = torch.randn(rows, 2 * f, generator=g).to(dtype)
    dh = torch.randn(rows, f, generator=g).to(dtype)
    ref_in = pre.float().requires_grad_()
    lin, gate = ref_in.chunk(2, dim=-1)
    h_ref = torch.nn.functional.silu(gate) * lin
    h_ref.backward(dh.float())
    h = ops.glu_fwd(pre.to(DEV))
    dpre = ops.glu_bwd(pre.to(DEV), dh.to(DEV))
    _close(h, h_ref.detach(), dtype, scale=0.1)
    _close(dpre, ref_in.grad, dtype, scale=0.1)


# ---------------------------------------------------------------------------------------------------
# gpt-oss gated unit: one pass each way against the oracle's chain of torch ops (fp32) and its autograd gradient
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,f", [(1, 4), (37, 50), (300, 2880), (64, 1001)])
def test_gpt_oss_glu(rows, f, dtype):
    g = torch.Generator().manual_seed(rows + f)
    pre = (torch.randn(rows, 2 * f, generator=g) * 4).to(dtype)      # +-4 sigma: both clamps (limit 7) are hit
    pre[0, :4] = torch.tensor([7.0, 7.0, 7.0, -7.0]).to(dtype)       # exactly on the bounds: gradient passes
    dh = torch.randn(rows, f, generator=g).to(dtype)
    ref_in = pre.float().requires_grad_()
    want = oracle.gpt_oss_glu(1.702, 7.0)(ref_in)
    (want_grad,) = torch.autograd.grad(want, ref_in, dh.float())
    x = pre.to(DEV).detach().requires_grad_()
    got = ops.gpt_oss_glu(x, 1.702, 7.0)
    (got_grad,) = torch.autograd.grad(got, x, dh.to(DEV))
    want = want.detach()
    _close(got.detach(), want, dtype, scale=max(1.0, float(want.abs().max())))
    _close(got_grad, want_grad, dtype, scale=max(1.0, float(want_grad.abs().max())))
    # strided rows (a column slice of a wider buffer)
    wide = torch.zeros(rows, 2 * f + 6, dtype=dtype, device=DEV)
    wide[:, :2 * f] = pre.to(DEV)
    _close(ops.gpt_oss_glu(wide[:, :2 * f], 1.702, 7.0), want, dtype, scale=max(1.0, float(want.abs().max())))


# ---------------------------------------------------------------------------------------------------
# sum over the k slots of a token (the `.sum(-2)` of reference parallel_experts.py:120-123): float32 accumulation
# in slot order, one rounding -> bit-exact against that very sequence written with torch ops
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,k,N", [(1, 2, 8), (37, 4, 100), (1000, 8, 2048), (513, 3, 2880), (64, 1, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_slot_sum_bit_exact(T, k, N, dtype):
    g = torch.Generator().manual_seed(T + k + N)
    y = torch.randn(T * k, N, generator=g).to(dtype)
    got = ops.slot_sum(y.to(DEV), T, k)
    acc = torch.zeros(T, N)
    for j in range(k):
        acc = acc + y.view(T, k, N)[:, j].float()
    assert got.shape == (T, N) and got.dtype == dtype
    assert torch.equal(got.cpu(), acc.to(dtype))
    if k > 1:     # and within rounding of the library reduction the reference calls
        _close(got, y.view(T, k, N).float().sum(-2), dtype, scale=float(k) ** 0.5)


def test_mfma_rate_probe_launches():
    """The measurement aid behind bench.py's `mfma_sustained` (a library of its own beside the product library):
    launches, reports its flop count, and its sums are what the operands say (zeros stay zero; 16-deep products of
    values below 2 stay finite)."""
    import ctypes
    from scattermoe_amd import _build
    lib = ctypes.CDLL(_build.PROBE_LIB_PATH)
    fn = lib.smoe_bench_mfma_rate
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    out = torch.full((65536,), float("nan"), device=DEV)
    flop = ctypes.c_double(0.0)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert fn(out.data_ptr(), 3, 0, ctypes.byref(flop), st) == 0
    torch.cuda.synchronize()
    assert flop.value == 1024 * 3 * 64 * 2.0 * 32 * 32 * 16
    assert bool((out == 0).all())
    assert fn(None, 3, 1, ctypes.byref(flop), st) == -1
    assert fn(out.data_ptr(), 0, 1, ctypes.byref(flop), st) == -5
    assert fn(out.data_ptr(), 3, 1, ctypes.byref(flop), st) == 0
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and float(out.abs().max()) > 0
