"""Pins the CPU oracle against facts that do not depend on its own formulas: brute-force loops over
Python floats, closed forms, finite-difference gradients and Hugging Face's independent expert loops.
The reference keeps no golden vectors (tests/test_mlp.py draws unseeded inputs), so these are the pins."""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

import oracle


def _rand_routing(T, E, k, seed):
    g = torch.Generator().manual_seed(seed)
    probs = torch.softmax(torch.randn(T, E, generator=g), -1)
    p, experts = torch.topk(probs, k)
    return p, experts


# ---------------------------------------------------------------------------------------------------
# routing
# ---------------------------------------------------------------------------------------------------
def _route_bruteforce(flat, E):
    pairs = []
    for e in range(E):                      # expert-major, original position ascending = stable order
        for pos, v in enumerate(flat):
            if v == e:
                pairs.append((e, pos))
    counts = [sum(1 for v in flat if v == e) for e in range(E)]
    off, run = [], 0
    for c in counts:
        run += c
        off.append(run)
    return [p[0] for p in pairs], [p[1] for p in pairs], off


@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (5, 3, 2), (17, 8, 3), (64, 4, 4), (9, 1, 1), (33, 16, 2)])
def test_route_bruteforce(T, E, k):
    _, experts = _rand_routing(T, E, k, seed=T * 131 + E)
    eid, idx, off = oracle.route_ref(experts, E)
    b_eid, b_idx, b_off = _route_bruteforce(experts.flatten().tolist(), E)
    assert eid.tolist() == b_eid and idx.tolist() == b_idx and off.tolist() == b_off
    assert eid.dtype == idx.dtype == off.dtype == torch.int64


def test_route_invariants_and_torch_stable_sort():
    g = torch.Generator().manual_seed(3)
    flat = torch.randint(0, 7, (4099,), generator=g)
    flat[flat == 5] = 4                      # expert 5 stays empty
    eid, idx, off = oracle.route_ref(flat, 7)
    s_eid, s_idx = torch.sort(flat, stable=True)
    assert torch.equal(eid, s_eid) and torch.equal(idx, s_idx)
    assert torch.equal(off, torch.bincount(flat, minlength=7).cumsum(0))
    assert torch.equal(torch.sort(idx).values, torch.arange(flat.numel()))        # permutation
    assert torch.equal(flat[idx], eid) and bool((eid[1:] >= eid[:-1]).all())
    same = eid[1:] == eid[:-1]
    assert bool((idx[1:][same] > idx[:-1][same]).all())                          # stable inside a segment
    assert off[-1] == flat.numel() and off[5] == off[4]


def test_route_special_cases():
    assert [t.tolist() for t in oracle.route_ref(torch.tensor([[2]]), 4)] == [[2], [0], [0, 0, 1, 1]]
    eid, idx, off = oracle.route_ref(torch.full((6, 2), 3), 5)                   # everything to one expert
    assert eid.tolist() == [3] * 12 and idx.tolist() == list(range(12)) and off.tolist() == [0, 0, 0, 12, 12]
    eid, idx, off = oracle.route_ref(torch.tensor([1, 0, 1, 0], dtype=torch.int32), 2)  # flat, int32 input
    assert eid.tolist() == [0, 0, 1, 1] and idx.tolist() == [1, 3, 0, 2] and off.tolist() == [2, 4]


# ---------------------------------------------------------------------------------------------------
# kernel models vs brute force
# ---------------------------------------------------------------------------------------------------
def _s2s_bruteforce(X, W, eid, idx, k, b, x_grouped, y_grouped):
    L, K, N = len(eid), len(X[0]), len(W[0][0])
    Y = [[0.0] * N for _ in range(L)]
    for n in range(L):
        e = eid[n]
        src = n if x_grouped else idx[n] // k
        dst = n if y_grouped else idx[n]
        for j in range(N):
            s = math.fsum(X[src][c] * W[e][c][j] for c in range(K))
            Y[dst][j] = s + (b[e][j] if b is not None else 0.0)
    return Y


@pytest.mark.parametrize("x_grouped,y_grouped", list(itertools.product([False, True], repeat=2)))
@pytest.mark.parametrize("bias", [False, True])
def test_scatter2scatter_bruteforce(x_grouped, y_grouped, bias):
    T, E, k, K, N = 7, 3, 2, 5, 4
    g = torch.Generator().manual_seed(11)
    _, experts = _rand_routing(T, E, k, seed=5)
    eid, idx, _ = oracle.route_ref(experts, E)
    fan = 1 if x_grouped else k
    X = torch.randn(T * k // fan, K, generator=g, dtype=torch.float64)
    W = torch.randn(E, K, N, generator=g, dtype=torch.float64)
    b = torch.randn(E, N, generator=g, dtype=torch.float64) if bias else None
    got = oracle.scatter2scatter_ref(X, W, eid, idx, fan, b, x_grouped, y_grouped, acc=torch.float64)
    want = _s2s_bruteforce(X.tolist(), W.tolist(), eid.tolist(), idx.tolist(), fan,
                           None if b is None else b.tolist(), x_grouped, y_grouped)
    assert torch.allclose(got, torch.tensor(want, dtype=torch.float64), atol=1e-12, rtol=0)


def test_scatter2scatter_closed_forms():
    g = torch.Generator().manual_seed(2)
    T, k, K, N = 6, 2, 4, 4
    # E = 1: a plain linear layer applied to every (token, slot) row
    X = torch.randn(T, K, generator=g)
    W = torch.randn(1, K, N, generator=g)
    eid, idx, _ = oracle.route_ref(torch.zeros(T, k, dtype=torch.long), 1)
    Y = oracle.scatter2scatter_ref(X, W, eid, idx, k)
    assert torch.allclose(Y, F.linear(X, W[0].T).repeat_interleave(k, 0), atol=1e-6)
    # identity weights copy the routed token into its slot row; a strided (transposed) W view is honoured
    _, experts = _rand_routing(T, 3, k, seed=9)
    eid, idx, _ = oracle.route_ref(experts, 3)
    eye = torch.eye(K).expand(3, K, K)
    assert torch.equal(oracle.scatter2scatter_ref(X, eye, eid, idx, k), X.repeat_interleave(k, 0))
    Wt = torch.randn(3, N, K, generator=g)
    a = oracle.scatter2scatter_ref(X, Wt.permute(0, 2, 1), eid, idx, k)
    b = oracle.scatter2scatter_ref(X, Wt.permute(0, 2, 1).contiguous(), eid, idx, k)
    assert torch.allclose(a, b, atol=1e-6)
    # one-hot rows pick out row c of the routed expert's matrix
    Xh = torch.zeros(T, K); Xh[:, 2] = 1.0
    Yh = oracle.scatter2scatter_ref(Xh, Wt.permute(0, 2, 1), eid, idx, k)
    assert torch.equal(Yh, Wt[experts.flatten(), :, 2])


def test_group_and_group_bwd_W_bruteforce():
    g = torch.Generator().manual_seed(4)
    T, E, k, K, N = 9, 4, 2, 3, 5
    p, experts = _rand_routing(T, E, k, seed=8)
    experts[experts == 2] = 1                                   # expert 2 empty
    eid, idx, off = oracle.route_ref(experts, E)
    A = torch.randn(T, K, generator=g, dtype=torch.float64)
    coeff = p.double()
    got = oracle.group_ref(A, idx, coeff.flatten(), fan_out=k)
    for n in range(T * k):
        i = int(idx[n])
        assert torch.allclose(got[n], A[i // k] * coeff.flatten()[i], atol=1e-15)
    assert torch.equal(oracle.group_ref(A, idx, None, fan_out=k), A[idx // k])
    Xg = torch.randn(T * k, K, generator=g, dtype=torch.float64)
    DY = torch.randn(T * k, N, generator=g, dtype=torch.float64)
    DW, Db = oracle.group_bwd_W_ref(DY, Xg, off, E, has_bias=True, acc=torch.float64)
    for e in range(E):
        rows = [n for n in range(T * k) if int(eid[n]) == e]
        for c in range(K):
            for j in range(N):
                want = math.fsum(float(Xg[r, c]) * float(DY[r, j]) for r in rows)
                assert abs(float(DW[e, c, j]) - want) < 1e-12
        for j in range(N):
            assert abs(float(Db[e, j]) - math.fsum(float(DY[r, j]) for r in rows)) < 1e-12
    assert not DW[2].any() and not Db[2].any()


# ---------------------------------------------------------------------------------------------------
# the naive MoE MLP
# ---------------------------------------------------------------------------------------------------
def _mlp_bruteforce(x, p, experts, W1, W2, b1, b2, act):
    T, k = len(experts), len(experts[0])
    out = []
    for t in range(T):
        y = [0.0] * len(W2[0])
        for j in range(k):
            e = experts[t][j]
            h = [act(math.fsum(W1[e][r][c] * x[t][c] for c in range(len(x[t]))) + (b1[e][r] if b1 else 0.0))
                 for r in range(len(W1[e]))]
            for o in range(len(W2[e])):
                v = math.fsum(W2[e][o][r] * h[r] for r in range(len(h))) + (b2[e][o] if b2 else 0.0)
                y[o] += p[t][j] * v
        out.append(y)
    return out


@pytest.mark.parametrize("bias", [False, True])
def test_naive_forms_vs_bruteforce(bias):
    g = torch.Generator().manual_seed(21)
    T, E, k, d, f = 5, 3, 2, 4, 6
    p, experts = _rand_routing(T, E, k, seed=1)
    p = p.double()
    x = torch.randn(T, d, generator=g, dtype=torch.float64)
    W1 = torch.randn(E, f, d, generator=g, dtype=torch.float64)
    W2 = torch.randn(E, d, f, generator=g, dtype=torch.float64)
    b1 = torch.randn(E, f, generator=g, dtype=torch.float64) if bias else None
    b2 = torch.randn(E, d, generator=g, dtype=torch.float64) if bias else None
    want = torch.tensor(_mlp_bruteforce(x.tolist(), p.tolist(), experts.tolist(), W1.tolist(), W2.tolist(),
                                        b1.tolist() if bias else None, b2.tolist() if bias else None,
                                        math.tanh), dtype=torch.float64)
    a = oracle.naive_token_forward(x, p, experts, W1, W2, torch.tanh, b1, b2)
    b = oracle.naive_expert_forward(x, p, experts, W1, W2, torch.tanh, b1, b2)
    assert torch.allclose(a, want, atol=1e-12) and torch.allclose(b, want, atol=1e-12)


def test_token_form_equals_expert_form_c1_shape():
    from _inputs import CONFIGS, make_inputs
    cfg = CONFIGS["c1"]
    t = make_inputs(cfg)
    act = torch.nn.GELU()
    a = oracle.naive_token_forward(t["x"][:64], t["p"][:64], t["experts"][:64], t["W1"], t["W2"], act)
    b = oracle.naive_expert_forward(t["x"][:64], t["p"][:64], t["experts"][:64], t["W1"], t["W2"], act)
    assert torch.allclose(a, b, atol=1e-6)


def test_glu_split_convention():
    pre = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    # first half linear, second half activated
    assert torch.allclose(oracle.glu(torch.tanh)(pre), torch.tanh(pre[:, 2:]) * pre[:, :2])
    pre = torch.tensor([[0.5, 9.0, -8.0, -9.0]])
    gate, up = torch.tensor([0.5, -8.0]), torch.tensor([7.0, -7.0])          # interleaved + clamped
    want = (up + 1) * gate * torch.sigmoid(1.702 * gate)
    assert torch.allclose(oracle.gpt_oss_glu()(pre), want[None])


def test_naive_expert_forward_gradcheck():
    g = torch.Generator().manual_seed(5)
    T, E, k, d, f = 4, 3, 2, 3, 4
    p, experts = _rand_routing(T, E, k, seed=2)
    args = [torch.randn(T, d, generator=g, dtype=torch.float64), p.double(),
            torch.randn(E, 2 * f, d, generator=g, dtype=torch.float64),
            torch.randn(E, d, f, generator=g, dtype=torch.float64),
            torch.randn(E, 2 * f, generator=g, dtype=torch.float64),
            torch.randn(E, d, generator=g, dtype=torch.float64)]
    for a in args:
        a.requires_grad_()
    fn = lambda x, p_, W1, W2, b1, b2: oracle.naive_expert_forward(
        x, p_, experts, W1, W2, oracle.glu(F.silu), b1, b2)
    assert torch.autograd.gradcheck(fn, args, eps=1e-6, atol=1e-5)


def test_against_huggingface_expert_loops():
    """Independent implementations: transformers' MixtralExperts / GptOssExperts forward loops."""
    mixtral = pytest.importorskip("transformers.models.mixtral.modeling_mixtral")
    gptoss = pytest.importorskip("transformers.models.gpt_oss.modeling_gpt_oss")
    from transformers import MixtralConfig, GptOssConfig
    T, E, k, d, f = 12, 4, 2, 8, 16
    p, experts = _rand_routing(T, E, k, seed=6)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, d, generator=g)

    m = mixtral.MixtralExperts(MixtralConfig(hidden_size=d, intermediate_size=f, num_local_experts=E,
                                             num_experts_per_tok=k, hidden_act="silu"))
    with torch.no_grad():
        m.gate_up_proj.copy_(torch.randn(E, 2 * f, d, generator=g) * 0.3)
        m.down_proj.copy_(torch.randn(E, d, f, generator=g) * 0.3)
        want = m(x, experts, p)
        # HF: act(first half) * second half; the oracle's GLU: act(second half) * first half
        gate, up = m.gate_up_proj.chunk(2, dim=1)
        got = oracle.naive_expert_forward(x, p, experts, torch.cat([up, gate], 1), m.down_proj, oracle.glu(F.silu))
    assert torch.allclose(got, want, atol=1e-5)

    o = gptoss.GptOssExperts(GptOssConfig(hidden_size=d, intermediate_size=f, num_local_experts=E,
                                          num_experts_per_tok=k))
    with torch.no_grad():
        o.gate_up_proj.copy_(torch.randn(E, d, 2 * f, generator=g) * 0.5)
        o.gate_up_proj_bias.copy_(torch.randn(E, 2 * f, generator=g))
        o.down_proj.copy_(torch.randn(E, f, d, generator=g) * 0.5)
        o.down_proj_bias.copy_(torch.randn(E, d, generator=g))
        want = o(x, experts, p)
        got = oracle.naive_expert_forward(x, p, experts, o.gate_up_proj.transpose(1, 2), o.down_proj.transpose(1, 2),
                                          oracle.gpt_oss_glu(o.alpha, o.limit), o.gate_up_proj_bias, o.down_proj_bias)
    assert torch.allclose(got, want, atol=1e-5)


# ---------------------------------------------------------------------------------------------------
# router front end
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (33, 8, 2), (64, 32, 4), (17, 128, 8), (5, 300, 3), (4, 4, 4)])
@pytest.mark.parametrize("renorm", [True, False])
def test_topk_softmax_matches_library_routines(T, E, k, renorm):
    logits = torch.randn(T, E, generator=torch.Generator().manual_seed(T * E + k)) * 3
    w, i = oracle.topk_softmax_ref(logits, k, renorm)
    p = torch.softmax(logits.float(), dim=-1)
    tw, ti = torch.topk(p, k, dim=-1)
    if renorm:
        tw = tw / tw.sum(-1, keepdim=True)
    assert torch.equal(i, ti)                       # random floats: no ties, so the order is fixed
    torch.testing.assert_close(w, tw, rtol=1e-5, atol=1e-7)


def test_topk_softmax_hand_worked_and_ties():
    # logits ln(1), ln(2), ln(3), ln(4): probabilities 0.1 .. 0.4
    logits = torch.log(torch.tensor([[1.0, 2.0, 3.0, 4.0]]))
    w, i = oracle.topk_softmax_ref(logits, 2, renormalize=False)
    assert i.tolist() == [[3, 2]]
    torch.testing.assert_close(w, torch.tensor([[0.4, 0.3]]), rtol=1e-6, atol=0)
    w, i = oracle.topk_softmax_ref(logits, 2, renormalize=True)
    torch.testing.assert_close(w, torch.tensor([[4 / 7, 3 / 7]]), rtol=1e-6, atol=0)
    # all equal: lowest ids first, uniform weights; shifting the logits changes nothing
    w, i = oracle.topk_softmax_ref(torch.zeros(2, 6), 3, renormalize=False)
    assert i.tolist() == [[0, 1, 2]] * 2 and torch.allclose(w, torch.full((2, 3), 1 / 6))
    a = oracle.topk_softmax_ref(logits + 50.0, 3)
    b = oracle.topk_softmax_ref(logits, 3)
    assert torch.equal(a[1], b[1]) and torch.allclose(a[0], b[0], rtol=1e-5)
    # k = E without renormalisation is the whole softmax, sorted
    w, i = oracle.topk_softmax_ref(logits, 4, renormalize=False)
    assert abs(float(w.sum()) - 1.0) < 1e-6 and i.tolist() == [[3, 2, 1, 0]]


# ---------------------------------------------------------------------------------------------------
# the hand-written forward + backward with storage-type rounding: without rounding (float32) it must be the autograd
# gradient of the naive forms; with rounding it must stay within the format's error of them
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bias", [False, True])
def test_rounded_step_without_rounding_is_autograd_of_the_naive_forms(bias):
    g = torch.Generator().manual_seed(5)
    T, d, f, E, k = 40, 24, 16, 4, 2
    x, dy = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g)
    experts = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    p = torch.rand(T, k, generator=g)
    W1, W2 = torch.randn(E, 2 * f, d, generator=g) * 0.3, torch.randn(E, d, f, generator=g) * 0.3
    b1 = torch.randn(E, 2 * f, generator=g) * 0.3 if bias else None
    b2 = torch.randn(E, d, generator=g) * 0.3 if bias else None
    leaves = [t.clone().requires_grad_() for t in (x, p, W1, W2)] + ([b1.clone().requires_grad_(), b2.clone().requires_grad_()] if bias else [])
    want_y = oracle.naive_expert_forward(leaves[0], leaves[1], experts, leaves[2], leaves[3], oracle.glu(torch.nn.SiLU()),
                                         *(leaves[4:] if bias else []))
    grads = torch.autograd.grad(want_y, leaves, dy)
    y, dx, dp = oracle.rounded_glu_token_step(x, p, experts, W1, W2, dy, torch.float32, b1, b2)
    assert torch.allclose(y, want_y.detach(), atol=1e-5)
    assert torch.allclose(dx, grads[0], atol=1e-5) and torch.allclose(dp, grads[1], atol=1e-5)
    S = torch.tensor([1, 5, 6, 15])
    S2 = torch.cat([S, f + S])
    dW1s, dW2s, db1s, db2 = oracle.rounded_glu_hidden_unit_grads(x, p, experts, W1[:, S2], W2[:, :, S], dy, torch.float32,
                                                                b1[:, S2] if bias else None, with_b2=bias)
    assert torch.allclose(dW1s, grads[2][:, S2], atol=1e-5) and torch.allclose(dW2s, grads[3][:, :, S], atol=1e-5)
    if bias:
        assert torch.allclose(db1s, grads[4][:, S2], atol=1e-5) and torch.allclose(db2, grads[5], atol=1e-5)


def test_rounded_step_in_bfloat16_stays_within_the_format_error():
    g = torch.Generator().manual_seed(6)
    T, d, f, E, k = 32, 64, 48, 4, 2
    bf = lambda t: t.bfloat16().float()
    x, dy = bf(torch.randn(T, d, generator=g)), bf(torch.randn(T, d, generator=g))
    experts = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    p = bf(torch.rand(T, k, generator=g))
    W1, W2 = bf(torch.randn(E, 2 * f, d, generator=g) * 0.1), bf(torch.randn(E, d, f, generator=g) * 0.1)
    exact = oracle.rounded_glu_token_step(x, p, experts, W1, W2, dy, torch.float32)
    rounded = oracle.rounded_glu_token_step(x, p, experts, W1, W2, dy, torch.bfloat16)
    for a, b in zip(exact, rounded):
        assert torch.equal(b, bf(b))                                             # results are values of the format
        assert float((a - b).abs().max()) <= 2e-2 * float(a.abs().max())         # a few roundings of 2^-9 each
        assert float((a - b).abs().max()) > 0                                    # ... and they do round
