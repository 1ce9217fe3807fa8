"""CPU restatement of the reference's MoE-MLP semantics (plain PyTorch / numpy, no kernels).

TEST INFRASTRUCTURE ONLY — see oracle/__init__.py.

What each function follows in the reference (shawntan/scattermoe):
  route_ref            scattermoe/parallel_experts.py:14-21   flatten -> sort -> bincount -> cumsum
  scatter2scatter_ref  scattermoe/kernels/ops.py:72-118       index conventions, bias, row masks
  group_ref            scattermoe/kernels/ops.py:426-457      Y[n] = A[idx[n] // fan_out] * coeff[idx[n]]
  group_bwd_W_ref      scattermoe/kernels/ops.py:191-199, 272-279, 340-366   per-expert X^T DY, column sums
  naive_token_forward  tests/test_mlp.py:10-26 (dumb_forward) per token, per slot, literal form
  naive_expert_forward the same sum regrouped per expert (gather rows -> 2 linears -> weighted index_add)
  glu / gpt_oss_glu    scattermoe/mlp.py:81-87 ; scattermoe/utils/replace_moe.py:39-43
  topk_softmax_ref     scattermoe/utils/replace_moe.py:67-71  softmax in float -> topk -> renormalise
  rounded_glu_token_step, rounded_glu_hidden_unit_grads
                       the forward + backward dataflow of scattermoe/mlp.py:74-95 and
                       scattermoe/parallel_experts.py:36-134 written out by hand (no autograd), with every tensor the
                       reference materialises in the storage type (layer-1 output, hidden, expanded layer-2 output,
                       gate-scaled grad_out, d hidden, d layer-1 output, expanded d input, and every result) rounded
                       to that type and float32 accumulation in between: what a bf16 run of the reference computes,
                       up to summation order

How it is pinned (tests/test_oracle.py): the reference stores no golden vectors (its single test
compares two live computations on unseeded inputs, tests/test_mlp.py:46-49), so every function is
checked against what the mathematics fixes: brute-force Python loops on tiny inputs, closed forms
(E = 1 reduces to torch.nn.functional.linear; one-hot rows pick out weight rows; identity weights copy),
token-form == expert-form, finite-difference gradients (torch.autograd.gradcheck, fp64), invariants of
the routing triple, and Hugging Face's own per-expert loops as an independent second implementation.
Tie order inside an expert segment is not fixed by the reference (torch.sort is called unstable);
this build defines it as the stable order and route_ref states exactly that.
"""
import numpy as np
import torch
import torch.nn.functional as F

__all__ = [
    "route_ref", "scatter2scatter_ref", "group_ref", "group_bwd_W_ref",
    "naive_token_forward", "naive_expert_forward", "glu", "gpt_oss_glu",
    "module_params", "naive_module_forward", "topk_softmax_ref",
    "rounded_glu_token_step", "rounded_glu_hidden_unit_grads",
]


# ---------------------------------------------------------------------------------------------------
# routing
# ---------------------------------------------------------------------------------------------------
def route_ref(expert_idxs, num_experts):
    """Stable sort of the flattened ids, source slots, inclusive per-expert offsets (all int64)."""
    flat = np.asarray(torch.as_tensor(expert_idxs).detach().cpu().reshape(-1).numpy()).astype(np.int64)
    order = np.argsort(flat, kind="stable").astype(np.int64)
    counts = np.bincount(flat, minlength=num_experts).astype(np.int64)
    return (torch.from_numpy(flat[order].copy()), torch.from_numpy(order),
            torch.from_numpy(np.cumsum(counts)))


def topk_softmax_ref(logits, k, renormalize=True):
    """Router front end: float32 softmax over the experts, the k largest probabilities in descending order
    (lowest expert id first among equals), optionally divided by their sum.  numpy only.
    Pinned in tests/test_oracle.py against torch.softmax + torch.topk, hand-worked rows and invariants."""
    z = np.asarray(torch.as_tensor(logits).detach().cpu().float().numpy(), dtype=np.float32)
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z, dtype=np.float32)
    p = e / e.sum(axis=-1, keepdims=True, dtype=np.float32)
    order = np.argsort(-p, axis=-1, kind="stable")[:, :k].astype(np.int64)
    w = np.take_along_axis(p, order, axis=-1)
    if renormalize:
        w = w / w.sum(axis=-1, keepdims=True, dtype=np.float32)
    return torch.from_numpy(w.astype(np.float32)), torch.from_numpy(order)


# ---------------------------------------------------------------------------------------------------
# functional models of the three kernels
# ---------------------------------------------------------------------------------------------------
def scatter2scatter_ref(X, W, eid, idx, k, b=None, x_grouped=False, y_grouped=False, acc=torch.float32):
    """Y[dst(n)] = X[src(n)] @ W[eid[n]] (+ b[eid[n]]); src = n | idx[n]//k, dst = n | idx[n]."""
    L, N = eid.numel(), W.size(-1)
    Y = torch.zeros(L, N, dtype=acc)
    rows = torch.arange(L)
    src = rows if x_grouped else idx // k
    dst = rows if y_grouped else idx
    for e in range(W.size(0)):
        sel = (eid == e).nonzero().flatten()
        if sel.numel() == 0:
            continue
        y = X[src[sel]].to(acc) @ W[e].to(acc)
        if b is not None:
            y = y + b[e].to(acc)
        Y[dst[sel]] = y
    return Y.to(X.dtype)


def group_ref(A, idx, coeff=None, fan_out=1):
    Y = A[idx // fan_out]
    if coeff is not None:
        Y = (Y.float() * coeff.reshape(-1)[idx].float()[:, None]).to(A.dtype)
    return Y


def group_bwd_W_ref(DY, X, off, E, has_bias=False, acc=torch.float32):
    """(DW (E,K,N), Db (E,N) | None) over expert-grouped rows; zeros for experts without rows."""
    K, N = X.size(-1), DY.size(-1)
    DW = torch.zeros(E, K, N, dtype=acc)
    Db = torch.zeros(E, N, dtype=acc) if has_bias else None
    lo = 0
    for e in range(E):
        hi = int(off[e])
        if hi > lo:
            DW[e] = X[lo:hi].to(acc).T @ DY[lo:hi].to(acc)
            if has_bias:
                Db[e] = DY[lo:hi].to(acc).sum(0)
        lo = hi
    return DW.to(DY.dtype), (Db.to(DY.dtype) if has_bias else None)


# ---------------------------------------------------------------------------------------------------
# hidden-layer nonlinearities of the module variants
# ---------------------------------------------------------------------------------------------------
def glu(act):
    """GLUMLP hidden: first half linear, second half activated (mlp.py:81-87)."""
    def f(pre):
        lin, gate = pre.chunk(2, dim=-1)
        return act(gate) * lin
    return f


def gpt_oss_glu(alpha=1.702, limit=7.0):
    """gpt-oss hidden: interleaved gate/up columns, clamps, gate*sigmoid(alpha*gate)*(up+1)."""
    def f(pre):
        gate, up = pre[..., ::2], pre[..., 1::2]
        gate = gate.clamp(max=limit)
        up = up.clamp(min=-limit, max=limit)
        return (up + 1) * (gate * torch.sigmoid(gate * alpha))
    return f


# ---------------------------------------------------------------------------------------------------
# the naive MoE MLP, two equivalent forms.  W1 (E, n1, d), W2 (E, d, f) in nn.Linear layout.
# ---------------------------------------------------------------------------------------------------
def naive_token_forward(x, p, experts, W1, W2, hidden, b1=None, b2=None):
    """Literal per-token / per-slot sum (the reference test's dumb_forward). O(T*k) tiny products."""
    rows = []
    for t in range(experts.size(0)):
        acc = 0
        for j in range(experts.size(1)):
            e = int(experts[t, j])
            h = hidden(F.linear(x[t], W1[e], None if b1 is None else b1[e]))
            acc = acc + p[t, j] * F.linear(h, W2[e], None if b2 is None else b2[e])
        rows.append(acc)
    return torch.stack(rows, dim=0)


def naive_expert_forward(x, p, experts, W1, W2, hidden, b1=None, b2=None):
    """Same function, regrouped: per expert gather its (token, slot) pairs, two linears, weighted add."""
    T, d_out = x.size(0), W2.size(1)
    y = torch.zeros(T, d_out, dtype=x.dtype)
    for e in range(W1.size(0)):
        tok, slot = (experts == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        h = hidden(F.linear(x[tok], W1[e], None if b1 is None else b1[e]))
        o = F.linear(h, W2[e], None if b2 is None else b2[e])
        y = y.index_add(0, tok, p[tok, slot].unsqueeze(-1) * o)
    return y


def module_params(m):
    """(W1, W2, b1, b2) of an MLP / GLUMLP-shaped module."""
    return m.experts.weight, m.output_experts.weight, m.experts.bias, m.output_experts.bias


def naive_module_forward(m, x, p, experts, per_token=False):
    W1, W2, b1, b2 = module_params(m)
    hidden = glu(m.activation) if W1.size(1) == 2 * W2.size(2) and type(m).__name__ == "GLUMLP" else m.activation
    f = naive_token_forward if per_token else naive_expert_forward
    return f(x, p, experts, W1, W2, hidden, b1, b2)


# ---------------------------------------------------------------------------------------------------
# The GLU MoE MLP step with the storage type's rounding where the reference materialises a tensor.
# Written out by hand, forward and backward; with dtype=torch.float32 nothing is rounded and the results
# are the autograd gradients of naive_token_forward / naive_expert_forward (tests/test_oracle.py pins that).
# Inputs are float32 tensors holding values of the storage type.
# ---------------------------------------------------------------------------------------------------
def _silu_parts(gat):
    s = torch.sigmoid(gat)
    return gat * s, s * (1.0 + gat * (1.0 - s))          # silu(g), silu'(g)


def rounded_glu_token_step(x, p, experts, W1, W2, dy, dtype, b1=None, b2=None):
    """(y, dx, dp) of the given tokens.  x (n, d), p / experts (n, k), dy (n, d); W1 (E, 2f, d), W2 (E, d, f)."""
    rnd = lambda t: t.to(dtype).float()
    n, k = experts.shape
    f = W2.size(2)
    y, dx, dp = torch.zeros_like(x), torch.zeros_like(x), torch.zeros_like(p)
    for t in range(n):
        out = torch.zeros(x.size(1))
        parts = []
        for j in range(k):
            e = int(experts[t, j])
            pre = W1[e] @ x[t]
            if b1 is not None:
                pre = pre + b1[e]
            pre = rnd(pre)                                           # layer-1 output as stored
            lin, gat = pre[:f], pre[f:]
            a, da = _silu_parts(gat)
            h = rnd(a * lin)                                         # hidden as stored
            yj = W2[e] @ h
            if b2 is not None:
                yj = yj + b2[e]
            yj = rnd(yj)                                             # expanded layer-2 output as stored
            out = out + p[t, j] * yj                                 # float32, slot order
            parts.append((e, lin, a, da, yj))
        y[t] = rnd(out)
        acc = torch.zeros(x.size(1))
        for j, (e, lin, a, da, yj) in enumerate(parts):
            dp[t, j] = rnd(torch.dot(yj, dy[t]))
            gdy = rnd(dy[t] * p[t, j])                               # gate-scaled output gradient as stored
            dh = rnd(W2[e].T @ gdy)                                  # d hidden as stored
            dpre = torch.cat([rnd(dh * a), rnd((dh * lin) * da)])    # d layer-1 output as stored
            acc = acc + rnd(W1[e].T @ dpre)                          # expanded d input as stored, summed in float32
        dx[t] = rnd(acc)
    return y, dx, dp


def rounded_glu_hidden_unit_grads(x, p, experts, W1s, W2s, dy, dtype, b1s=None, with_b2=False):
    """(dW1s, dW2s, db1s, db2) for a model cut down to a subset S of hidden units: W1s (E, 2|S|, d) holds the rows
    S and f + S of W1, W2s (E, d, |S|) the columns S of W2 (a hidden unit's weight gradients depend on the other
    units only through dy, which is given).  All tokens, all experts."""
    rnd = lambda t: t.to(dtype).float()
    E, k = W1s.size(0), experts.size(1)
    ns = W2s.size(2)
    _, idx, off = route_ref(experts, E)
    tok = idx // k
    gdy = rnd(dy[tok] * p.reshape(-1)[idx].unsqueeze(-1))            # expert-sorted, gate-scaled, as stored
    dW1s, dW2s = torch.zeros_like(W1s), torch.zeros_like(W2s)
    db1s = torch.zeros(E, 2 * ns) if b1s is not None else None
    db2 = torch.zeros(E, x.size(1)) if with_b2 else None
    lo = 0
    for e in range(E):
        hi = int(off[e])
        if hi > lo:
            xe, ge = x[tok[lo:hi]], gdy[lo:hi]
            pre = xe @ W1s[e].T
            if b1s is not None:
                pre = pre + b1s[e]
            pre = rnd(pre)
            lin, gat = pre[:, :ns], pre[:, ns:]
            a, da = _silu_parts(gat)
            h = rnd(a * lin)
            dh = rnd(ge @ W2s[e])
            dpre = torch.cat([rnd(dh * a), rnd((dh * lin) * da)], dim=1)
            dW1s[e] = rnd(dpre.T @ xe)
            dW2s[e] = rnd(ge.T @ h)
            if db1s is not None:
                db1s[e] = rnd(dpre.sum(0))
            if db2 is not None:
                db2[e] = rnd(ge.sum(0))
        lo = hi
    return dW1s, dW2s, db1s, db2
