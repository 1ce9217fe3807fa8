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
