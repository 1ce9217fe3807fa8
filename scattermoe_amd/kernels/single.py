"""Decode helper with the signature of the reference's `single2scatter` (scattermoe/kernels/single.py:41-59):
one token (or k already-expanded rows) times the k experts it is routed to.

The reference has a dedicated GEMV kernel that nothing calls; here the call goes through
`scatter2scatter`, which sends launches of a handful of rows to its own weight-streaming kernels (the row-dot
kernel for weights with a contiguous contraction axis, ring-buffered 32-row tiles otherwise): each routed
expert's weights are read exactly once."""

from . import ops


def single2scatter(X, W, expert_idxs):
    """Y[j] = X[j if X.size(0) == k else 0] @ W[expert_idxs[0, j]]  ->  (k, N)."""
    E, xdim, ydim = W.size()
    k = expert_idxs.size(1)
    assert X.size(0) == k or X.size(0) == 1
    assert X.size(1) == xdim
    eid, idx, off = ops.route(expert_idxs, E)
    return ops.scatter2scatter(X, W, eid, idx, k // X.size(0), expert_offsets=off)
