"""Sparse MoE MLP modules with the constructor / forward signatures of scattermoe/mlp.py
(`MLP` :6-49, `GLUMLP` :51-95) and the same state-dict keys
(`experts.weight`, `experts.bias`, `output_experts.weight`, `output_experts.bias`)."""
import torch
from torch import nn

from .kernels import ops
from .parallel_experts import ParallelExperts, flatten_sort_count


class _FusedGLU(torch.autograd.Function):
    """act(second half) * first half in one pass each way (saves the pre-activation, recomputes act)."""

    @staticmethod
    def forward(ctx, pre, act):
        ctx.save_for_backward(pre)
        ctx.act = act
        return ops.glu_fwd(pre, act)

    @staticmethod
    def backward(ctx, dh):
        (pre,) = ctx.saved_tensors
        return ops.glu_bwd(pre, dh, ctx.act), None


class _SparseMLP(nn.Module):
    """Shared body: route once, expert layer 1 (grouped output), activation, expert layer 2 (+gates)."""

    _hidden_mult = 1

    def __init__(self, input_size, hidden_size, num_experts, top_k, bias, activation):
        super().__init__()
        self.num_experts = num_experts
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.experts = ParallelExperts(num_experts, input_size, self._hidden_mult * hidden_size, bias=bias)
        self.output_experts = ParallelExperts(num_experts, hidden_size, input_size, bias=bias)
        self.top_k = min(top_k, self.num_experts)
        self.activation = activation

    def extra_repr(self):
        return "k={}".format(self.top_k)

    def _hidden(self, pre):
        raise NotImplementedError

    def forward(self, x: torch.Tensor, expert_p: torch.Tensor, expert_idxs: torch.Tensor):
        lead = x.shape[:-1]
        tokens = x.view(-1, x.size(-1))
        eid, idx, off = flatten_sort_count(expert_idxs, num_experts=self.num_experts)
        pre = self.experts(tokens, self.top_k, eid, idx, off, grouped_out=True)
        hid = self._hidden(pre)
        out = self.output_experts(hid, 1, eid, idx, off, grouped_in=True, gates=expert_p)
        return out.view(*lead, out.size(-1))


class MLP(_SparseMLP):
    """y = sum_j p_j * W2[e_j] act(W1[e_j] x)."""

    def __init__(self, input_size, hidden_size, num_experts, top_k, bias=False, activation=None):
        super().__init__(input_size, hidden_size, num_experts, top_k, bias, activation)

    def _hidden(self, pre):
        return self.activation(pre)


class GLUMLP(_SparseMLP):
    """Gated variant: layer 1 produces 2*hidden columns; the FIRST half is the linear branch and the
    SECOND half goes through the activation (reference mlp.py:81-87)."""

    _hidden_mult = 2

    def __init__(self, input_size, hidden_size, num_experts, top_k, bias=False, activation=nn.SiLU()):
        super().__init__(input_size, hidden_size, num_experts, top_k, bias, activation)

    def _hidden(self, pre):
        if type(self.activation) is nn.SiLU and pre.dim() == 2:
            return _FusedGLU.apply(pre, ops.ACT_SILU)
        lin, gate = pre.chunk(2, dim=-1)
        return self.activation(gate) * lin
