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


class _GatedMLP(torch.autograd.Function):
    """The whole gated expert MLP as one autograd node, so that the gated linear unit can ride in the epilogues
    of the GEMMs around it: forward = layer 1 + GLU (one launch), layer 2, gate-weighted combine; backward =
    the dataflow of two chained ParallelLinear nodes (reference parallel_experts.py:64-134) with the layer-2
    input gradient and the GLU gradient in one launch.  Same numerics as the unfused chain (intermediates are
    rounded to the storage type at the same points).

    w1 (E, d, 2F) and w2 (E, F, d) are the (E, in, out) views the kernels take, in either memory layout: the
    permuted ParallelExperts parameters, or weights stored that way (gpt-oss); their gradients come back in the
    layout of the weight they belong to.  `act`: ops.ACT_SILU / ACT_SILU_GATE_FIRST / ACT_GPT_OSS (+ alpha, limit)."""

    @staticmethod
    def forward(ctx, x, w1, b1, w2, b2, gates, eid, idx, off, k, act, alpha=1.702, limit=7.0):
        T = x.size(0)
        need_grad = any(ctx.needs_input_grad[:6])
        pre, h = ops.scatter2scatter_glu(x, w1, eid, idx, k, b=b1, act=act, expert_offsets=off,
                                         need_pre=need_grad, alpha=alpha, limit=limit)
        expanded = ops.scatter2scatter(h, w2, eid, idx, 1, b=b2, x_grouped=True, y_grouped=False,
                                       expert_offsets=off)
        kept = expanded.view(T, k, expanded.size(-1))
        out = ops.combine(kept, gates)
        if need_grad:
            ctx.save_for_backward(x, w1, b1, w2, b2, gates, eid, idx, off, pre, h, kept)
        ctx.k, ctx.act, ctx.alpha, ctx.limit = k, act, alpha, limit
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w1, b1, w2, b2, gates, eid, idx, off, pre, h, kept = ctx.saved_tensors
        k, act = ctx.k, ctx.act
        need_x, need_w1, need_b1, need_w2, need_b2, need_g = ctx.needs_input_grad[:6]
        need_b1 = need_b1 and b1 is not None
        need_b2 = need_b2 and b2 is not None
        E = w1.size(0)
        if not grad_out.is_contiguous():
            grad_out = grad_out.contiguous()
        if need_g:
            # gate gradient and dY of layer 2 (expert-sorted, scaled by each row's gate) in one pass over the
            # expert outputs
            d_gates, dy = ops.gate_grad_group(kept, grad_out, gates, idx)
        else:
            # dY alone reuses the expert-output buffer
            d_gates = None
            dy = ops.group(grad_out, idx, coeff=gates.reshape(-1).to(grad_out.dtype), fan_out=k, permutation=True,
                           out=kept.view(-1, kept.size(-1)))
        d_w2 = d_b2 = None
        if need_w2 or need_b2:
            d_w2, d_b2 = ops.group_bwd_W(DY=dy, X=h, expert_offsets=off, E=E, has_bias=b2 is not None, like=w2)
            d_w2 = d_w2 if need_w2 else None
        d_x = d_w1 = d_b1 = None
        if need_x or need_w1 or need_b1:
            dpre = ops.scatter2scatter_glu_bwd(dy, w2.permute(0, 2, 1), pre, eid, idx, act=act, expert_offsets=off,
                                               alpha=ctx.alpha, limit=ctx.limit)
            if need_w1 or need_b1:
                # the weight gradient reads the rows of x through idx: no gathered copy of x is made
                d_w1, d_b1 = ops.group_bwd_W(DY=dpre, X=x, expert_offsets=off, E=E, has_bias=b1 is not None, like=w1,
                                             gather=(idx, k))
                d_w1 = d_w1 if need_w1 else None
            if need_x:
                d_exp = ops.scatter2scatter(dpre, w1.permute(0, 2, 1), eid, idx, 1, x_grouped=True, y_grouped=False,
                                            expert_offsets=off)
                d_x = ops.slot_sum(d_exp, x.size(0), k)
        return d_x, d_w1, (d_b1 if need_b1 else None), d_w2, (d_b2 if need_b2 else None), d_gates, \
            None, None, None, None, None, None, None


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

    def forward(self, x: torch.Tensor, expert_p: torch.Tensor, expert_idxs: torch.Tensor):
        if type(self.activation) is not nn.SiLU:
            return super().forward(x, expert_p, expert_idxs)
        lead = x.shape[:-1]
        tokens = x.view(-1, x.size(-1))
        if expert_idxs.numel() <= ops.DECODE_MAX_ROWS and not torch.is_grad_enabled() and expert_idxs.dim() == 2:
            out = ops.decode_glu_mlp(tokens, expert_p, expert_idxs, self.experts.weight, self.experts.bias,
                                     self.output_experts.weight, self.output_experts.bias, ops.ACT_SILU)
            if out is not None:
                return out.view(*lead, out.size(-1))
        eid, idx, off = flatten_sort_count(expert_idxs, num_experts=self.num_experts)
        out = _GatedMLP.apply(tokens, self.experts.weight.permute(0, 2, 1), self.experts.bias,
                              self.output_experts.weight.permute(0, 2, 1), self.output_experts.bias, expert_p,
                              eid, idx, off, self.top_k, ops.ACT_SILU)
        return out.view(*lead, out.size(-1))
