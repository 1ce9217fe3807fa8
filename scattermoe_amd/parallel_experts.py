"""Routing prep, the expert-parallel linear autograd function, and its parameter module.

Mirrors scattermoe/parallel_experts.py of the reference: `flatten_sort_count` (:14-21),
`ParallelLinear` (:25-134), `parallel_linear` (:136-146) and `ParallelExperts` (:148-182), with the
same call signatures, saved-tensor dataflow and parameter names.  All heavy lifting happens in
`kernels.ops`, i.e. in the HIP library.
"""
from typing import Optional

import torch
import torch.nn as nn

from .kernels import ops


@torch.library.custom_op("scattermoe::bincount", mutates_args={})
def compileable_bincount(x: torch.Tensor, minlength: int) -> torch.Tensor:
    """Per-expert counts (reference parallel_experts.py:6-12), from the routing kernel's offsets.

    Ids are expected to lie in [0, minlength), which is how the reference uses it.
    """
    _, _, off = ops.route(x, minlength)
    return torch.diff(off, prepend=off.new_zeros(1))


@compileable_bincount.register_fake
def _(x: torch.Tensor, minlength: int) -> torch.Tensor:
    return torch.empty(minlength, dtype=torch.long, device=x.device)


def flatten_sort_count(expert_idxs: torch.Tensor, num_experts: int):
    """(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets) of a (T, k) top-k index tensor.

    One counting-sort launch sequence instead of sort + bincount + cumsum.  Rows of one expert keep
    their original order (stable), which is the order torch.sort(..., stable=True) produces.
    """
    with torch.no_grad():
        return ops.route(expert_idxs, num_experts)


# name used by earlier releases of the reference for the same routine
flatten_and_sort = flatten_sort_count


class ParallelLinear(torch.autograd.Function):
    """y = scatter2scatter(x, W[, b]) [combined with gates]; backward via group / groupXtY / scatter2scatter."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, expert_weights: torch.Tensor, k: int,
                sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor,
                expert_offsets: torch.Tensor,
                expert_biases: Optional[torch.Tensor] = None,
                gates: Optional[torch.Tensor] = None,
                grouped_in: bool = False, grouped_out: bool = False):
        expanded = ops.scatter2scatter(
            X=x, W=expert_weights, b=expert_biases, k=k,
            sorted_expert_idxs=sorted_expert_idxs, sorted_scattered_idxs=sorted_scattered_idxs,
            x_grouped=grouped_in, y_grouped=grouped_out, expert_offsets=expert_offsets)
        if gates is None:
            result, kept = expanded, None
        else:
            kept = expanded.view(gates.size(0), gates.size(1), expanded.size(-1))
            result = ops.combine(kept, gates)
        ctx.save_for_backward(x, expert_weights, expert_biases, sorted_expert_idxs,
                              sorted_scattered_idxs, expert_offsets, gates, kept)
        ctx.k, ctx.grouped_in, ctx.grouped_out = k, grouped_in, grouped_out
        return result

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        (x, W, bias, eid, idx, off, gates, kept) = ctx.saved_tensors
        k, grouped_in, grouped_out = ctx.k, ctx.grouped_in, ctx.grouped_out
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = bias is not None and ctx.needs_input_grad[6]
        need_g = gates is not None and ctx.needs_input_grad[7]
        E = W.size(0)
        if not grad_out.is_contiguous():
            grad_out = grad_out.contiguous()

        d_gates = dy = None
        coeff, coeff_fan, dy_buf = None, 1, None
        if gates is not None:
            if need_g and not grouped_out:
                # (T, k) row dots of every expert output with dY, and dY in expert-sorted order scaled by the gate
                # of each (token, slot), in one pass
                d_gates, dy = ops.gate_grad_group(kept, grad_out, gates, idx)
            elif need_g:
                d_gates = ops.gate_grad(kept, grad_out)
            coeff, coeff_fan = gates.reshape(-1), gates.size(1)
            dy_buf = kept.view(-1, kept.size(-1))   # its contents are dead once d_gates exists

        # dY in expert-sorted order, scaled by the gate of each (token, slot)
        if grouped_out:
            dy = grad_out
        elif dy is None:
            dy = ops.group(grad_out, idx, coeff=coeff, fan_out=coeff_fan, out=dy_buf, permutation=True)

        d_w = d_b = None
        if need_w or need_b:
            # ungrouped input: the weight gradient reads the rows of x through idx (the reference gathers a copy
            # of x first, parallel_experts.py:95-99)
            d_w, d_b = ops.group_bwd_W(DY=dy, X=x, expert_offsets=off, E=E, has_bias=bias is not None, like=W,
                                       gather=None if grouped_in else (idx, k))
            if not need_w:
                d_w = None

        d_x = None
        if need_x:
            # dX rows: dY @ W[e]^T, written grouped (grouped_in) or scattered back to slot order
            d_exp = ops.scatter2scatter(
                X=dy, W=W.permute(0, 2, 1), k=1, x_grouped=True, y_grouped=grouped_in,
                sorted_expert_idxs=eid, sorted_scattered_idxs=idx, expert_offsets=off)
            d_x = ops.slot_sum(d_exp, x.size(0), k)

        return d_x, d_w, None, None, None, None, d_b, d_gates, None, None


def parallel_linear(inputs, expert_weights, k,
                    sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                    expert_biases=None, gates=None, grouped_in=False, grouped_out=False):
    """Reference parallel_experts.py:136-146, same arguments.

    `sorted_scattered_idxs` must be what `flatten_sort_count` returns for this batch: a permutation of
    range(tokens * k).  The forward pass already depends on that (with `grouped_out=False` row idx[n] of the output
    is written by row n: a repeated entry leaves another row unwritten, here as in the reference); the backward pass
    depends on it too, because the gate-scaled output gradient is written by source row through the inverse
    permutation - rows of a vector that is no permutation would keep stale contents."""
    return ParallelLinear.apply(inputs, expert_weights, k,
                                sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                                expert_biases, gates, grouped_in, grouped_out)


class ParallelExperts(nn.Module):
    """E independent linear maps stored as one (E, out, in) parameter (+ optional (E, out) bias)."""

    def __init__(self, num_experts, input_size, output_size, bias=False) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.input_size = input_size
        self.output_size = output_size
        self.weight = nn.Parameter(torch.empty(num_experts, output_size, input_size))
        self.bias = nn.Parameter(torch.empty(num_experts, output_size)) if bias else None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, std=0.02)
        if self.bias is not None:
            nn.init.zeros_(self.bias)

    def extra_repr(self):
        return "num_experts={}, input_size={}, output_size={}".format(
            self.num_experts, self.input_size, self.output_size)

    def forward(self, inputs, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                gates=None, grouped_in=False, grouped_out=False):
        # the kernels see the weight as (E, in, out) with the `in` axis contiguous
        return parallel_linear(inputs, self.weight.permute(0, 2, 1), k,
                               sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                               expert_biases=self.bias, gates=gates,
                               grouped_in=grouped_in, grouped_out=grouped_out)
