"""Hugging Face injection: route the expert computation of transformers MoE blocks through the
scattermoe_amd kernels by replacing their `forward` lazily, on first call.

Counterpart of scattermoe/utils/replace_moe.py of the reference: `replace_function` (:8-17),
`gpt_oss_forward` (:19-57) and `granite_moe_forward` (:60-95).  The reference patches were written against
transformers 4.5x; the module layouts changed in 5.x (gpt-oss hands the experts already-selected
(T, k) weights; GraniteMoeHybridMoE owns a router that returns `(top_k_index, top_k_weights, logits)` and an
`experts` module with `gate_up_proj (E, 2I, H)` / `down_proj (E, H, I)` and returns a single tensor), so each
forward below accepts both layouts and keeps the return convention of the layout it finds.
`experts_forward` is the same computation for every 5.x `*Experts.forward(hidden_states, top_k_index,
top_k_weights)` module (Mixtral, GraniteMoeHybrid, ...); `patch_experts_class(cls)` installs it.
"""
import logging

import torch
from torch import nn
from torch.nn import functional as F

from ..kernels import ops
from ..parallel_experts import flatten_sort_count, parallel_linear


def replace_function(cls, fun_name):
    """Decorator: install `fun` as `cls.fun_name`, announcing the swap when it is first used."""
    def decorator(fun):
        fun.__original__ = getattr(cls, fun_name, None)       # what the class had before; kept for comparisons / undo

        def first_call(*args, **kwargs):
            logging.info("Replacing `%s.%s` with %s:%s", cls.__name__, fun_name,
                         fun.__code__.co_filename, fun.__name__)
            setattr(cls, fun_name, fun)
            return fun(*args, **kwargs)
        first_call.__wrapped__ = fun
        first_call.__original__ = fun.__original__
        setattr(cls, fun_name, first_call)
        return fun
    return decorator


def _is_silu(act_fn):
    return isinstance(act_fn, nn.SiLU) or act_fn is F.silu or type(act_fn).__name__ in ("SiLUActivation", "SiLU")


def _gated_mlp(tokens, gate_up_w, down_w, k, eid, idx, off, weights, act_fn):
    """Gated expert MLP with `act(gate) * up`, gate = first half of the (E, 2I, H) layer-1 weights.  With SiLU the
    whole block is one autograd node whose GLU rides in the GEMM epilogues; other activations use three nodes."""
    if _is_silu(act_fn) and tokens.dim() == 2:
        from ..mlp import _GatedMLP
        return _GatedMLP.apply(tokens, gate_up_w.permute(0, 2, 1), None, down_w.permute(0, 2, 1), None,
                               weights.to(tokens.dtype), eid, idx, off, k, ops.ACT_SILU_GATE_FIRST)
    pre = parallel_linear(tokens, gate_up_w.transpose(1, 2), k, eid, idx, off, grouped_in=False, grouped_out=True)
    h = _glu(pre, act_fn, gate_first=True)
    return parallel_linear(h, down_w.transpose(1, 2), 1, eid, idx, off, grouped_in=True, grouped_out=False,
                           gates=weights.to(h.dtype))


def _glu(pre, act_fn, gate_first):
    """act(gate) * linear over the two halves of `pre`; fused kernel when the activation is SiLU."""
    silu = _is_silu(act_fn)
    if silu and pre.dim() == 2:
        from ..mlp import _FusedGLU
        return _FusedGLU.apply(pre, ops.ACT_SILU_GATE_FIRST if gate_first else ops.ACT_SILU)
    a, b = pre.chunk(2, dim=-1)
    return act_fn(a) * b if gate_first else act_fn(b) * a


def experts_forward(self, hidden_states, top_k_index, top_k_weights):
    """Drop-in for transformers 5.x `*Experts.forward`: gate_up_proj (E, 2I, H), down_proj (E, H, I),
    `act_fn(gate) * up` with gate = first half; returns (T, H)."""
    k = top_k_index.shape[-1]
    if (top_k_index.numel() <= ops.DECODE_MAX_ROWS and not torch.is_grad_enabled() and _is_silu(self.act_fn)
            and hidden_states.dim() == 2 and top_k_index.dim() == 2):
        out = ops.decode_glu_mlp(hidden_states, top_k_weights, top_k_index, self.gate_up_proj, None, self.down_proj,
                                 None, ops.ACT_SILU_GATE_FIRST)
        if out is not None:
            return out
    eid, idx, off = flatten_sort_count(top_k_index, num_experts=self.num_experts)
    return _gated_mlp(hidden_states, self.gate_up_proj, self.down_proj, k, eid, idx, off, top_k_weights, self.act_fn)


def patch_experts_class(cls):
    """Install `experts_forward` on a transformers 5.x experts class (lazy, like the built-in patches)."""
    replace_function(cls=cls, fun_name="forward")(experts_forward)
    return cls


try:
    from transformers.models.gpt_oss.modeling_gpt_oss import GptOssExperts

    @replace_function(cls=GptOssExperts, fun_name="forward")
    def gpt_oss_forward(self, hidden_states: torch.Tensor, router_indices=None, routing_weights=None) -> torch.Tensor:
        lead_shape = hidden_states.shape
        hidden_states = hidden_states.reshape(-1, self.hidden_size)
        k = router_indices.shape[-1]
        router_indices = router_indices.reshape(-1, k)
        routing_weights = routing_weights.reshape(hidden_states.shape[0], -1)
        if routing_weights.shape[-1] == self.num_experts and k != self.num_experts:
            # 4.x layout: dense (T, E) scores, pick the routed ones
            routing_weights = torch.gather(routing_weights, dim=1, index=router_indices)
        eid, idx, off = flatten_sort_count(router_indices, num_experts=self.num_experts)

        if hidden_states.dtype in (torch.bfloat16, torch.float16) and hidden_states.is_cuda:
            # one autograd node; the gated unit rides in the epilogues of the GEMMs around it
            from ..mlp import _GatedMLP
            out = _GatedMLP.apply(hidden_states, self.gate_up_proj, self.gate_up_proj_bias, self.down_proj,
                                  self.down_proj_bias, routing_weights.to(hidden_states.dtype), eid, idx, off, k,
                                  ops.ACT_GPT_OSS, float(self.alpha), float(self.limit))
        else:
            gate_up = parallel_linear(hidden_states, self.gate_up_proj, k, eid, idx, off,
                                      expert_biases=self.gate_up_proj_bias, grouped_in=False, grouped_out=True)
            hidden = ops.gpt_oss_glu(gate_up, self.alpha, self.limit)      # clamp, sigmoid gate, (up + 1) * glu: one pass
            out = parallel_linear(hidden, self.down_proj, 1, eid, idx, off,
                                  expert_biases=self.down_proj_bias, grouped_in=True, grouped_out=False,
                                  gates=routing_weights.to(hidden.dtype))
        if len(lead_shape) == 3:       # 4.x callers pass (batch, seq, hidden) and expect it back
            return out.view(lead_shape[0], -1, self.hidden_size)
        return out
except Exception:   # transformers missing or without this model: nothing to patch
    logging.info("Failed to replace GptOssExperts")


try:
    from transformers.models.granitemoehybrid.modeling_granitemoehybrid import GraniteMoeHybridMoE

    @replace_function(cls=GraniteMoeHybridMoE, fun_name="forward")
    def granite_moe_forward(self, layer_input):
        bsz, length, emb_size = layer_input.size()
        tokens = layer_input.reshape(-1, emb_size)
        if hasattr(self, "input_linear"):
            # 4.x layout: router.layer + input_linear / output_linear, returns (output, router_logits)
            router_logits = self.router.layer(tokens)
            weights, selected = ops.topk_softmax(router_logits, self.router.top_k, renormalize=True)  # one launch
            weights = weights.to(tokens.dtype)
            eid, idx, off = flatten_sort_count(selected, num_experts=self.router.num_experts)
            out = _gated_mlp(tokens, self.input_linear.weight, self.output_linear.weight, self.router.top_k,
                             eid, idx, off, weights, self.activation)
            return out.view(bsz, length, emb_size), router_logits
        top_k_index, top_k_weights, _ = self.router(tokens)
        out = experts_forward(self.experts, tokens, top_k_index, top_k_weights)
        return out.view(bsz, length, self.input_size)
except Exception:
    logging.info("Failed to replace GraniteMoeHybridMoE")
