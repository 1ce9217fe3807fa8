"""Test double for scattermoe_amd.kernels.ops._backend built on the CPU oracle (tests only)."""
import torch

import oracle


class OracleBackend:
    name = "oracle"

    @staticmethod
    def route(flat_ids, num_experts, eid, idx, off):
        e, i, o = oracle.route_ref(flat_ids, num_experts)
        eid.copy_(e); idx.copy_(i); off.copy_(o)

    @staticmethod
    def offsets(eid, num_experts, off):
        off.copy_(torch.bincount(eid, minlength=num_experts).cumsum(0))

    @staticmethod
    def s2s(X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped):
        Y.copy_(oracle.scatter2scatter_ref(X, W, eid, idx, k, b, x_grouped, y_grouped))

    @staticmethod
    def group(A, coeff, Y, idx, fan_out):
        Y.copy_(oracle.group_ref(A, idx, coeff, fan_out))

    @staticmethod
    def xty(DY, X, DW, Db, off, E):
        dw, db = oracle.group_bwd_W_ref(DY, X, off, E, has_bias=Db is not None)
        DW.copy_(dw)
        if Db is not None:
            Db.copy_(db)

    @staticmethod
    def combine(Y, gates, out, k):
        if gates is None:
            gates = torch.ones(out.size(0), k)
        out.copy_((Y.view(out.size(0), k, -1).float() * gates.float().unsqueeze(-1)).sum(1))

    @staticmethod
    def gate_grad(Y, d_out, d_gates, k):
        d_gates.copy_((Y.view(d_out.size(0), k, -1).float() * d_out.float().unsqueeze(1)).sum(-1))

    @staticmethod
    def glu_fwd(pre, h, act):
        lin, gate = pre.float().chunk(2, dim=-1)
        if act & 1:
            lin, gate = gate, lin
        h.copy_(torch.nn.functional.silu(gate) * lin)

    @staticmethod
    def glu_bwd(pre, dh, dpre, act):
        lin, gate = pre.float().chunk(2, dim=-1)
        if act & 1:
            lin, gate = gate, lin
        s = torch.sigmoid(gate)
        d_lin, d_gate = dh.float() * gate * s, dh.float() * lin * s * (1 + gate * (1 - s))
        dpre.copy_(torch.cat([d_gate, d_lin] if act & 1 else [d_lin, d_gate], dim=-1))

    @staticmethod
    def topk_softmax(logits, weights, experts, renormalize):
        w, i = oracle.topk_softmax_ref(logits, weights.size(1), renormalize)
        weights.copy_(w); experts.copy_(i)

    @staticmethod
    def oss_glu_fwd(pre, h, alpha, limit):
        h.copy_(oracle.gpt_oss_glu(alpha, limit)(pre.float()))

    @staticmethod
    def oss_glu_bwd(pre, dh, dpre, alpha, limit):
        with torch.enable_grad():
            p = pre.detach().float().requires_grad_()
            (g,) = torch.autograd.grad(oracle.gpt_oss_glu(alpha, limit)(p), p, dh.float())
        dpre.copy_(g)
