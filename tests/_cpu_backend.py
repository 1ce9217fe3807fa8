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
