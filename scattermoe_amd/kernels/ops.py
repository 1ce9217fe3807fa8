"""Host half of the expert kernels: output allocation, shape checks, and the hand-off to the C ABI.

Mirrors the wrapper layer of the reference, scattermoe/kernels/ops.py — `scatter2scatter` (:120-137),
`group_bwd_W` (:191-199), `group` (:377-386) and the four `torch.library` ops (:140, :202, :389 and
parallel_experts.py:6) — with the Triton launches replaced by calls into libscattermoe_amd.so.

All device work goes through `_backend`, an object with `route / offsets / s2s / group / xty` methods.
The only backend shipped is `HipBackend` (the C ABI); it refuses CPU tensors.
"""
from typing import Optional

import torch

from .. import _C

# Kept so that code written against the reference keeps working.  Tile heights are picked inside the
# library per launch, and gfx950 has no TF32 mode: fp32 inputs are always multiplied in full fp32.
BLOCK_M = 128
ALLOW_TF32 = True


class HipBackend:
    """Launches the gfx950 kernels on the current torch stream of the tensors' device."""

    name = "hip"

    @staticmethod
    def route(flat_ids, num_experts, eid, idx, off):
        _C.require_gpu(flat_ids, "flatten_sort_count")
        lib = _C.load()
        L = flat_ids.numel()
        need = lib.smoe_route_workspace_bytes(L, num_experts)
        ws = torch.empty(need, dtype=torch.uint8, device=flat_ids.device) if need else None
        with _C.on_device(flat_ids.device):
            rc = lib.smoe_route(_C.ptr(flat_ids), _C.index_code(flat_ids.dtype), L, num_experts,
                                _C.ptr(eid), _C.ptr(idx), _C.ptr(off), _C.ptr(ws), need,
                                _C.stream_ptr(flat_ids.device))
        _C.check(rc, "smoe_route")

    @staticmethod
    def offsets(eid, num_experts, off):
        _C.require_gpu(eid, "expert offsets")
        lib = _C.load()
        with _C.on_device(eid.device):
            rc = lib.smoe_offsets_from_sorted(_C.ptr(eid), eid.numel(), num_experts, _C.ptr(off),
                                              _C.stream_ptr(eid.device))
        _C.check(rc, "smoe_offsets_from_sorted")

    @staticmethod
    def s2s(X, W, b, Y, eid, idx, off, k, x_grouped, y_grouped):
        _C.require_gpu(X, "scatter2scatter")
        lib = _C.load()
        sbe, sbn = (b.stride(0), b.stride(1)) if b is not None else (0, 0)
        code = _C.float_code(X.dtype)
        # scratch for the products that split the contraction of their experts' last tiles (0 bytes for the others);
        # torch's allocator hands the same block out again step after step
        need = lib.smoe_scatter2scatter_workspace_bytes(eid.numel(), X.size(1), Y.size(1), W.size(0), code)
        ws = torch.empty(need, dtype=torch.uint8, device=X.device) if need else None
        with _C.on_device(X.device):
            rc = lib.smoe_scatter2scatter_ws(
                _C.ptr(X), X.stride(0), X.stride(1),
                _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                _C.ptr(b), sbe, sbn,
                _C.ptr(Y), Y.stride(0), Y.stride(1),
                _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                eid.numel(), X.size(1), Y.size(1), W.size(0), k,
                int(bool(x_grouped)), int(bool(y_grouped)), code,
                _C.ptr(ws), need, _C.stream_ptr(X.device))
        _C.check(rc, "smoe_scatter2scatter")

    @staticmethod
    def group(A, coeff, Y, idx, fan_out):
        _C.require_gpu(A, "group")
        lib = _C.load()
        with _C.on_device(A.device):
            rc = lib.smoe_group(_C.ptr(A), A.stride(0), A.stride(1), _C.ptr(coeff),
                                _C.ptr(Y), Y.stride(0), Y.stride(1), _C.ptr(idx),
                                idx.numel(), A.size(1), fan_out, _C.float_code(A.dtype),
                                _C.stream_ptr(A.device))
        _C.check(rc, "smoe_group")

    @staticmethod
    def group_by_source(A, coeff, Y, idx, inverse, fan_out):
        """True if launched; False if the library does not take these operands (the caller then uses `group`)."""
        _C.require_gpu(A, "group")
        lib = _C.load()
        with _C.on_device(A.device):
            rc = lib.smoe_group_by_source(_C.ptr(A), A.stride(0), A.stride(1), _C.ptr(coeff),
                                          _C.ptr(Y), Y.stride(0), Y.stride(1), _C.ptr(idx), _C.ptr(inverse),
                                          idx.numel(), A.size(1), fan_out, _C.float_code(A.dtype),
                                          _C.stream_ptr(A.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_group_by_source")
        return True

    @staticmethod
    def xty(DY, X, DW, Db, off, E):
        _C.require_gpu(DY, "group_bwd_W")
        lib = _C.load()
        sdbe, sdbn = (Db.stride(0), Db.stride(1)) if Db is not None else (0, 0)
        with _C.on_device(DY.device):
            rc = lib.smoe_groupXtY(
                _C.ptr(DY), DY.stride(0), DY.stride(1),
                _C.ptr(X), X.stride(0), X.stride(1),
                _C.ptr(DW), DW.stride(0), DW.stride(1), DW.stride(2),
                _C.ptr(Db), sdbe, sdbn,
                _C.ptr(off), DY.size(0), X.size(1), DY.size(1), E, _C.float_code(DY.dtype),
                _C.stream_ptr(DY.device))
        _C.check(rc, "smoe_groupXtY")

    @staticmethod
    def xty_gathered(DY, X, idx, fan_out, DW, Db, off, E):
        """groupXtY with X read through idx; False when the library has no such kernel for this call."""
        _C.require_gpu(DY, "group_bwd_W")
        lib = _C.load()
        sdbe, sdbn = (Db.stride(0), Db.stride(1)) if Db is not None else (0, 0)
        with _C.on_device(DY.device):
            rc = lib.smoe_groupXtY_gathered(
                _C.ptr(DY), DY.stride(0), DY.stride(1),
                _C.ptr(X), X.stride(0), X.stride(1), _C.ptr(idx), fan_out,
                _C.ptr(DW), DW.stride(0), DW.stride(1), DW.stride(2),
                _C.ptr(Db), sdbe, sdbn,
                _C.ptr(off), DY.size(0), X.size(1), DY.size(1), E, _C.float_code(DY.dtype),
                _C.stream_ptr(DY.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_groupXtY_gathered")
        return True

    @staticmethod
    def combine(Y, gates, out, k):
        _C.require_gpu(Y, "combine")
        lib = _C.load()
        with _C.on_device(Y.device):
            sg = (gates.stride(0), gates.stride(1)) if gates is not None else (0, 0)
            rc = lib.smoe_combine(_C.ptr(Y), Y.stride(0), _C.ptr(gates), sg[0], sg[1],
                                  _C.ptr(out), out.stride(0), out.size(0), k, Y.size(1),
                                  _C.float_code(Y.dtype), _C.stream_ptr(Y.device))
        _C.check(rc, "smoe_combine")

    @staticmethod
    def gate_grad(Y, d_out, d_gates, k):
        _C.require_gpu(Y, "gate_grad")
        lib = _C.load()
        with _C.on_device(Y.device):
            rc = lib.smoe_gate_grad(_C.ptr(Y), Y.stride(0), _C.ptr(d_out), d_out.stride(0),
                                    _C.ptr(d_gates), d_gates.stride(0), d_gates.stride(1),
                                    d_out.size(0), k, Y.size(1), _C.float_code(Y.dtype),
                                    _C.stream_ptr(Y.device))
        _C.check(rc, "smoe_gate_grad")

    @staticmethod
    def gate_grad_group(Y, d_out, gates, idx, inverse, dy, d_gates, k):
        """Gate gradient + scaled expert-sorted copy of d_out in one pass; False if the library declines."""
        _C.require_gpu(Y, "gate_grad_group")
        lib = _C.load()
        with _C.on_device(Y.device):
            rc = lib.smoe_gate_grad_group(_C.ptr(Y), Y.stride(0), _C.ptr(d_out), d_out.stride(0),
                                          _C.ptr(gates), gates.stride(0), gates.stride(1), _C.ptr(idx), _C.ptr(inverse),
                                          _C.ptr(dy), dy.stride(0), _C.ptr(d_gates), d_gates.stride(0), d_gates.stride(1),
                                          d_out.size(0), k, Y.size(1), _C.float_code(Y.dtype), _C.stream_ptr(Y.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_gate_grad_group")
        return True

    @staticmethod
    def glu_fwd(pre, h, act):
        _C.require_gpu(pre, "glu_fwd")
        lib = _C.load()
        with _C.on_device(pre.device):
            rc = lib.smoe_glu_fwd(_C.ptr(pre), pre.stride(0), _C.ptr(h), h.stride(0), pre.size(0), h.size(1),
                                  act, _C.float_code(pre.dtype), _C.stream_ptr(pre.device))
        _C.check(rc, "smoe_glu_fwd")

    @staticmethod
    def glu_bwd(pre, dh, dpre, act):
        _C.require_gpu(pre, "glu_bwd")
        lib = _C.load()
        with _C.on_device(pre.device):
            rc = lib.smoe_glu_bwd(_C.ptr(pre), pre.stride(0), _C.ptr(dh), dh.stride(0), _C.ptr(dpre),
                                  dpre.stride(0), pre.size(0), dh.size(1), act, _C.float_code(pre.dtype),
                                  _C.stream_ptr(pre.device))
        _C.check(rc, "smoe_glu_bwd")

    @staticmethod
    def s2s_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, act):
        """Fused layer-1 GEMM + GLU; False when the library has no fused kernel for this call."""
        _C.require_gpu(X, "scatter2scatter_glu")
        lib = _C.load()
        sbe, sbn = (b.stride(0), b.stride(1)) if b is not None else (0, 0)
        with _C.on_device(X.device):
            rc = lib.smoe_scatter2scatter_glu(
                _C.ptr(X), X.stride(0), X.stride(1),
                _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                _C.ptr(b), sbe, sbn,
                _C.ptr(pre), pre.stride(0) if pre is not None else 0, _C.ptr(h), h.stride(0),
                _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                eid.numel(), X.size(1), h.size(1), W.size(0), k, int(bool(x_grouped)), act,
                _C.float_code(X.dtype), _C.stream_ptr(X.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_scatter2scatter_glu")
        return True

    @staticmethod
    def s2s_glu_bwd(DY, W, pre, dpre, eid, idx, off, act):
        """Fused layer-2 input gradient + GLU gradient; False when there is no fused kernel for this call."""
        _C.require_gpu(DY, "scatter2scatter_glu_bwd")
        lib = _C.load()
        with _C.on_device(DY.device):
            rc = lib.smoe_scatter2scatter_glu_bwd(
                _C.ptr(DY), DY.stride(0), DY.stride(1),
                _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                _C.ptr(pre), pre.stride(0), _C.ptr(dpre), dpre.stride(0),
                _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                eid.numel(), DY.size(1), W.size(2), W.size(0), act,
                _C.float_code(DY.dtype), _C.stream_ptr(DY.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_scatter2scatter_glu_bwd")
        return True


    @staticmethod
    def s2s_oss_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, alpha, limit):
        """Fused layer-1 GEMM + gpt-oss gated unit; False when the library has no fused kernel for this call."""
        _C.require_gpu(X, "scatter2scatter_glu")
        lib = _C.load()
        sbe, sbn = (b.stride(0), b.stride(1)) if b is not None else (0, 0)
        with _C.on_device(X.device):
            rc = lib.smoe_scatter2scatter_oss_glu(
                _C.ptr(X), X.stride(0), X.stride(1), _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                _C.ptr(b), sbe, sbn, _C.ptr(pre), pre.stride(0) if pre is not None else 0, _C.ptr(h), h.stride(0),
                _C.ptr(eid), _C.ptr(idx), _C.ptr(off), eid.numel(), X.size(1), h.size(1), W.size(0), k,
                int(bool(x_grouped)), alpha, limit, _C.float_code(X.dtype), _C.stream_ptr(X.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_scatter2scatter_oss_glu")
        return True

    @staticmethod
    def s2s_oss_glu_bwd(DY, W, pre, dpre, eid, idx, off, alpha, limit):
        _C.require_gpu(DY, "scatter2scatter_glu_bwd")
        lib = _C.load()
        with _C.on_device(DY.device):
            rc = lib.smoe_scatter2scatter_oss_glu_bwd(
                _C.ptr(DY), DY.stride(0), DY.stride(1), _C.ptr(W), W.stride(0), W.stride(1), W.stride(2),
                _C.ptr(pre), pre.stride(0), _C.ptr(dpre), dpre.stride(0), _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                eid.numel(), DY.size(1), W.size(2), W.size(0), alpha, limit, _C.float_code(DY.dtype),
                _C.stream_ptr(DY.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_scatter2scatter_oss_glu_bwd")
        return True

    @staticmethod
    def oss_glu_fwd(pre, h, alpha, limit):
        _C.require_gpu(pre, "gpt_oss_glu")
        lib = _C.load()
        with _C.on_device(pre.device):
            rc = lib.smoe_gpt_oss_glu_fwd(_C.ptr(pre), pre.stride(0), _C.ptr(h), h.stride(0), pre.size(0), h.size(1),
                                          alpha, limit, _C.float_code(pre.dtype), _C.stream_ptr(pre.device))
        _C.check(rc, "smoe_gpt_oss_glu_fwd")

    @staticmethod
    def oss_glu_bwd(pre, dh, dpre, alpha, limit):
        _C.require_gpu(pre, "gpt_oss_glu backward")
        lib = _C.load()
        with _C.on_device(pre.device):
            rc = lib.smoe_gpt_oss_glu_bwd(_C.ptr(pre), pre.stride(0), _C.ptr(dh), dh.stride(0), _C.ptr(dpre),
                                          dpre.stride(0), pre.size(0), dh.size(1), alpha, limit,
                                          _C.float_code(pre.dtype), _C.stream_ptr(pre.device))
        _C.check(rc, "smoe_gpt_oss_glu_bwd")

    @staticmethod
    def decode_glu_mlp(x, experts, gates, w1, b1, w2, b2, h, out, act):
        """Whole gated MLP of a decode step; False when the library has no such kernel for this call."""
        _C.require_gpu(x, "decode_glu_mlp")
        lib = _C.load()
        sb1 = (b1.stride(0), b1.stride(1)) if b1 is not None else (0, 0)
        sb2 = (b2.stride(0), b2.stride(1)) if b2 is not None else (0, 0)
        with _C.on_device(x.device):
            rc = lib.smoe_decode_glu_mlp(
                _C.ptr(x), x.stride(0), _C.ptr(experts), experts.stride(0), experts.stride(1),
                _C.ptr(gates), gates.stride(0), gates.stride(1),
                _C.ptr(w1), w1.stride(0), w1.stride(1), _C.ptr(b1), sb1[0], sb1[1],
                _C.ptr(w2), w2.stride(0), w2.stride(1), _C.ptr(b2), sb2[0], sb2[1],
                _C.ptr(h), h.stride(0), _C.ptr(out), out.stride(0),
                x.size(0), experts.size(1), x.size(1), h.size(1), w1.size(0), act,
                _C.float_code(x.dtype), _C.stream_ptr(x.device))
        if rc == _C.ERR_UNSUPPORTED:
            return False
        _C.check(rc, "smoe_decode_glu_mlp")
        return True

    @staticmethod
    def topk_softmax(logits, weights, experts, renormalize):
        _C.require_gpu(logits, "topk_softmax")
        lib = _C.load()
        with _C.on_device(logits.device):
            rc = lib.smoe_topk_softmax(_C.ptr(logits), logits.stride(0), logits.stride(1), logits.size(0),
                                       logits.size(1), weights.size(1), int(bool(renormalize)),
                                       _C.ptr(weights), weights.stride(0), weights.stride(1),
                                       _C.ptr(experts), experts.stride(0), experts.stride(1),
                                       _C.float_code(logits.dtype), _C.stream_ptr(logits.device))
        _C.check(rc, "smoe_topk_softmax")


_backend = HipBackend()


# ------------------------------------------------------------------------------------------------
# Under torch.compile every launch has to be an operator the tracer knows (it cannot look inside a ctypes call).
# The three kernels of the reference are registered further down under the reference's own operator names; the
# remaining launches of this build are registered here.  All of them write into buffers the caller allocated.
# ------------------------------------------------------------------------------------------------
@torch.library.custom_op("scattermoe::route", mutates_args={"eid", "idx", "off"})
def _route_op(flat_ids: torch.Tensor, num_experts: int, eid: torch.Tensor, idx: torch.Tensor,
              off: torch.Tensor) -> None:
    _backend.route(flat_ids, num_experts, eid, idx, off)


@torch.library.custom_op("scattermoe::offsets", mutates_args={"off"})
def _offsets_op(eid: torch.Tensor, num_experts: int, off: torch.Tensor) -> None:
    _backend.offsets(eid, num_experts, off)


@torch.library.custom_op("scattermoe::combine", mutates_args={"out"})
def _combine_op(Y: torch.Tensor, gates: Optional[torch.Tensor], out: torch.Tensor, k: int) -> None:
    _backend.combine(Y, gates, out, k)


@torch.library.custom_op("scattermoe::gate_grad", mutates_args={"d_gates"})
def _gate_grad_op(Y: torch.Tensor, d_out: torch.Tensor, d_gates: torch.Tensor, k: int) -> None:
    _backend.gate_grad(Y, d_out, d_gates, k)


@torch.library.custom_op("scattermoe::gate_grad_group", mutates_args={"dy", "d_gates"})
def _gate_grad_group_op(Y: torch.Tensor, d_out: torch.Tensor, gates: torch.Tensor, idx: torch.Tensor, dy: torch.Tensor,
                        d_gates: torch.Tensor, k: int) -> None:
    _gate_grad_group_launch(Y, d_out, gates, idx, dy, d_gates, k)


def _gate_grad_group_launch(Y, d_out, gates, idx, dy, d_gates, k):
    inverse = torch.empty(idx.numel(), dtype=torch.int32, device=Y.device)
    if not (hasattr(_backend, "gate_grad_group")
            and _backend.gate_grad_group(Y, d_out, gates, idx, inverse, dy, d_gates, k)):
        _backend.gate_grad(Y, d_out, d_gates, k)                       # the two passes it stands for
        _group_launch(d_out, dy, gates.reshape(-1), k, idx, True)


@torch.library.custom_op("scattermoe::glu_fwd", mutates_args={"h"})
def _glu_fwd_op(pre: torch.Tensor, h: torch.Tensor, act: int) -> None:
    _backend.glu_fwd(pre, h, act)


@torch.library.custom_op("scattermoe::glu_bwd", mutates_args={"dpre"})
def _glu_bwd_op(pre: torch.Tensor, dh: torch.Tensor, dpre: torch.Tensor, act: int) -> None:
    _backend.glu_bwd(pre, dh, dpre, act)


@torch.library.custom_op("scattermoe::gpt_oss_glu_fwd", mutates_args={"h"})
def _oss_glu_fwd_op(pre: torch.Tensor, h: torch.Tensor, alpha: float, limit: float) -> None:
    _backend.oss_glu_fwd(pre, h, alpha, limit)


@torch.library.custom_op("scattermoe::gpt_oss_glu_bwd", mutates_args={"dpre"})
def _oss_glu_bwd_op(pre: torch.Tensor, dh: torch.Tensor, dpre: torch.Tensor, alpha: float, limit: float) -> None:
    _backend.oss_glu_bwd(pre, dh, dpre, alpha, limit)


@torch.library.custom_op("scattermoe::topk_softmax", mutates_args={"weights", "experts"})
def _topk_softmax_op(logits: torch.Tensor, weights: torch.Tensor, experts: torch.Tensor,
                     renormalize: bool) -> None:
    _backend.topk_softmax(logits, weights, experts, renormalize)


@torch.library.custom_op("scattermoe::scatter2scatter_glu", mutates_args={"pre", "h"})
def _s2s_glu_op(X: torch.Tensor, W: torch.Tensor, b: Optional[torch.Tensor], pre: Optional[torch.Tensor],
                h: torch.Tensor, eid: torch.Tensor, idx: torch.Tensor, off: torch.Tensor, k: int,
                x_grouped: bool, act: int) -> None:
    if not _backend.s2s_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, act):   # no fused kernel: two launches
        tmp = pre if pre is not None else torch.empty((h.size(0), 2 * h.size(1)), dtype=h.dtype, device=h.device)
        _backend.s2s(X, W, b, tmp, eid, idx, off, k, x_grouped, True)
        _backend.glu_fwd(tmp, h, act)


@torch.library.custom_op("scattermoe::scatter2scatter_oss_glu", mutates_args={"pre", "h"})
def _s2s_oss_glu_op(X: torch.Tensor, W: torch.Tensor, b: Optional[torch.Tensor], pre: Optional[torch.Tensor],
                    h: torch.Tensor, eid: torch.Tensor, idx: torch.Tensor, off: torch.Tensor, k: int,
                    x_grouped: bool, alpha: float, limit: float) -> None:
    if not _backend.s2s_oss_glu(X, W, b, pre, h, eid, idx, off, k, x_grouped, alpha, limit):
        tmp = pre if pre is not None else torch.empty((h.size(0), 2 * h.size(1)), dtype=h.dtype, device=h.device)
        _backend.s2s(X, W, b, tmp, eid, idx, off, k, x_grouped, True)
        _backend.oss_glu_fwd(tmp, h, alpha, limit)


@torch.library.custom_op("scattermoe::scatter2scatter_oss_glu_bwd", mutates_args={"dpre"})
def _s2s_oss_glu_bwd_op(DY: torch.Tensor, W: torch.Tensor, pre: torch.Tensor, dpre: torch.Tensor, eid: torch.Tensor,
                        idx: torch.Tensor, off: torch.Tensor, alpha: float, limit: float) -> None:
    if not _backend.s2s_oss_glu_bwd(DY, W, pre, dpre, eid, idx, off, alpha, limit):
        dh = torch.empty((DY.size(0), W.size(2)), dtype=DY.dtype, device=DY.device)
        _backend.s2s(DY, W, None, dh, eid, idx, off, 1, True, True)
        _backend.oss_glu_bwd(pre, dh, dpre, alpha, limit)


@torch.library.custom_op("scattermoe::scatter2scatter_glu_bwd", mutates_args={"dpre"})
def _s2s_glu_bwd_op(DY: torch.Tensor, W: torch.Tensor, pre: torch.Tensor, dpre: torch.Tensor, eid: torch.Tensor,
                    idx: torch.Tensor, off: torch.Tensor, act: int) -> None:
    if not _backend.s2s_glu_bwd(DY, W, pre, dpre, eid, idx, off, act):
        dh = torch.empty((DY.size(0), W.size(2)), dtype=DY.dtype, device=DY.device)
        _backend.s2s(DY, W, None, dh, eid, idx, off, 1, True, True)
        _backend.glu_bwd(pre, dh, dpre, act)


_COMPILED_OPS = {"route": _route_op, "offsets": _offsets_op, "combine": _combine_op, "gate_grad": _gate_grad_op,
                 "glu_fwd": _glu_fwd_op, "glu_bwd": _glu_bwd_op, "topk_softmax": _topk_softmax_op,
                 "oss_glu_fwd": _oss_glu_fwd_op, "oss_glu_bwd": _oss_glu_bwd_op}


def _launch(name, *args):
    """`_backend.<name>(*args)`, through the registered operator while a compiler is tracing."""
    if torch.compiler.is_compiling():
        return _COMPILED_OPS[name](*args)
    return getattr(_backend, name)(*args)


def _same_dtype(what, ref, *others):
    for t in others:
        if t is not None and t.dtype != ref.dtype:
            raise TypeError("%s: dtype mismatch (%s vs %s)" % (what, ref.dtype, t.dtype))


def _as_i64(t):
    return t if t.dtype == torch.int64 else t.to(torch.int64)


# ------------------------------------------------------------------------------------------------
# routing prep
# ------------------------------------------------------------------------------------------------
def route(expert_idxs: torch.Tensor, num_experts: int):
    """Stable sort of the flattened expert ids; returns (sorted ids, source slots, inclusive offsets)."""
    flat = expert_idxs.reshape(-1)
    if not flat.is_contiguous():
        flat = flat.contiguous()
    if flat.dtype not in (torch.int64, torch.int32, torch.int16, torch.uint8):
        flat = flat.to(torch.int64)
    L = flat.numel()
    eid = torch.empty(L, dtype=torch.int64, device=flat.device)
    idx = torch.empty(L, dtype=torch.int64, device=flat.device)
    off = torch.empty(num_experts, dtype=torch.int64, device=flat.device)
    _launch("route", flat, num_experts, eid, idx, off)
    return eid, idx, off


def offsets_from_sorted(sorted_expert_idxs: torch.Tensor, num_experts: int):
    off = torch.empty(num_experts, dtype=torch.int64, device=sorted_expert_idxs.device)
    _launch("offsets", _as_i64(sorted_expert_idxs).contiguous(), num_experts, off)
    return off


# ------------------------------------------------------------------------------------------------
# scatter2scatter
# ------------------------------------------------------------------------------------------------
def scatter2scatter(X, W, sorted_expert_idxs, sorted_scattered_idxs, k,
                    b=None, x_grouped=False, y_grouped=False, out=None, expert_offsets=None):
    """Y[dst(n)] = X[src(n)] @ W[eid[n]] (+ b[eid[n]]) over the L expert-sorted rows.

    Same contract as the reference wrapper (ops.py:120-137).  `expert_offsets` is an optional extra:
    callers that already hold the inclusive offsets pass them and save one small launch.
    """
    L = sorted_expert_idxs.size(0)
    assert sorted_scattered_idxs.size(0) == L
    assert L == X.size(0) * k
    assert W.dim() == 3 and W.size(1) == X.size(1)
    N = W.size(-1)
    given = out
    if out is None:
        out = torch.empty((L, N), device=X.device, dtype=X.dtype)
    else:
        assert out.size(0) == L and out.size(1) == N
    if torch.compiler.is_compiling():
        if expert_offsets is None:
            scatter2scatter_compileable(out, W, X, k, sorted_expert_idxs, sorted_scattered_idxs,
                                        b, x_grouped, y_grouped)
        else:       # same launch, without deriving the offsets again from the sorted ids
            _s2s_offsets_op(out, W, X, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                            b, x_grouped, y_grouped)
    else:
        _s2s_launch(out, W, X, k, sorted_expert_idxs, sorted_scattered_idxs, b,
                    x_grouped, y_grouped, expert_offsets)
        _wrote_into(given)
    return out


def _s2s_launch(out, W, X, k, eid, idx, b, x_grouped, y_grouped, off):
    _same_dtype("scatter2scatter", X, W, b, out)
    eid, idx = _as_i64(eid).contiguous(), _as_i64(idx).contiguous()
    if off is None:
        off = offsets_from_sorted(eid, W.size(0))
    else:
        off = _as_i64(off).contiguous()
        assert off.numel() == W.size(0)
    _backend.s2s(X, W, b, out, eid, idx, off, k, x_grouped, y_grouped)


@torch.library.custom_op("scattermoe::scatter2scatter", mutates_args={"output"})
def scatter2scatter_compileable(
        output: torch.Tensor, W: torch.Tensor, X: torch.Tensor, k: int,
        sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor,
        b: Optional[torch.Tensor], x_grouped: bool, y_grouped: bool) -> None:
    _s2s_launch(output, W, X, k, sorted_expert_idxs, sorted_scattered_idxs, b, x_grouped, y_grouped, None)


@torch.library.custom_op("scattermoe::scatter2scatter_offsets", mutates_args={"output"})
def _s2s_offsets_op(
        output: torch.Tensor, W: torch.Tensor, X: torch.Tensor, k: int,
        sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor,
        b: Optional[torch.Tensor], x_grouped: bool, y_grouped: bool) -> None:
    """scattermoe::scatter2scatter for callers that hold the expert offsets (the reference's schema has no such
    argument: its kernel finds the expert boundaries itself)."""
    _s2s_launch(output, W, X, k, sorted_expert_idxs, sorted_scattered_idxs, b, x_grouped, y_grouped, expert_offsets)


# ------------------------------------------------------------------------------------------------
# groupXtY
# ------------------------------------------------------------------------------------------------
def group_bwd_W(DY, X, expert_offsets, E, has_bias=False, like=None, gather=None):
    """Per-expert dW / db over expert-grouped rows (reference ops.py:191-199).

    `gather=(sorted_scattered_idxs, fan_out)`: X is not the grouped (L, K) matrix but the (L / fan_out, K) matrix it
    would be gathered from, i.e. the call stands for `group_bwd_W(DY, group(X, idxs, fan_out=fan_out), ...)`
    (reference parallel_experts.py:95-107) without the gathered copy ever being written.

    The returned DW is (E, K, N).  By default it is a view of a contiguous (E, N, K) buffer, so that after autograd
    undoes the `weight.permute(0, 2, 1)` of ParallelExperts the parameter gradient is contiguous.  `like` (the
    (E, K, N) weight the gradient belongs to) overrides that: a weight stored with N contiguous (the gpt-oss
    parameters) gets a gradient stored the same way, so that accumulating it into `.grad` is not a transposing
    copy of the whole tensor.  The kernel writes every element (zeros for experts without rows), hence `empty`.
    """
    N, K = DY.size(-1), X.size(-1)
    if like is not None and like.dim() == 3 and like.stride(2) == 1 and like.stride(1) != 1:
        DW = torch.empty((E, K, N), device=DY.device, dtype=DY.dtype)
    else:
        DW = torch.empty((E, N, K), device=DY.device, dtype=DY.dtype).permute(0, 2, 1)
    Db = torch.empty((E, N), device=DY.device, dtype=DY.dtype) if has_bias else None
    if gather is not None:
        idx, fan_out = gather
        assert idx.size(0) == DY.size(0) and X.size(0) * fan_out == DY.size(0)
        if torch.compiler.is_compiling():
            _xty_gathered_op(E, DW, Db, DY, X, idx, fan_out, expert_offsets)
        else:
            _xty_gathered_launch(E, DW, Db, DY, X, idx, fan_out, expert_offsets)
        return DW, Db
    if torch.compiler.is_compiling():
        groupXtY_compileable(E, DW, Db, DY, X, expert_offsets)
    else:
        _xty_launch(E, DW, Db, DY, X, expert_offsets)
    return DW, Db


def _xty_launch(E, DW, Db, DY, X, expert_offsets):
    assert DY.size(0) == X.size(0)
    assert expert_offsets.numel() == E
    _same_dtype("group_bwd_W", DY, X, DW, Db)
    _backend.xty(DY, X, DW, Db, _as_i64(expert_offsets).contiguous(), E)


def _xty_gathered_launch(E, DW, Db, DY, X, idx, fan_out, expert_offsets):
    """groupXtY over X[idx // fan_out]: one launch that reads the rows of X through idx where the library has one,
    else the gathered copy and the plain launch."""
    if DY.is_cuda and hasattr(_backend, "xty_gathered") and DY.dtype in (torch.bfloat16, torch.float16):
        _same_dtype("group_bwd_W", DY, X, DW, Db)
        if _backend.xty_gathered(DY, X, _as_i64(idx).contiguous(), fan_out, DW, Db,
                                 _as_i64(expert_offsets).contiguous(), E):
            return
    Xg = torch.empty((idx.size(0), X.size(1)), dtype=X.dtype, device=X.device)
    _group_launch(X, Xg, None, fan_out, idx, True)            # `idx` is the routing's index vector
    _xty_launch(E, DW, Db, DY, Xg, expert_offsets)


@torch.library.custom_op("scattermoe::groupXtY_gathered", mutates_args={"DW", "Db"})
def _xty_gathered_op(E: int, DW: torch.Tensor, Db: Optional[torch.Tensor], DY: torch.Tensor, X: torch.Tensor,
                     idx: torch.Tensor, fan_out: int, expert_offsets: torch.Tensor) -> None:
    _xty_gathered_launch(E, DW, Db, DY, X, idx, fan_out, expert_offsets)


@torch.library.custom_op("scattermoe::groupXtY", mutates_args={"DW", "Db"})
def groupXtY_compileable(E: int, DW: torch.Tensor, Db: Optional[torch.Tensor],
                         DY: torch.Tensor, X: torch.Tensor, expert_offsets: torch.Tensor) -> None:
    _xty_launch(E, DW, Db, DY, X, expert_offsets)


# ------------------------------------------------------------------------------------------------
# group
# ------------------------------------------------------------------------------------------------
def group(A, sorted_expert_idxs, coeff=None, fan_out=1, out=None, permutation=False):
    """Y[n] = A[idx[n] // fan_out] * coeff[idx[n]]  (reference ops.py:377-386).

    As in the reference the second argument is, despite its name, the sorted *scattered* index vector.
    `permutation=True` (not in the reference) says that it is a permutation of range(N), as the routing's is: with
    fan_out > 1 the rows of A are then read once each instead of fan_out times; same result.
    """
    N, K = sorted_expert_idxs.size(0), A.size(1)
    assert A.size(0) * fan_out == N
    Y = out if out is not None else torch.empty((N, K), dtype=A.dtype, device=A.device)
    if torch.compiler.is_compiling():
        if permutation:
            _group_permutation_op(A, K, N, Y, coeff, coeff is not None, fan_out, sorted_expert_idxs)
        else:
            group_compileable(A, K, N, Y, coeff, coeff is not None, fan_out, sorted_expert_idxs)
    else:
        _group_launch(A, Y, coeff, fan_out, sorted_expert_idxs, permutation)
        _wrote_into(out)
    return Y


def _group_launch(A, Y, coeff, fan_out, idx, permutation=False):
    assert Y.size(0) == idx.size(0) and Y.size(1) == A.size(1)
    _same_dtype("group", A, Y)
    if coeff is not None:
        assert coeff.numel() == idx.size(0)
        coeff = coeff.reshape(-1).to(A.dtype).contiguous()
    idx = _as_i64(idx).contiguous()
    if permutation and fan_out > 1 and A.is_cuda and hasattr(_backend, "group_by_source"):
        inverse = torch.empty(idx.numel(), dtype=torch.int32, device=A.device)
        if _backend.group_by_source(A, coeff, Y, idx, inverse, fan_out):
            return
    _backend.group(A, coeff, Y, idx, fan_out)


@torch.library.custom_op("scattermoe::group", mutates_args={"Y"})
def group_compileable(A: torch.Tensor, K: int, N: int, Y: torch.Tensor, coeff: Optional[torch.Tensor],
                      has_coeff: bool, fan_out: int, sorted_expert_idxs: torch.Tensor) -> None:
    _group_launch(A, Y, coeff if has_coeff else None, fan_out, sorted_expert_idxs)


@torch.library.custom_op("scattermoe::group_permutation", mutates_args={"Y"})
def _group_permutation_op(A: torch.Tensor, K: int, N: int, Y: torch.Tensor, coeff: Optional[torch.Tensor],
                          has_coeff: bool, fan_out: int, sorted_expert_idxs: torch.Tensor) -> None:
    """scattermoe::group for an index vector known to be a permutation (the routing's): same schema, same result,
    every source row read once."""
    _group_launch(A, Y, coeff if has_coeff else None, fan_out, sorted_expert_idxs, True)


# ------------------------------------------------------------------------------------------------
# fused passes around the expert GEMMs
# ------------------------------------------------------------------------------------------------
ACT_SILU = 0               # h = silu(second half) * first half   (GLUMLP of the reference)
ACT_SILU_GATE_FIRST = 1    # h = silu(first half) * second half   (Hugging Face `act(gate) * up`)
ACT_GPT_OSS = 2            # (gate, up) in adjacent columns, clamps, (up + 1) * gate * sigmoid(alpha * gate)


def _rows_contiguous(t):
    return t if t.stride(-1) == 1 else t.contiguous()


def combine(expanded, gates=None):
    """out[t] = sum_j gates[t, j] * expanded[t, j]  for expanded (T, k, N) -> (T, N)
    (the bmm of reference parallel_experts.py:44-46 as one HBM pass).  Without gates: the plain sum over the k
    slots, accumulated in float32 in slot order and rounded once (the `.sum(-2)` of parallel_experts.py:120-123)."""
    T, k, N = expanded.shape
    assert gates is None or gates.shape == (T, k)
    Y = _rows_contiguous(expanded.reshape(T * k, N))
    out = torch.empty((T, N), dtype=expanded.dtype, device=expanded.device)
    _launch("combine", Y, None if gates is None else gates.to(expanded.dtype), out, k)
    return out


def slot_sum(expanded_rows, T, k):
    """(T*k, N) rows in slot order -> (T, N): sum over each token's k slots (one pass, no gates)."""
    if k == 1:
        return expanded_rows
    return combine(expanded_rows.view(T, k, expanded_rows.size(-1)))


def _wrote_into(t):
    """A launch has overwritten `t` behind autograd's back: tell the version counter, so that a graph that saved
    `t` earlier refuses to run backward a second time instead of reading the new contents (the reference gets
    the same check from its mutating custom ops, e.g. `group` with mutates_args={'Y'}, ops.py:389)."""
    if t is not None and not torch.compiler.is_compiling():
        torch.autograd.graph.increment_version(t)


def gate_grad(expanded, grad_out):
    """d_gates[t, j] = <expanded[t, j], grad_out[t]>  (the bmm of reference parallel_experts.py:79)."""
    T, k, N = expanded.shape
    assert grad_out.shape == (T, N)
    Y = _rows_contiguous(expanded.reshape(T * k, N))
    d_gates = torch.empty((T, k), dtype=expanded.dtype, device=expanded.device)
    _launch("gate_grad", Y, _rows_contiguous(grad_out), d_gates, k)
    return d_gates


def gate_grad_group(expanded, grad_out, gates, sorted_scattered_idxs):
    """(d_gates, dy): `gate_grad(expanded, grad_out)` and `group(grad_out, idxs, coeff=gates.flatten(), fan_out=k)`
    - the first two steps of the backward of a gate-weighted expert layer (reference parallel_experts.py:76-93) -
    in one pass that reads grad_out from memory once.  dy is a new (T * k, N) buffer in expert-sorted order (the
    reference reuses the buffer of `expanded`, which a single pass cannot: it reads and writes different rows at the
    same time).  `sorted_scattered_idxs` must be the routing's permutation of range(T * k)."""
    T, k, N = expanded.shape
    assert grad_out.shape == (T, N) and gates.shape == (T, k) and sorted_scattered_idxs.numel() == T * k
    Y = _rows_contiguous(expanded.reshape(T * k, N))
    d_out = _rows_contiguous(grad_out)
    g = gates.to(expanded.dtype)
    idx = _as_i64(sorted_scattered_idxs).contiguous()
    dy = torch.empty((T * k, N), dtype=expanded.dtype, device=expanded.device)
    d_gates = torch.empty((T, k), dtype=expanded.dtype, device=expanded.device)
    if torch.compiler.is_compiling():
        _gate_grad_group_op(Y, d_out, g, idx, dy, d_gates, k)
    else:
        _same_dtype("gate_grad_group", Y, d_out)
        _gate_grad_group_launch(Y, d_out, g, idx, dy, d_gates, k)
    return d_gates, dy


def glu_fwd(pre, act=ACT_SILU):
    """h = act(pre[:, f:]) * pre[:, :f] for pre (rows, 2f)."""
    assert pre.dim() == 2 and pre.size(1) % 2 == 0
    pre = _rows_contiguous(pre)
    h = torch.empty((pre.size(0), pre.size(1) // 2), dtype=pre.dtype, device=pre.device)
    _launch("glu_fwd", pre, h, act)
    return h


def glu_bwd(pre, dh, act=ACT_SILU):
    pre, dh = _rows_contiguous(pre), _rows_contiguous(dh)
    assert dh.size(0) == pre.size(0) and 2 * dh.size(1) == pre.size(1)
    dpre = torch.empty_like(pre)
    _launch("glu_bwd", pre, dh, dpre, act)
    return dpre


class _GptOssGLU(torch.autograd.Function):
    """(up + 1) * gate * sigmoid(alpha * gate) over interleaved (gate, up) columns with the clamps of the gpt-oss
    experts, one pass each way; the pre-activation is saved and the sigmoid recomputed."""

    @staticmethod
    def forward(ctx, pre, alpha, limit):
        pre = _rows_contiguous(pre)
        ctx.save_for_backward(pre)
        ctx.alpha, ctx.limit = alpha, limit
        h = torch.empty((pre.size(0), pre.size(1) // 2), dtype=pre.dtype, device=pre.device)
        _launch("oss_glu_fwd", pre, h, alpha, limit)
        return h

    @staticmethod
    def backward(ctx, dh):
        (pre,) = ctx.saved_tensors
        dpre = torch.empty_like(pre)
        _launch("oss_glu_bwd", pre, _rows_contiguous(dh), dpre, ctx.alpha, ctx.limit)
        return dpre, None, None


def gpt_oss_glu(pre, alpha=1.702, limit=7.0):
    """Hidden layer of the gpt-oss experts from the (rows, 2f) layer-1 output with (gate, up) in adjacent columns
    (reference replace_moe.py:39-43): gate clamped from above and up clamped to [-limit, limit], then
    (up + 1) * gate * sigmoid(alpha * gate).  Differentiable."""
    assert pre.dim() == 2 and pre.size(1) % 2 == 0
    return _GptOssGLU.apply(pre, float(alpha), float(limit))


def scatter2scatter_glu(X, W, sorted_expert_idxs, sorted_scattered_idxs, k, b=None, x_grouped=False,
                        act=ACT_SILU, expert_offsets=None, need_pre=True, alpha=1.702, limit=7.0):
    """Layer 1 of a gated MLP with its GLU: returns (pre, h) with rows in expert-sorted order, where
    pre = scatter2scatter(X, W, ..., y_grouped=True) (L, 2F) and h = glu_fwd(pre) (L, F)
    (reference mlp.py:74-87; `act=ACT_GPT_OSS`: the gated unit of replace_moe.py:39-43 with `alpha`, `limit`).
    One fused launch where the library has one, the two calls otherwise (same results up to one unit in the last
    place of rare elements).  `need_pre=False` (inference) lets the fused launch skip storing `pre`."""
    L = sorted_expert_idxs.size(0)
    assert W.dim() == 3 and W.size(1) == X.size(1) and W.size(2) % 2 == 0
    assert L == (X.size(0) if x_grouped else X.size(0) * k)
    F = W.size(2) // 2
    oss = act == ACT_GPT_OSS
    if X.is_cuda and X.dtype in (torch.bfloat16, torch.float16) and hasattr(_backend, "s2s_glu"):
        _same_dtype("scatter2scatter_glu", X, W, b)
        off = expert_offsets if expert_offsets is not None else offsets_from_sorted(sorted_expert_idxs, W.size(0))
        pre = torch.empty((L, 2 * F), device=X.device, dtype=X.dtype) if need_pre else None
        h = torch.empty((L, F), device=X.device, dtype=X.dtype)
        args = (_rows_contiguous(X), W, b, pre, h, _as_i64(sorted_expert_idxs), _as_i64(sorted_scattered_idxs),
                _as_i64(off), k, x_grouped)
        if torch.compiler.is_compiling():       # the operators fall back to the two launches by themselves
            if oss:
                _s2s_oss_glu_op(*args, float(alpha), float(limit))
            else:
                _s2s_glu_op(*args, act)
            return pre, h
        elif (_backend.s2s_oss_glu(*args, float(alpha), float(limit)) if oss else _backend.s2s_glu(*args, act)):
            return pre, h
    pre = scatter2scatter(X, W, sorted_expert_idxs, sorted_scattered_idxs, k, b=b, x_grouped=x_grouped,
                          y_grouped=True, expert_offsets=expert_offsets)
    if oss:
        h = torch.empty((L, F), dtype=pre.dtype, device=pre.device)
        _launch("oss_glu_fwd", pre, h, float(alpha), float(limit))
        return pre, h
    return pre, glu_fwd(pre, act)


def scatter2scatter_glu_bwd(DY, W, pre, sorted_expert_idxs, sorted_scattered_idxs, act=ACT_SILU,
                            expert_offsets=None, alpha=1.702, limit=7.0):
    """d(pre) (L, 2F) from the grouped output gradient DY (L, K) of layer 2, its weights W (E, K, F) and the
    saved pre-activation: glu_bwd(pre, scatter2scatter(DY, W, grouped in and out)) in one launch where possible."""
    L = sorted_expert_idxs.size(0)
    assert DY.size(0) == L and pre.size(0) == L and pre.size(1) == 2 * W.size(2) and W.size(1) == DY.size(1)
    oss = act == ACT_GPT_OSS
    if DY.is_cuda and DY.dtype in (torch.bfloat16, torch.float16) and hasattr(_backend, "s2s_glu_bwd"):
        _same_dtype("scatter2scatter_glu_bwd", DY, W, pre)
        off = expert_offsets if expert_offsets is not None else offsets_from_sorted(sorted_expert_idxs, W.size(0))
        pre_c = _rows_contiguous(pre)
        dpre = torch.empty_like(pre_c)
        args = (_rows_contiguous(DY), W, pre_c, dpre, _as_i64(sorted_expert_idxs), _as_i64(sorted_scattered_idxs),
                _as_i64(off))
        if torch.compiler.is_compiling():
            if oss:
                _s2s_oss_glu_bwd_op(*args, float(alpha), float(limit))
            else:
                _s2s_glu_bwd_op(*args, act)
            return dpre
        elif (_backend.s2s_oss_glu_bwd(*args, float(alpha), float(limit)) if oss
              else _backend.s2s_glu_bwd(*args, act)):
            return dpre
    dh = scatter2scatter(DY, W, sorted_expert_idxs, sorted_scattered_idxs, 1, x_grouped=True, y_grouped=True,
                         expert_offsets=expert_offsets)
    if oss:
        pre_c = _rows_contiguous(pre)
        dpre = torch.empty_like(pre_c)
        _launch("oss_glu_bwd", pre_c, _rows_contiguous(dh), dpre, float(alpha), float(limit))
        return dpre
    return glu_bwd(pre, dh, act)


class _TopkSoftmax(torch.autograd.Function):
    """Forward in one launch; backward is the chain rule of gather -> (renormalise) -> softmax written with
    torch ops on the (T, E) probabilities, which are recomputed from the logits."""

    @staticmethod
    def forward(ctx, logits, k, renormalize):
        T, E = logits.shape
        weights = torch.empty((T, k), dtype=torch.float32, device=logits.device)
        experts = torch.empty((T, k), dtype=torch.int64, device=logits.device)
        _launch("topk_softmax", logits, weights, experts, renormalize)
        ctx.save_for_backward(logits, weights, experts)
        ctx.renormalize = renormalize
        ctx.mark_non_differentiable(experts)
        return weights, experts

    @staticmethod
    def backward(ctx, d_weights, _):
        logits, weights, experts = ctx.saved_tensors
        p = torch.softmax(logits.float(), dim=-1)
        d_sel = d_weights.float()
        if ctx.renormalize:
            s = p.gather(1, experts).sum(-1, keepdim=True)
            d_sel = (d_sel - (d_sel * weights).sum(-1, keepdim=True)) / s
        d_p = torch.zeros_like(p).scatter_(1, experts, d_sel)
        d_logits = p * (d_p - (d_p * p).sum(-1, keepdim=True))
        return d_logits.to(logits.dtype), None, None


def topk_softmax(router_logits, k, renormalize=True):
    """`w, i = topk(softmax(router_logits.float(), -1), k)`, then `w /= w.sum(-1, keepdim=True)` when
    `renormalize` (the routing of scattermoe/utils/replace_moe.py:67-71), in one launch.  Returns float32
    weights (T, k), in descending order, and int64 expert ids (T, k); equal probabilities are taken lowest
    expert id first."""
    if router_logits.dim() != 2:
        raise ValueError("router_logits must be (tokens, experts)")
    if not 0 < k <= router_logits.size(1):
        raise ValueError("k must be in 1..num_experts")
    return _TopkSoftmax.apply(router_logits, k, renormalize)


DECODE_MAX_ROWS = 8


def decode_glu_mlp(x, expert_p, expert_idxs, w1, b1, w2, b2, act=ACT_SILU):
    """Forward of a gated expert MLP for at most DECODE_MAX_ROWS (token, slot) rows in two launches, routing and
    gate combine included (reference GLUMLP.forward, mlp.py:74-95).  x (T, d), expert_p / expert_idxs (T, k),
    w1 (E, 2F, d) and w2 (E, d, F) in the ParallelExperts parameter layout.  Returns the (T, d) output, or None
    when this call is not the kernels' (more rows, float32, CPU tensors, a compiler tracing, unaligned operands):
    the caller then takes the general path, whose result these kernels reproduce bit for bit."""
    if (expert_idxs.numel() > DECODE_MAX_ROWS or expert_idxs.numel() == 0 or not x.is_cuda or x.dim() != 2
            or x.dtype not in (torch.bfloat16, torch.float16) or torch.compiler.is_compiling()
            or not hasattr(_backend, "decode_glu_mlp")
            or w1.stride(2) != 1 or w2.stride(2) != 1 or x.stride(1) != 1):
        return None
    _same_dtype("decode_glu_mlp", x, w1, w2, b1, b2)
    T, k = expert_idxs.shape
    F = w2.size(2)
    h = torch.empty((T * k, F), dtype=x.dtype, device=x.device)
    out = torch.empty((T, x.size(1)), dtype=x.dtype, device=x.device)
    if _backend.decode_glu_mlp(x, _as_i64(expert_idxs), expert_p.to(x.dtype), w1, b1, w2, b2, h, out, act):
        return out
    return None
