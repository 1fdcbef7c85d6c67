"""Fused edge-probability operators used by layer-wise samplers
(reference: python/gs/ops/fused_op.py:51-243).

  fused_u_mul_v : two u*v SDDMMs in one sweep over the edges
  e_square_sum  : out[t] = sum of e^2 over the edges of column (axis 0) / row (axis 1) t
  e_div_u_sum   : out[t] = sum of e / u[other endpoint]
"""
import torch

from ..format import _COO, _CSC, _CSR
from ._common import infer_broadcast_shape

torch.fx.wrap("_before_e_div_u_sum")

__all__ = ["fused_u_mul_v", "e_square_sum", "e_div_u_sum"]


def _before_e_div_u_sum(num_rows, num_cols, e, u, u_target):
    """Operands of _CAPI_FusedEDivUSum for the compiled rewrite of
    `div` followed by `sum`: both with the broadcast feature shape the two
    separate operators would have produced, and the zero-filled accumulator."""
    if u.device != e.device:
        raise ValueError(f"operand devices differ: {u.device} and {e.device}")
    if u.dtype != e.dtype:
        raise ValueError(f"operand dtypes differ: {u.dtype} and {e.dtype}")
    squeeze = e.dim() == 1 and u.dim() == 1
    e2 = e.unsqueeze(-1) if e.dim() == 1 else e
    u2 = u.unsqueeze(-1) if u.dim() == 1 else u
    feat = infer_broadcast_shape("div", tuple(e2.shape[1:]), tuple(u2.shape[1:]))
    e2 = e2.expand((e2.shape[0],) + feat).contiguous()
    u2 = u2.expand((u2.shape[0],) + feat).contiguous()
    n_out = num_cols if u_target == 0 else num_rows
    v = torch.zeros((n_out,) + feat, dtype=e.dtype, device=e.device)
    return u2, e2, v, squeeze


def fused_u_mul_v(m, lhs1, rhs1, lhs2, rhs2, on_format=_COO):
    g = m._graph
    if lhs1.device != rhs1.device:
        raise ValueError(f"operand devices differ: {lhs1.device} and {rhs1.device}")
    if lhs1.dtype != rhs1.dtype:
        raise ValueError(f"operand dtypes differ: {lhs1.dtype} and {rhs1.dtype}")
    exp_l = exp_r = False
    if lhs1.dim() == 1:
        lhs1, lhs2, exp_l = lhs1.unsqueeze(-1), lhs2.unsqueeze(-1), True
    if rhs1.dim() == 1:
        rhs1, rhs2, exp_r = rhs1.unsqueeze(-1), rhs2.unsqueeze(-1), True
    num_edges = g._CAPI_GetNumEdges()
    shape = (num_edges,) + infer_broadcast_shape("mul", tuple(lhs1.shape[1:]),
                                                 tuple(rhs1.shape[1:]))
    out1 = torch.zeros(shape, dtype=lhs1.dtype, device=lhs1.device)
    out2 = torch.zeros(shape, dtype=lhs1.dtype, device=lhs1.device)
    if num_edges > 0:
        g._CAPI_FusedUOPV("mul", lhs1, rhs1, out1, lhs2, rhs2, out2, on_format)
    if exp_l and exp_r:
        out1, out2 = out1.squeeze(-1), out2.squeeze(-1)
    return out1, out2


def _reduce_target(g, axis):
    if axis == 0:
        return g._CAPI_GetNumCols(), 0
    if axis == 1:
        return g._CAPI_GetNumRows(), 2
    raise ValueError("axis should be 0 or 1")


def e_square_sum(m, key, axis, on_format=_CSR) -> torch.Tensor:
    g = m._graph
    e = m.edata[key]
    n_out, u_target = _reduce_target(g, axis)
    if e.dim() == 1:
        e = e.unsqueeze(-1)
    v = torch.zeros((n_out,), dtype=e.dtype, device=e.device)
    if g._CAPI_GetNumEdges() > 0:
        fmt = _CSC if axis == 0 else on_format
        g._CAPI_FusedESquareSum("copy_rhs", "sum", None, e, v, None, None, u_target, fmt)
    return v


def e_div_u_sum(m, key, u, axis, on_format=_CSC) -> torch.Tensor:
    g = m._graph
    e = m.edata[key]
    if u.device != e.device:
        raise ValueError(f"operand devices differ: {u.device} and {e.device}")
    if u.dtype != e.dtype:
        raise ValueError(f"operand dtypes differ: {u.dtype} and {e.dtype}")
    n_out, u_target = _reduce_target(g, axis)
    if u.dim() == 1:
        u = u.unsqueeze(-1)
    if e.dim() == 1:
        e = e.unsqueeze(-1)
    v = torch.zeros((n_out,), dtype=e.dtype, device=e.device)
    if g._CAPI_GetNumEdges() > 0:
        g._CAPI_FusedEDivUSum("div", "sum", u, e, v, None, None, u_target, on_format)
    return v
