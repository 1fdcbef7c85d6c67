"""Generalized SpMM on a Matrix: out[v] = reduce over edges of op(u, e).
Wrapper around _CAPI_SpMM with the reference's calling convention
(python/gs/ops/spmm.py:109-124): u_target 0 reduces onto columns, 2 onto rows."""
import sys

import torch

from ..format import _CSC
from ._common import prepare_binary

torch.fx.wrap("_before_spmm")
torch.fx.wrap("_after_spmm")

__all__ = ["gspmm"]


def _before_spmm(num_rows, num_cols, op, reduce_op, lhs_data, rhs_data, lhs_target):
    u, e, feat, squeeze, dtype, device = prepare_binary(op, lhs_data, rhs_data)
    n_out = num_cols if lhs_target == 0 else num_rows
    shape = (n_out,) + tuple(feat)
    v = torch.zeros(shape, dtype=dtype, device=device)
    arg_u = arg_e = None
    if reduce_op in ("max", "min"):
        if op != "copy_rhs":
            arg_u = torch.zeros(shape, dtype=torch.int64, device=device)
        if op != "copy_lhs":
            arg_e = torch.zeros(shape, dtype=torch.int64, device=device)
    return v, arg_u, arg_e, squeeze


def _after_spmm(v, squeeze):
    return v.squeeze(-1) if squeeze else v


def gspmm(g, op, reduce_op, lhs_data, rhs_data, lhs_target, on_format):
    num_rows = g._graph._CAPI_GetNumRows()
    num_cols = g._graph._CAPI_GetNumCols()
    v, arg_u, arg_e, squeeze = _before_spmm(
        num_rows, num_cols, op, reduce_op, lhs_data, rhs_data, lhs_target)
    # the operands go in as given (scalar features stay 1-D): the operator
    # treats [n] and [n, 1] alike, and the traced graph keeps a direct
    # producer -> SpMM edge for the fusion passes to match
    g._graph._CAPI_SpMM(op, reduce_op, lhs_data, rhs_data, v, arg_u, arg_e, lhs_target,
                        on_format)
    return _after_spmm(v, squeeze)


def _register():
    mod = sys.modules[__name__]
    for op in ("add", "sub", "mul", "div"):
        for red in ("sum", "max", "min"):
            def func(g, x, y, on_format=_CSC, _op=op, _red=red):
                return gspmm(g, _op, _red, x, y, 0, on_format)
            func.__name__ = f"u_{op}_e_{red}"
            setattr(mod, func.__name__, func)
            __all__.append(func.__name__)
    for red in ("sum", "max", "min"):
        def copy_u(g, x, on_format=_CSC, _red=red):
            return gspmm(g, "copy_lhs", _red, x, None, 0, on_format)
        copy_u.__name__ = f"copy_u_{red}"
        setattr(mod, copy_u.__name__, copy_u)
        __all__.append(copy_u.__name__)

        def copy_e(g, x, on_format=_CSC, _red=red):
            return gspmm(g, "copy_rhs", _red, None, x, 0, on_format)
        copy_e.__name__ = f"copy_e_{red}"
        setattr(mod, copy_e.__name__, copy_e)
        __all__.append(copy_e.__name__)


_register()
