"""Generalized SDDMM on a Matrix: out[e] = lhs[t_l(e)] op rhs[t_r(e)].
Wrapper around _CAPI_SDDMM with the reference's calling convention
(python/gs/ops/sddmm.py:103-110)."""
import sys
from itertools import product

import torch

from ..format import _COO
from ._common import TARGET, prepare_binary

torch.fx.wrap("_before_sddmm")
torch.fx.wrap("_after_sddmm")

__all__ = ["gsddmm", "copy_u", "copy_v"]


def _before_sddmm(num_edges, op, lhs_data, rhs_data):
    lhs, rhs, feat, squeeze, dtype, device = prepare_binary(op, lhs_data, rhs_data)
    # every element is written by the operator: no need to clear it first
    out = torch.empty((num_edges,) + tuple(feat), dtype=dtype, device=device)
    return lhs, rhs, out, squeeze


def _after_sddmm(out, squeeze):
    return out.squeeze(-1) if squeeze else out


def gsddmm(g, op, lhs_data, rhs_data, lhs_target="u", rhs_target="v", on_format=_COO):
    num_edges = g._graph._CAPI_GetNumEdges()
    # sub and div go to the operator as they are (the reference's wrapper turns
    # them into add / mul of the negated / reciprocal operand first,
    # python/gs/ops/sddmm.py:20-25: two more passes over the operand and one
    # more rounding)
    lhs, rhs, out, squeeze = _before_sddmm(num_edges, op, lhs_data, rhs_data)
    g._graph._CAPI_SDDMM(op, lhs, rhs, out, TARGET[lhs_target], TARGET[rhs_target],
                         on_format)
    return _after_sddmm(out, squeeze)


def copy_u(g, x):
    return gsddmm(g, "copy_lhs", x, None)


def copy_v(g, x):
    return gsddmm(g, "copy_rhs", None, x)


def _register():
    mod = sys.modules[__name__]
    for lhs, rhs in product("uve", "uve"):
        if lhs == rhs:
            continue
        for op in ("add", "sub", "mul", "div", "dot"):
            def func(g, x, y, on_format=_COO, _op=op, _l=lhs, _r=rhs):
                return gsddmm(g, _op, x, y, lhs_target=_l, rhs_target=_r, on_format=on_format)
            func.__name__ = f"{lhs}_{op}_{rhs}"
            func.__doc__ = f"Edge feature = {lhs} features {op} {rhs} features."
            setattr(mod, func.__name__, func)
            __all__.append(func.__name__)


_register()
