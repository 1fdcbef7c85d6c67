"""Operand preparation shared by the SDDMM / SpMM wrappers: broadcasting
rules, scalar-feature unsqueezing.  Same observable behaviour as the reference's
python/gs/ops/sddmm.py:16-100 and spmm.py:13-107."""
from typing import Optional, Tuple

import torch

TARGET = {"u": 0, "e": 1, "v": 2, "src": 0, "edge": 1, "dst": 2}


def infer_broadcast_shape(op: str, shp1: Tuple[int, ...], shp2: Tuple[int, ...]):
    if op == "dot" and shp1[-1] != shp2[-1]:
        raise ValueError(f"dot needs equal last dimensions, got {shp1} and {shp2}")
    n = max(len(shp1), len(shp2))
    p1 = (1,) * (n - len(shp1)) + tuple(shp1)
    p2 = (1,) * (n - len(shp2)) + tuple(shp2)
    for d1, d2 in zip(p1, p2):
        if d1 != d2 and d1 != 1 and d2 != 1:
            raise ValueError(f"feature shapes {shp1} and {shp2} do not broadcast")
    out = tuple(max(d1, d2) for d1, d2 in zip(p1, p2))
    return out[:-1] + (1,) if op == "dot" else out


def pad_feature_dims(lhs: torch.Tensor, rhs: torch.Tensor):
    """Give both operands the same number of feature dims (leading 1s)."""
    if lhs.dim() != rhs.dim():
        n = max(lhs.dim(), rhs.dim())
        lhs = lhs.view((lhs.shape[0],) + (1,) * (n - lhs.dim()) + tuple(lhs.shape[1:]))
        rhs = rhs.view((rhs.shape[0],) + (1,) * (n - rhs.dim()) + tuple(rhs.shape[1:]))
    return lhs, rhs


def prepare_binary(op: str, lhs: Optional[torch.Tensor], rhs: Optional[torch.Tensor]):
    """-> (lhs, rhs, feature_shape, squeeze, dtype, device)."""
    if op not in ("copy_lhs", "copy_rhs"):
        lhs, rhs = pad_feature_dims(lhs, rhs)
    use_l, use_r = op != "copy_rhs", op != "copy_lhs"
    if use_l and use_r:
        if lhs.device != rhs.device:
            raise ValueError(f"operand devices differ: {lhs.device} and {rhs.device}")
        if lhs.dtype != rhs.dtype:
            raise ValueError(f"operand dtypes differ: {lhs.dtype} and {rhs.dtype}")
    exp_l = exp_r = False
    if use_l and lhs.dim() == 1:
        lhs, exp_l = lhs.unsqueeze(-1), True
    if use_r and rhs.dim() == 1:
        rhs, exp_r = rhs.unsqueeze(-1), True
    ref = lhs if use_l else rhs
    feat = infer_broadcast_shape(op, tuple(lhs.shape[1:]) if use_l else (0,),
                                 tuple(rhs.shape[1:]) if use_r else (0,)) \
        if (use_l and use_r) else tuple(ref.shape[1:])
    squeeze = (exp_l or not use_l) and (exp_r or not use_r)
    return lhs, rhs, feat, squeeze, ref.dtype, ref.device
