"""Message-flow-graph hand-off.

The reference builds a DGLBlock from the relabelled COO
(python/gs/utils/to_dgl_block.py:19-23).  DGL is optional here: `Block` keeps
exactly the tensors that go into `create_unitgraph_from_coo` (row -> col edges,
num_src, num_dst) plus the `_ID` bookkeeping, and converts to a real DGLBlock
on request when dgl is importable.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch


class Block:
    # A super-batched sampler builds hundreds of these per step: fixed slots
    # and a plain constructor keep that loop short.
    __slots__ = ("row", "col", "num_src", "num_dst", "srcdata", "dstdata", "edata")

    def __init__(self, row: torch.Tensor, col: torch.Tensor, num_src: int, num_dst: int):
        self.row = row
        self.col = col
        self.num_src = num_src if type(num_src) is int else int(num_src)
        self.num_dst = num_dst if type(num_dst) is int else int(num_dst)
        self.srcdata: Dict[str, torch.Tensor] = {}
        self.dstdata: Dict[str, torch.Tensor] = {}
        self.edata: Dict[str, torch.Tensor] = {}

    def num_src_nodes(self) -> int:
        return self.num_src

    def num_dst_nodes(self) -> int:
        return self.num_dst

    def num_edges(self) -> int:
        return int(self.row.numel())

    def edges(self):
        return self.row, self.col

    def to_dgl(self):
        import dgl
        from dgl.heterograph import DGLBlock
        idx = dgl.heterograph_index.create_unitgraph_from_coo(
            2, self.num_src, self.num_dst, self.row, self.col, formats=["coo", "csr", "csc"])
        block = DGLBlock(idx, (["_N"], ["_N"]), ["_E"])
        for k, v in self.srcdata.items():
            block.srcdata[k] = v
        for k, v in self.edata.items():
            block.edata[k] = v
        return block

    def __repr__(self) -> str:
        return (f"Block(num_src_nodes={self.num_src}, num_dst_nodes={self.num_dst}, "
                f"num_edges={self.num_edges()})")


def create_block_from_coo(row, col, num_src, num_dst) -> Block:
    return Block(row, col, num_src, num_dst)


def create_block_from_csc(indptr, indices, e_ids, num_src, num_dst) -> Block:
    from .. import capi
    col = capi.csc2coo(indptr, int(indices.numel()))
    block = Block(indices, col, num_src, num_dst)
    if e_ids is not None and e_ids.numel() > 0:
        block.edata["_ID"] = e_ids
    return block
