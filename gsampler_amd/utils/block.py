"""Message-flow-graph hand-off.

The reference builds a DGLBlock from the relabelled COO
(python/gs/utils/to_dgl_block.py:19-23).  DGL is optional here: `Block` keeps
exactly the tensors that go into `create_unitgraph_from_coo` (row -> col edges,
num_src, num_dst) plus the `_ID` bookkeeping, and converts to a real DGLBlock
on request when dgl is importable.
"""
from __future__ import annotations

from collections.abc import Sequence
from typing import Dict, List, Optional

import torch


class Block:
    # A super-batched sampler hands out hundreds of these per step: fixed slots
    # and a plain constructor keep that short.
    __slots__ = ("row", "col", "num_src", "num_dst", "srcdata", "dstdata", "edata", "indptr")

    def __init__(self, row: torch.Tensor, col: torch.Tensor, num_src: int, num_dst: int,
                 indptr: Optional[torch.Tensor] = None):
        self.row = row
        self.col = col
        self.num_src = num_src if type(num_src) is int else int(num_src)
        self.num_dst = num_dst if type(num_dst) is int else int(num_dst)
        self.srcdata: Dict[str, torch.Tensor] = {}
        self.dstdata: Dict[str, torch.Tensor] = {}
        self.edata: Dict[str, torch.Tensor] = {}
        # offsets by destination node when the edges are grouped by destination
        # (every sampled block is): the block's CSC is then (indptr, row)
        self.indptr = indptr

    def csc(self):
        """(indptr[num_dst + 1], indices = source id per edge, edge ids or None),
        the compressed form by destination, without a conversion when the
        producer emitted the offsets."""
        if self.indptr is None:
            from .. import capi
            order = torch.argsort(self.col, stable=True)
            counts = torch.bincount(self.col, minlength=self.num_dst)
            indptr = torch.zeros(self.num_dst + 1, dtype=torch.int64, device=self.col.device)
            torch.cumsum(counts, 0, out=indptr[1:])
            eids = self.edata.get("_ID")
            return indptr, self.row[order], (eids[order] if eids is not None else order)
        return self.indptr, self.row, self.edata.get("_ID")

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
        if self.indptr is not None:
            # python/gs/utils/to_dgl_block.py:5-16: the unit graph straight from the CSC.
            # The edge-id argument maps compressed positions to the block's own
            # edge numbers (a permutation of 0..E-1); an empty tensor numbers the
            # edges in compressed order, which is the order of row / col / edata.
            # edata["_ID"] holds positions in the parent matrix and stays edge data.
            idx = dgl.heterograph_index.create_unitgraph_from_csr(
                2, self.num_src, self.num_dst, self.indptr, self.row,
                torch.empty(0, dtype=torch.int64, device=self.row.device),
                ["coo", "csr", "csc"], transpose=True)
        else:
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


class BlockList(Sequence):
    """The blocks of one layer of a super-batched sampler, one per mini-batch.

    A list as far as callers are concerned (len, indexing, iteration), backed by
    the layer's concatenated arrays: `batch` is the operator library's BlockBatch,
    whose single call relabelled the whole super-batch and laid out every block's
    edge list, compressed form and source ids as views.  A Block object is made
    when it is asked for; `materialize()` makes all of them from one call."""

    def __init__(self, batch, edata: Optional[Dict[str, torch.Tensor]] = None):
        self._batch = batch
        self._edata = dict(edata) if edata else {}
        self._blocks: Optional[List[Optional[Block]]] = None
        self._edge_offsets = None

    def __len__(self) -> int:
        return self._batch.size()

    @property
    def batch(self):
        return self._batch

    def totals(self):
        """(source nodes, destination nodes, edges) summed over the blocks,
        from tensor sizes alone."""
        return tuple(self._batch.totals())

    def _wrap(self, index: int, views) -> Block:
        row, col, indptr, frontier, eids, num_src, num_dst = views
        block = Block(row, col, num_src, num_dst, indptr)
        block.srcdata["_ID"] = frontier
        if eids is not None:
            block.edata["_ID"] = eids
        if self._edata:
            if self._edge_offsets is None:
                self._edge_offsets = self._batch.offsets()[2]
            lo, hi = self._edge_offsets[index], self._edge_offsets[index + 1]
            for key, value in self._edata.items():
                block.edata[key] = value[lo:hi]
        return block

    def materialize(self) -> List[Block]:
        """Every block of the layer, from one call that cuts the layer's arrays into
        per-batch views.  The objects are filled slot by slot (no constructor call,
        no per-block conversions): a step hands out a few hundred of them."""
        if self._blocks is not None and all(b is not None for b in self._blocks):
            return self._blocks
        rows, cols, indptrs, fronts, eids, num_src, num_dst = self._batch.blocks()
        have = self._blocks or [None] * len(rows)
        edata = self._edata
        if edata and self._edge_offsets is None:
            self._edge_offsets = self._batch.offsets()[2]
        off = self._edge_offsets
        new = Block.__new__
        blocks = []
        for i in range(len(rows)):
            b = have[i]
            if b is None:
                b = new(Block)
                b.row, b.col, b.indptr = rows[i], cols[i], indptrs[i]
                b.num_src, b.num_dst = num_src[i], num_dst[i]
                b.srcdata = {"_ID": fronts[i]}
                b.dstdata = {}
                e = eids[i]
                b.edata = {} if e is None else {"_ID": e}
                if edata:
                    lo, hi = off[i], off[i + 1]
                    for key, value in edata.items():
                        b.edata[key] = value[lo:hi]
            blocks.append(b)
        self._blocks = blocks
        return blocks

    def __getitem__(self, index):
        if isinstance(index, slice):
            return self.materialize()[index]
        n = len(self)
        if index < 0:
            index += n
        if not 0 <= index < n:
            raise IndexError("block index out of range")
        if self._blocks is None:
            self._blocks = [None] * n
        if self._blocks[index] is None:
            self._blocks[index] = self._wrap(index, self._batch.block(index))
        return self._blocks[index]

    def __iter__(self):
        return iter(self.materialize())

    def __repr__(self) -> str:
        src, dst, edges = self.totals()
        return (f"BlockList({len(self)} blocks, num_src_nodes={src}, num_dst_nodes={dst}, "
                f"num_edges={edges})")
