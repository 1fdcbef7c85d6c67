"""BatchMatrix: the super-batched Matrix.  B independent mini-batches are
concatenated and travel through every operator in one launch; index arguments
are `ids::ptr` slices (a Python slice whose start is the id tensor and whose
step is the int64[B + 1] pointer array), as in the reference's
python/gs/matrix_api/batch_matrix.py:39-263."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..format import _COO
from ..ops import gsddmm, gspmm
from ..utils.block import Block, BlockList
from .matrix import Matrix, data_index

torch.fx.wrap("batch_gen_block")
torch.fx.wrap("batch_block_list")
torch.fx.wrap("data_index")


def batch_block_list(batch, edata: Dict[str, torch.Tensor]) -> BlockList:
    """The layer's blocks around the operator library's BlockBatch."""
    return BlockList(batch, edata)


def batch_gen_block(frontier_list, coo_row_list, coo_col_list, coo_eids, coo_ptr,
                    edata: Dict[str, torch.Tensor], col_counts) -> List[Block]:
    """One Block per mini-batch from the split relabelled COO."""
    split = torch.ops.gs_ops._CAPI_BatchSplitByOffset
    edata_list = {}
    if coo_eids is not None:
        edata_list["_ID"] = split(coo_eids, coo_ptr)
    for key, value in edata.items():
        edata_list[key] = split(value, coo_ptr)
    blocks = []
    for frontier, row, col, num_dst in zip(frontier_list, coo_row_list, coo_col_list, col_counts):
        block = Block(row, col, frontier.shape[0], num_dst)
        block.srcdata["_ID"] = frontier
        blocks.append(block)
    for key, parts in edata_list.items():
        for block, part in zip(blocks, parts):
            block.edata[key] = part
    return blocks


class BatchMatrix(Matrix):
    def __init__(self, graph=None, row_ndata=None, col_ndata=None, edata=None,
                 encoding: bool = True):
        super().__init__(graph, row_ndata, col_ndata, edata, False)
        self.encoding = encoding

    def load_from_matrix(self, matrix: Matrix, encoding: bool = True) -> "BatchMatrix":
        self.__init__(matrix._graph, matrix.row_ndata, matrix.col_ndata, matrix.edata)
        self.encoding = encoding
        return self

    # ------------------------------------------------------------- extract
    def __getitem__(self, data) -> "BatchMatrix":
        assert len(data) == 2
        r, c = data
        assert isinstance(r, slice) and isinstance(c, slice)
        rows, rows_ptr = r.start, r.step
        cols, cols_ptr = c.start, c.step
        has_r = rows is not None and rows_ptr is not None
        has_c = cols is not None and cols_ptr is not None
        out = BatchMatrix(encoding=self.encoding)

        if has_r and has_c:
            if "_ID" in self.row_ndata or "_ID" in self.col_ndata:
                raise NotImplementedError("row+column slicing of an already sliced BatchMatrix")
            graph, edge_index = self._graph._CAPI_BatchColRowSlcing(cols, cols_ptr, rows, rows_ptr)
            out.row_ndata["_ID"] = rows
            out.col_ndata["_ID"] = cols
            row_pick, col_pick = rows, cols
        elif has_r and not (cols is not None or cols_ptr is not None):
            graph, edge_index = self._graph._CAPI_BatchRowSlicing(rows, rows_ptr)
            if "_ID" not in self.row_ndata:
                out.row_ndata["_ID"] = rows
            row_pick, col_pick = rows, None
        elif has_c and not (rows is not None or rows_ptr is not None):
            if "_ID" in self.col_ndata:
                raise NotImplementedError("column slicing of an already column-sliced BatchMatrix")
            graph, edge_index = self._graph._CAPI_BatchColSlicing(cols, cols_ptr, self.encoding)
            out.col_ndata["_ID"] = cols
            if self.encoding:
                if "_ID" in self.row_ndata:
                    raise NotImplementedError("encoded slicing of an already row-sliced BatchMatrix")
                row_ids, _ = graph._CAPI_BatchGetRows()
                out.row_ndata["_ID"] = row_ids
            # Encoded slicing renumbers the rows (one run of compact ids per
            # batch), so other per-row data follows them.  The reference keeps
            # the old arrays there (python/gs/matrix_api/batch_matrix.py:140-141),
            # which a later row slice then indexes with compact ids.
            row_pick, col_pick = (row_ids if self.encoding else None), cols
        else:
            raise NotImplementedError("BatchMatrix indices must be `ids::ptr` slices")

        out._graph = graph
        for key, value in self.edata.items():
            out.edata[key] = data_index(value, edge_index)
        for key, value in self.row_ndata.items():
            out.row_ndata[key] = value[row_pick] if row_pick is not None else value
        for key, value in self.col_ndata.items():
            out.col_ndata[key] = value[col_pick] if col_pick is not None else value
        return out

    # -------------------------------------------------------------- select
    def individual_sampling(self, K, probs, replace) -> "BatchMatrix":
        out = BatchMatrix(encoding=self.encoding)
        if probs is None:
            subgraph, edge_index = self._graph._CAPI_BatchRowSampling(K, replace)
        else:
            subgraph, edge_index = self._graph._CAPI_BatchRowSamplingProbs(K, replace, probs)
        out._graph = subgraph
        out.row_ndata = self.row_ndata
        out.col_ndata = self.col_ndata
        for key, value in self.edata.items():
            out.edata[key] = value[edge_index]
        return out

    def collective_sampling(self, K, probs, probs_ptr, replace):
        if probs is None:
            selected, index_ptr = torch.ops.gs_ops._CAPI_BatchListSampling(K, replace, probs_ptr)
        else:
            selected, index_ptr = torch.ops.gs_ops._CAPI_BatchListSamplingWithProbs(
                probs, K, replace, probs_ptr)
        return self[selected::index_ptr, :], selected

    # ------------------------------------------------------------- compute
    def sum(self, key, axis) -> torch.Tensor:
        rhs = self.edata[key]
        if axis == 0:
            return gspmm(self, "copy_rhs", "sum", None, rhs, 0, _COO)
        if axis == 1:
            return gspmm(self, "copy_rhs", "sum", None, rhs, 2, _COO)
        raise ValueError("axis should be 0 or 1")

    def div(self, key, divisor, axis) -> "BatchMatrix":
        out = BatchMatrix(self._graph, self.row_ndata, self.col_ndata, dict(self.edata),
                          self.encoding)
        lhs = self.edata[key]
        if axis == 0:
            out.edata[key] = gsddmm(out, "div", lhs, divisor, "e", "v", _COO)
        elif axis == 1:
            out.edata[key] = gsddmm(out, "div", lhs, divisor, "e", "u", _COO)
        else:
            raise ValueError("axis should be 0 or 1")
        return out

    # ------------------------------------------------------------ finalize
    def to_dgl_block(self, prefetch_edata=()) -> BlockList:
        """One block per mini-batch.  The reference relabels, splits three arrays
        per batch and builds the blocks in a Python loop
        (python/gs/matrix_api/batch_matrix.py:232-248, batch_gen_block above);
        here one operator call relabels the super-batch and lays out every
        block's edge list and compressed form, and the returned sequence makes a
        Block object when it is asked for."""
        batch = self._graph._CAPI_BatchBlocks(
            self.col_ndata.get("_ID", self.null_tensor),
            self.row_ndata.get("_ID", self.null_tensor))
        edata = {key: self.edata[key] for key in prefetch_edata}
        return batch_block_list(batch, edata)

    def all_nodes(self):
        return self._graph._CAPI_BatchGetValidNodes(
            self.col_ndata.get("_ID", self.null_tensor),
            self.row_ndata.get("_ID", self.null_tensor))

    def all_rows(self):
        return self._graph._CAPI_BatchGetRows()

    def all_cols(self):
        return self._graph._CAPI_BatchGetCols()

    # ---------------------------------------------------------------- walks
    def random_walk(self, seeds, seeds_ptr, walk_length):
        return torch.ops.gs_ops._CAPI_BatchSplitByOffset(
            self._graph._CAPI_RandomWalk(seeds, walk_length), seeds_ptr)

    def node2vec(self, seeds, seeds_ptr, walk_length, p, q):
        return torch.ops.gs_ops._CAPI_BatchSplitByOffset(
            self._graph._CAPI_Node2Vec(seeds, walk_length, p, q), seeds_ptr)
