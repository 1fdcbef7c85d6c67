"""Matrix: the matrix-centric sampling API (extract / select / compute /
finalize steps).  Same surface as the reference's
python/gs/matrix_api/matrix.py:42-303; every method is a thin composition of
`_CAPI_*` operators so that torch.fx can trace a sampler written against it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
from torch.fx import Proxy

from ..format import _COO, _CSC, _CSR
from ..ops import gsddmm, gspmm
from ..utils.block import Block, create_block_from_coo, create_block_from_csc  # noqa: F401
from ..utils.gather import gather_pinned_tensor_rows, gather_rows

torch.fx.wrap("create_block_from_coo")
torch.fx.wrap("create_block_from_csc")
torch.fx.wrap("assign_block")
torch.fx.wrap("gen_arange")
torch.fx.wrap("data_index")


def data_index(data: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """data[index]; pinned host data is gathered in place by the GPU
    (python/gs/matrix_api/matrix.py:19-23 of the reference)."""
    if data.is_pinned():
        return gather_pinned_tensor_rows(data, index)
    if (data.is_cuda and index.is_cuda and index.dtype == torch.int64 and index.dim() == 1
            and data.dim() >= 1 and data.is_contiguous()):
        return gather_rows(data, index)      # edge indices come from the operators: in range
    return data[index]


def gen_arange(size: int, dtype: torch.dtype, device) -> torch.Tensor:
    return torch.arange(size, dtype=dtype, device=device)


def assign_block(block: Block, e_ids, edata: Dict[str, torch.Tensor],
                 unique_tensor: torch.Tensor) -> Block:
    if e_ids is not None:
        block.edata["_ID"] = e_ids
    for key, value in edata.items():
        block.edata[key] = value
    block.srcdata["_ID"] = unique_tensor
    return block


_NULL_TENSOR = None


def _is_index(x) -> bool:
    return isinstance(x, (Proxy, torch.Tensor))


class Matrix:
    def __init__(self, graph=None, row_ndata=None, col_ndata=None, edata=None,
                 compact: bool = False):
        self._graph = graph
        self.row_ndata = {} if row_ndata is None else row_ndata
        self.col_ndata = {} if col_ndata is None else col_ndata
        self.edata = {} if edata is None else edata
        self._compact = compact

    # An empty int64 tensor stands for "no id mapping on this axis".
    @property
    def null_tensor(self) -> torch.Tensor:
        global _NULL_TENSOR
        if _NULL_TENSOR is None:
            _NULL_TENSOR = torch.empty(0, dtype=torch.int64)
        return _NULL_TENSOR

    def load_graph(self, format: str, format_tensors: List[torch.Tensor]) -> "Matrix":
        assert format in ("CSC", "COO", "CSR")
        assert len(format_tensors) == 2
        Graph = torch.classes.gs_classes.Graph
        if format == "COO":
            row, col = format_tensors
            self._graph = Graph(int(row.max()) + 1, int(col.max()) + 1)
            self._graph._CAPI_LoadCOO(row, col, False, False)
        elif format == "CSC":
            indptr, indices = format_tensors
            self._graph = Graph(int(indices.max()) + 1, indptr.numel() - 1)
            self._graph._CAPI_LoadCSC(indptr, indices)
        else:
            indptr, indices = format_tensors
            self._graph = Graph(indptr.numel() - 1, int(indices.max()) + 1)
            self._graph._CAPI_LoadCSR(indptr, indices)
        return self

    # ------------------------------------------------------------- extract
    def __getitem__(self, data) -> "Matrix":
        assert len(data) == 2
        r_slice, c_slice = data
        out = Matrix()
        graph = self._graph
        edge_index = None
        col_index = row_index = None

        if _is_index(c_slice):
            if "_ID" not in self.col_ndata:
                out.col_ndata["_ID"] = c_slice
            graph, edge_index = graph._CAPI_Slicing(c_slice, 1, _CSC, _COO)
            col_index = c_slice

        if _is_index(r_slice):
            if "_ID" not in self.row_ndata:
                out.row_ndata["_ID"] = r_slice
            graph, sub_index = graph._CAPI_Slicing(r_slice, 0, _CSR, _COO)
            edge_index = sub_index if edge_index is None else edge_index[sub_index]
            row_index = r_slice

        out._graph = graph
        if edge_index is not None:
            for key, value in self.edata.items():
                out.edata[key] = data_index(value, edge_index)
        else:
            out.edata = dict(self.edata)
        for key, value in self.col_ndata.items():
            out.col_ndata[key] = value[col_index] if col_index is not None else value
        for key, value in self.row_ndata.items():
            out.row_ndata[key] = value[row_index] if row_index is not None else value

        if self._compact:
            out.compact(0)
            out.compact(1)
        return out

    def compact(self, axis: int) -> "Matrix":
        ndata = self.row_ndata if axis == 0 else self.col_ndata
        if axis not in (0, 1):
            raise ValueError("axis should be 0 or 1")
        if "_ID" not in ndata:
            new_graph, unique_tensor = self._graph._CAPI_Compact(axis)
            for key, value in list(ndata.items()):
                ndata[key] = value[unique_tensor]
            ndata["_ID"] = unique_tensor
            self._graph = new_graph
        return self

    # -------------------------------------------------------------- select
    def individual_sampling(self, K: int, probs: Optional[torch.Tensor],
                            replace: bool) -> "Matrix":
        out = Matrix()
        if probs is None:
            subgraph, edge_index = self._graph._CAPI_Sampling(1, K, replace, _CSC, _COO)
        else:
            subgraph, edge_index = self._graph._CAPI_SamplingProbs(
                1, probs, K, replace, _CSC, _COO)
        out._graph = subgraph
        out.row_ndata = self.row_ndata
        out.col_ndata = self.col_ndata
        for key, value in self.edata.items():
            out.edata[key] = value[edge_index]
        return out

    def collective_sampling(self, K: int, probs: Optional[torch.Tensor], replace: bool):
        if probs is None:
            selected = torch.ops.gs_ops._CAPI_ListSampling(self.num_rows(), K, replace)
        else:
            selected = torch.ops.gs_ops._CAPI_ListSamplingWithProbs(probs, K, replace)
        return self[selected, :], selected

    # ------------------------------------------------------------- compute
    def sum(self, key: str, axis: int, on_format=_CSC) -> torch.Tensor:
        rhs = self.edata[key]
        if axis == 0:
            return gspmm(self, "copy_rhs", "sum", None, rhs, 0, _CSC)
        if axis == 1:
            return gspmm(self, "copy_rhs", "sum", None, rhs, 2, _CSR)
        raise ValueError("axis should be 0 or 1")

    def div(self, key: str, divisor: torch.Tensor, axis: int) -> "Matrix":
        out = Matrix(self._graph, self.row_ndata, self.col_ndata)
        lhs = self.edata[key]
        if axis == 0:
            data = gsddmm(out, "div", lhs, divisor, "e", "v", _COO)
        elif axis == 1:
            data = gsddmm(out, "div", lhs, divisor, "e", "u", _COO)
        else:
            raise ValueError("axis should be 0 or 1")
        out.edata = dict(self.edata)
        out.edata[key] = data
        return out

    # ------------------------------------------------------------ finalize
    def to_dgl_block(self, prefetch_edata=()) -> Block:
        col_seeds = self.col_ndata.get("_ID", self.null_tensor)
        unique_tensor, row, col, e_ids = self._graph._CAPI_GraphRelabel(
            col_seeds, self.row_ndata.get("_ID", self.null_tensor))
        block = create_block_from_coo(row, col, num_src=unique_tensor.numel(),
                                      num_dst=col_seeds.numel())
        edata = {key: self.edata[key] for key in prefetch_edata}
        return assign_block(block, e_ids, edata, unique_tensor)

    def all_nodes(self) -> torch.Tensor:
        return self._graph._CAPI_GetValidNodes(
            self.col_ndata.get("_ID", self.null_tensor),
            self.row_ndata.get("_ID", self.null_tensor))

    # ---------------------------------------------------------- inspection
    def num_rows(self) -> int:
        return self._graph._CAPI_GetNumRows()

    def num_cols(self) -> int:
        return self._graph._CAPI_GetNumCols()

    def num_edges(self) -> int:
        return self._graph._CAPI_GetNumEdges()

    @property
    def csc(self) -> List[torch.Tensor]:
        g = self._graph
        return [g._CAPI_GetCSCIndptr(), g._CAPI_GetCSCIndices(), g._CAPI_GetCSCEids()]

    @property
    def csr(self) -> List[torch.Tensor]:
        g = self._graph
        return [g._CAPI_GetCSRIndptr(), g._CAPI_GetCSRIndices(), g._CAPI_GetCSREids()]

    @property
    def coo(self) -> List[torch.Tensor]:
        g = self._graph
        return [g._CAPI_GetCOORows(), g._CAPI_GetCOOCols(), g._CAPI_GetCOOEids()]

    def rows(self) -> torch.Tensor:
        if "_ID" in self.row_ndata:
            return self.row_ndata["_ID"]
        return gen_arange(self.num_rows(), dtype=torch.int64, device="cuda")

    def cols(self) -> torch.Tensor:
        if "_ID" in self.col_ndata:
            return self.col_ndata["_ID"]
        return gen_arange(self.num_cols(), dtype=torch.int64, device="cuda")

    # ---------------------------------------------------------------- walks
    def random_walk(self, seeds: torch.Tensor, walk_length: int) -> torch.Tensor:
        return self._graph._CAPI_RandomWalk(seeds, walk_length)

    def node2vec(self, seeds: torch.Tensor, walk_length: int, p: float, q: float) -> torch.Tensor:
        return self._graph._CAPI_Node2Vec(seeds, walk_length, p, q)
