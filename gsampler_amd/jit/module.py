"""gs.jit.compile: trace a sampler once, rewrite it, run the rewritten graph.

`compile(func, args)` classifies the example arguments (Matrix / BatchMatrix ->
rebuilt inside the trace from their operator object; lists, ints, floats and
bools -> compile-time constants; everything else -> run-time input), traces
`func` with torch.fx, applies the passes of `passes.py` and keeps the resulting
GraphModule in `.gm`.  Calling the object runs that module.  Same interface as
the reference's python/gs/jit/module.py:191-259."""
from typing import Any, List, Sequence, Tuple

import torch
from torch.fx import PH
from torch.utils import _pytree as pytree

from ..matrix_api import BatchMatrix, Matrix
from . import passes
from .trace import gs_symbolic_trace

MATRIX, BATCH_MATRIX, STATIC, DYNAMIC = "matrix", "batch_matrix", "static", "dynamic"


def classify(args: Sequence[Any]) -> List[str]:
    kinds = []
    for a in args:
        if isinstance(a, BatchMatrix):
            kinds.append(BATCH_MATRIX)
        elif isinstance(a, Matrix):
            kinds.append(MATRIX)
        elif isinstance(a, (list, bool, int, float)):
            kinds.append(STATIC)
        else:
            kinds.append(DYNAMIC)
    return kinds


def matrix_parts(args: Sequence[Any], kinds: Sequence[str]) -> Tuple[list, list]:
    """Operator objects and node / edge data of every matrix argument."""
    graphs, data = [], []
    for a, k in zip(args, kinds):
        if k in (MATRIX, BATCH_MATRIX):
            graphs.append(a._graph)
            data.append([a.row_ndata, a.col_ndata, a.edata])
    return graphs, data


class compile:  # noqa: N801 -- the reference's public name
    def __init__(self, func, args, try_compact=None, format_select=True, must_compact=False):
        """try_compact: None (the default) or False keep row ids as they are;
        True runs the reference's search (python/gs/jit/module.py:306-421): both
        variants of the graph are built and timed on `args`, the faster is kept.
        Compaction renumbers rows densely after every slice, so a sampler that
        draws from the rows of a slice draws other (equally valid) samples in
        the compact variant: the search is therefore only run on request, and
        the sampler's random state is put back afterwards.  must_compact forces
        the compact variant.  Super-batches are never compacted."""
        self.func = func
        self.kinds = classify(args)
        self.static_args = [a for a, k in zip(args, self.kinds) if k == STATIC]
        self.encodings = [a.encoding for a, k in zip(args, self.kinds) if k == BATCH_MATRIX]
        self.use_batchmatrix = BATCH_MATRIX in self.kinds
        self._format_select = format_select
        self.compact = bool(must_compact) and not self.use_batchmatrix
        self.try_compact = bool(try_compact)
        self.gm = self._build(args, self.compact)
        self.compact_search_ms = None
        if self.try_compact and not self.compact and not self.use_batchmatrix:
            other = self._build(args, True)
            plain_ms, compact_ms = self._time(self.gm, args), self._time(other, args)
            self.compact_search_ms = (plain_ms, compact_ms)
            if compact_ms < plain_ms:
                self.gm, self.compact = other, True

    def _time(self, gm, args, runs=3):
        """Milliseconds per call of one variant on the example arguments."""
        import time
        seed, next_call = torch.ops.gs_ops._CAPI_GetRandomState()
        graphs, data = matrix_parts(args, self.kinds)
        passthrough = tuple(None if k in (MATRIX, BATCH_MATRIX, STATIC) else a
                            for a, k in zip(args, self.kinds))
        try:
            gm(passthrough, graphs, data)                 # warm-up
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(runs):
                gm(passthrough, graphs, data)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / runs * 1e3
        finally:
            torch.ops.gs_ops._CAPI_SetRandomSeed(int(seed))
            torch.ops.gs_ops._CAPI_SetNextCallId(int(next_call))

    # ------------------------------------------------------------------ build
    def _rebuild_args(self, inner_args, graphs, data, compact):
        out, gi, si, bi = [], 0, 0, 0
        for index, kind in enumerate(self.kinds):
            if kind == MATRIX:
                out.append(Matrix(graphs[gi], data[gi][0], data[gi][1], data[gi][2], compact))
                gi += 1
            elif kind == BATCH_MATRIX:
                out.append(BatchMatrix(graphs[gi], data[gi][0], data[gi][1], data[gi][2],
                                       self.encodings[bi]))
                gi, bi = gi + 1, bi + 1
            elif kind == STATIC:
                out.append(self.static_args[si])
                si += 1
            else:
                out.append(inner_args[index])
        return tuple(out)

    def _build(self, args, compact):
        def inner_wrapper(inner_args, inner_graph_args, inner_graph_data_args):
            return self.func(*self._rebuild_args(inner_args, inner_graph_args,
                                                 inner_graph_data_args, compact))

        _, data = matrix_parts(args, self.kinds)
        # node / edge data stay run-time inputs: one placeholder per tensor
        data_spec = pytree.tree_map(lambda _: PH, data)
        gm = gs_symbolic_trace(inner_wrapper,
                               concrete_args={"inner_graph_data_args": data_spec})
        return self._optimize(gm)

    def _optimize(self, gm):
        gm = passes.cse(gm)
        gm = passes.dce(gm)
        gm = passes.move_constant_to_top(gm)
        gm = passes.merge_relabel_and_all_nodes(gm)
        gm = passes.fuse_slicing_and_sampling(gm)
        gm = passes.fuse_slicing_and_weighted_sampling(gm)
        gm = passes.fuse_square_and_sum(gm)
        gm = passes.fuse_div_and_sum(gm)
        gm = passes.read_column_slice_in_place(gm)
        gm = passes.merge_u_mul_v(gm)
        gm = passes.batch_fuse_slicing_and_sampling(gm)
        gm = passes.batch_fuse_slicing_and_weighted_sampling(gm)
        gm = passes.dce(gm)
        if self._format_select and not self.use_batchmatrix:
            gm = passes.select_formats(gm)
        gm = passes.sink_block_construction(gm)
        return gm

    # -------------------------------------------------------------------- run
    def __call__(self, *args):
        graphs, data = matrix_parts(args, self.kinds)
        # matrix arguments are rebuilt inside the graph; their slots only keep
        # the positions of the other run-time inputs
        passthrough = tuple(None if k in (MATRIX, BATCH_MATRIX, STATIC) else a
                            for a, k in zip(args, self.kinds))
        return self.gm(passthrough, graphs, data)
