"""Rewrite passes over the traced operator graph.

Structural clean-up: common-subexpression elimination, dead-code elimination,
hoisting of tensor constants.  Operator rewrites (observable in
`compiled.gm.graph`, same set as the reference's python/gs/jit/optimize.py):

  merge_relabel_and_all_nodes   _CAPI_GetValidNodes + _CAPI_GraphRelabel on one
                                matrix            -> one _CAPI_GraphRelabel;
                                _CAPI_BatchGetValidNodes + _CAPI_BatchBlocks
                                                  -> the block batch's frontier
  fuse_slicing_and_sampling     _CAPI_Slicing -> _CAPI_Sampling on one axis
                                                  -> _CAPI_SlicingSampling
  batch_fuse_slicing_and_sampling  _CAPI_BatchColSlicing(encoding=False) ->
                                _CAPI_BatchRowSampling
                                                  -> _CAPI_BatchFusedSlicingSampling
  fuse_square_and_sum           (e ** 2) summed by a copy_rhs / sum SpMM
                                                  -> _CAPI_FusedESquareSum
  fuse_div_and_sum              e / u[endpoint] summed onto the other endpoint,
                                quotient not used otherwise
                                                  -> _CAPI_FusedEDivUSum
  merge_u_mul_v                 two u-op-v SDDMMs on one matrix
                                                  -> _CAPI_FusedUOPV
  read_column_slice_in_place    a column slice that is only summed (squares
                                onto rows) and row-sliced is never written:
                                                  -> _CAPI_SlicedESquareSum,
                                                     _CAPI_ColRowSlicing on the
                                                     parent matrix
  select_formats                deterministic on_format / output_format choice
"""
import operator
from typing import Dict, Iterable, List, Optional

import torch.fx as fx

from ..format import _COO, _CSC, _CSR

# Operators that write into a caller-allocated tensor: they have no users in the
# graph but must survive dead-code elimination.
IN_PLACE_OPS = ("_CAPI_SDDMM", "_CAPI_SpMM", "_CAPI_FusedUOPV", "_CAPI_FusedESquareSum",
                "_CAPI_FusedEDivUSum", "_CAPI_SlicedESquareSum")


def _input_nodes(node: fx.Node) -> Iterable[fx.Node]:
    return node.all_input_nodes


def _finish(gm: fx.GraphModule) -> fx.GraphModule:
    gm.graph.lint()
    gm.recompile()
    return gm


def dce(gm: fx.GraphModule) -> fx.GraphModule:
    live = set()
    for node in reversed(gm.graph.nodes):
        if node.op in ("output", "placeholder") or node.target in IN_PLACE_OPS:
            live.add(node)
        if node in live:
            live.update(_input_nodes(node))
    for node in reversed(gm.graph.nodes):
        if node not in live:
            gm.graph.erase_node(node)
    return _finish(gm)


def _draws_random_numbers(node: fx.Node) -> bool:
    """Sampling and walk operators, whether methods of the graph class
    (call_method, target is the name) or free operators of gs_ops
    (call_function, target is the operator object)."""
    name = node.target if isinstance(node.target, str) else str(node.target)
    return any(word in name for word in ("Sampling", "RandomWalk", "Node2Vec"))


def cse(gm: fx.GraphModule) -> fx.GraphModule:
    """Merges nodes with identical target and arguments.  Sampling operators are
    left alone: two textually identical sampling calls draw different samples."""
    seen: Dict[str, fx.Node] = {}
    for node in list(gm.graph.nodes):
        if node.op in ("placeholder", "output"):
            continue
        if _draws_random_numbers(node):
            continue
        if node.target in IN_PLACE_OPS:
            continue
        key = f"{node.op}|{node.target}|{node.args}|{node.kwargs}"
        if key in seen:
            node.replace_all_uses_with(seen[key])
            gm.graph.erase_node(node)
        else:
            seen[key] = node
    return _finish(gm)


def move_constant_to_top(gm: fx.GraphModule) -> fx.GraphModule:
    first = next(iter(gm.graph.nodes))
    constants = [n for n in gm.graph.nodes if n.op == "get_attr" and "constant" in n.name]
    with gm.graph.inserting_before(first):
        for node in constants:
            if node is first:
                continue
            node.replace_all_uses_with(gm.graph.node_copy(node))
            gm.graph.erase_node(node)
    return _finish(gm)


def _is_method(node: fx.Node, name: str) -> bool:
    return node.op == "call_method" and node.target == name


def _getitem_users(node: fx.Node, index: int) -> List[fx.Node]:
    return [u for u in node.users
            if u.op == "call_function" and u.target is operator.getitem and u.args[1] == index]


def merge_relabel_and_all_nodes(gm: fx.GraphModule) -> fx.GraphModule:
    """all_nodes() and to_dgl_block() of one matrix share a single relabel."""
    gm = cse(gm)
    by_graph: Dict[fx.Node, List[fx.Node]] = {}
    for node in gm.graph.nodes:
        if _is_method(node, "_CAPI_GetValidNodes") or _is_method(node, "_CAPI_GraphRelabel"):
            by_graph.setdefault(node.args[0], []).append(node)
    for group in by_graph.values():
        relabels = [n for n in group if n.target == "_CAPI_GraphRelabel"]
        valid = [n for n in group if n.target == "_CAPI_GetValidNodes"]
        if not relabels or not valid:
            continue
        keep = relabels[0]
        first = min(group, key=lambda n: list(gm.graph.nodes).index(n))
        if first is not keep:
            first.prepend(keep)  # the relabel must precede every former user
        with gm.graph.inserting_after(keep):
            frontier = gm.graph.call_function(operator.getitem, args=(keep, 0))
        for v in valid:
            if v.args[1:] == keep.args[1:]:
                v.replace_all_uses_with(frontier)
    return dce(_merge_batch_blocks_and_all_nodes(gm))


def _merge_batch_blocks_and_all_nodes(gm: fx.GraphModule) -> fx.GraphModule:
    """The super-batched twin: all_nodes() reads the frontier and its batch
    pointer off the layer's block batch, which is built first.  The relabel is
    then queued before the host waits for the size of the frontier, so the
    device has work while that number travels."""
    by_graph: Dict[fx.Node, List[fx.Node]] = {}
    for node in gm.graph.nodes:
        if _is_method(node, "_CAPI_BatchGetValidNodes") or _is_method(node, "_CAPI_BatchBlocks"):
            by_graph.setdefault(node.args[0], []).append(node)
    for group in by_graph.values():
        # (numbered anew for every group: the rewrite of an earlier layer added nodes)
        order = {n: i for i, n in enumerate(gm.graph.nodes)}
        builders = [n for n in group if n.target == "_CAPI_BatchBlocks"]
        valid = [n for n in group if n.target == "_CAPI_BatchGetValidNodes"]
        if not builders or not valid:
            continue
        keep = builders[0]
        # only all_nodes() calls with the builder's own id tensors read its frontier
        matching = [v for v in valid if v.args[1:] == keep.args[1:]]
        if not matching:
            continue
        first = min(matching + [keep], key=lambda n: order[n])
        if first is not keep:
            # the builder moves in front of its first reader, but never in front of
            # one of its own arguments
            if any(order[a] > order[first] for a in keep.all_input_nodes):
                continue
            first.prepend(keep)
        with gm.graph.inserting_after(keep):
            ptr = gm.graph.call_method("frontier_ptr", args=(keep,))
            frontier = gm.graph.call_method("frontier", args=(keep,))
        for v in matching:
            for user in list(v.users):
                if (user.op == "call_function" and user.target is operator.getitem
                        and user.args[1] in (0, 1)):
                    user.replace_all_uses_with(frontier if user.args[1] == 0 else ptr)
    gm.graph.lint()
    return gm


def fuse_slicing_and_sampling(gm: fx.GraphModule) -> fx.GraphModule:
    """Slicing(seeds, axis, on, out) -> [0] -> Sampling(axis, K, replace, on, out)
       => SlicingSampling(axis, seeds, K, replace, on, out).

    Edge data gathered through the slice index and then through the sampling
    index is re-gathered from the parent with the fused index, which addresses
    the parent's edges directly."""
    for sampling in list(gm.graph.nodes):
        if not _is_method(sampling, "_CAPI_Sampling"):
            continue
        sliced_graph = sampling.args[0]
        if not (sliced_graph.op == "call_function" and sliced_graph.target is operator.getitem
                and sliced_graph.args[1] == 0):
            continue
        slicing = sliced_graph.args[0]
        if not _is_method(slicing, "_CAPI_Slicing"):
            continue
        if sampling.args[1] != slicing.args[2]:      # same axis
            continue
        if len(sliced_graph.users) > 1:              # the slice itself is used
            continue
        slice_index = _getitem_users(slicing, 1)
        sample_index = _getitem_users(sampling, 1)
        # every tensor gathered with the slice index may only feed a gather with
        # the sampling index
        rewires = []
        ok = True
        for idx_node in slice_index:
            for gathered in idx_node.users:
                users = list(gathered.users)
                if len(users) != 1 or not sample_index or sample_index[0] not in users[0].args:
                    ok = False
                rewires.append((gathered, users[0] if users else None))
        if not ok:
            continue
        with gm.graph.inserting_before(slicing):
            fused = gm.graph.call_method(
                "_CAPI_SlicingSampling",
                args=(slicing.args[0], slicing.args[2], slicing.args[1], sampling.args[2],
                      sampling.args[3], sampling.args[4], sampling.args[5]))
            fused_graph = gm.graph.call_function(operator.getitem, args=(fused, 0))
            fused_index = gm.graph.call_function(operator.getitem, args=(fused, 1))
        for g in _getitem_users(sampling, 0):
            g.replace_all_uses_with(fused_graph)
        for gathered, second in rewires:
            with gm.graph.inserting_before(second):
                direct = gm.graph.call_function(operator.getitem,
                                                args=(gathered.args[0], fused_index))
            second.replace_all_uses_with(direct)
    return dce(gm)


def _fuse_weighted(gm: fx.GraphModule, slice_name: str, sample_name: str,
                   probs_arg: int, compatible, make_fused) -> fx.GraphModule:
    """Shared by the two passes below.  The weights of the sampling call must be
    a gather of some edge tensor through the slice index; the fused operator
    takes that edge tensor itself (the parent's weights), and every edge tensor
    that went through the slice index and then through the sampling index is
    re-gathered from the parent with the fused index."""
    for sampling in list(gm.graph.nodes):
        if not _is_method(sampling, sample_name):
            continue
        sliced_graph = sampling.args[0]
        if not (sliced_graph.op == "call_function" and sliced_graph.target is operator.getitem
                and sliced_graph.args[1] == 0 and len(sliced_graph.users) == 1):
            continue
        slicing = sliced_graph.args[0]
        if not _is_method(slicing, slice_name) or not compatible(slicing, sampling):
            continue
        slice_index = _getitem_users(slicing, 1)
        sample_index = _getitem_users(sampling, 1)
        probs = sampling.args[probs_arg]
        if not (isinstance(probs, fx.Node) and probs.op == "call_function"
                and len(probs.args) == 2 and probs.args[1] in slice_index):
            continue
        rewires, ok = [], True
        for idx_node in slice_index:
            for gathered in idx_node.users:
                for user in list(gathered.users):
                    if user is sampling:
                        continue
                    if not (sample_index and sample_index[0] in user.args):
                        ok = False
                    rewires.append((gathered, user))
        if not ok:
            continue
        with gm.graph.inserting_before(slicing):
            fused = make_fused(gm.graph, slicing, sampling, probs.args[0])
            fused_graph = gm.graph.call_function(operator.getitem, args=(fused, 0))
            fused_index = gm.graph.call_function(operator.getitem, args=(fused, 1))
        for g in _getitem_users(sampling, 0):
            g.replace_all_uses_with(fused_graph)
        for gathered, second in rewires:
            with gm.graph.inserting_before(second):
                direct = gm.graph.call_function(operator.getitem,
                                                args=(gathered.args[0], fused_index))
            second.replace_all_uses_with(direct)
    return dce(gm)


def fuse_slicing_and_weighted_sampling(gm: fx.GraphModule) -> fx.GraphModule:
    """Slicing(seeds, axis, on, out) -> [0] -> SamplingProbs(axis, w[slice index], K, ...)
       => SlicingSamplingProbs(axis, seeds, w, K, replace, on, out): the slice is
    never materialised and the draws go through the parent's weight CDF."""
    def compatible(slicing, sampling):          # same axis, same format
        return sampling.args[1] == slicing.args[2] and sampling.args[5] == slicing.args[3]

    def make(graph, slicing, sampling, weights):
        return graph.call_method(
            "_CAPI_SlicingSamplingProbs",
            args=(slicing.args[0], slicing.args[2], slicing.args[1], weights, sampling.args[3],
                  sampling.args[4], sampling.args[5], sampling.args[6]))

    return _fuse_weighted(gm, "_CAPI_Slicing", "_CAPI_SamplingProbs", 2, compatible, make)


def batch_fuse_slicing_and_weighted_sampling(gm: fx.GraphModule) -> fx.GraphModule:
    """BatchColSlicing(seeds, ptr, encoding=False) -> [0] -> BatchRowSamplingProbs(K, replace,
    w[slice index]) => BatchFusedSlicingSamplingProbs(seeds, ptr, w, K, replace)."""
    def compatible(slicing, sampling):          # encoded rows cannot be fused
        return slicing.args[3] is False

    def make(graph, slicing, sampling, weights):
        return graph.call_method(
            "_CAPI_BatchFusedSlicingSamplingProbs",
            args=(slicing.args[0], slicing.args[1], slicing.args[2], weights, sampling.args[1],
                  sampling.args[2]))

    return _fuse_weighted(gm, "_CAPI_BatchColSlicing", "_CAPI_BatchRowSamplingProbs", 3,
                          compatible, make)


def batch_fuse_slicing_and_sampling(gm: fx.GraphModule) -> fx.GraphModule:
    """BatchColSlicing(seeds, ptr, encoding=False) -> [0] -> BatchRowSampling(K, replace)
       => BatchFusedSlicingSampling(seeds, ptr, K, replace)."""
    for sampling in list(gm.graph.nodes):
        if not _is_method(sampling, "_CAPI_BatchRowSampling"):
            continue
        sliced_graph = sampling.args[0]
        if not (sliced_graph.op == "call_function" and sliced_graph.target is operator.getitem):
            continue
        slicing = sliced_graph.args[0]
        if not _is_method(slicing, "_CAPI_BatchColSlicing"):
            continue
        if slicing.args[3] is not False or len(sliced_graph.users) > 1:
            continue
        # edge data gathered through the slice index cannot be re-routed here
        if any(list(i.users) for i in _getitem_users(slicing, 1)):
            continue
        with gm.graph.inserting_before(slicing):
            fused = gm.graph.call_method(
                "_CAPI_BatchFusedSlicingSampling",
                args=(slicing.args[0], slicing.args[1], slicing.args[2], sampling.args[1],
                      sampling.args[2]))
        sampling.replace_all_uses_with(fused)
    return dce(gm)


def _is_wrapped(node, name: str) -> bool:
    return (isinstance(node, fx.Node) and node.op == "call_function"
            and getattr(node.target, "__name__", "") == name)


def fuse_square_and_sum(gm: fx.GraphModule) -> fx.GraphModule:
    """SpMM("copy_rhs", "sum", _, e ** 2, ...) => FusedESquareSum(..., e, ...)."""
    for spmm in list(gm.graph.nodes):
        if not _is_method(spmm, "_CAPI_SpMM"):
            continue
        if spmm.args[1] != "copy_rhs" or spmm.args[2] != "sum":
            continue
        efeat = spmm.args[4]
        if not (isinstance(efeat, fx.Node) and efeat.op == "call_function"
                and efeat.target is operator.pow and efeat.args[1] == 2):
            continue
        new_args = list(spmm.args)
        new_args[4] = efeat.args[0]
        with gm.graph.inserting_before(spmm):
            gm.graph.call_method("_CAPI_FusedESquareSum", args=tuple(new_args))
        gm.graph.erase_node(spmm)
        # the step that shapes the accumulator only looks at shape and dtype:
        # give it the plain weights, so that the square is dead and goes away
        for user in list(efeat.users):
            if _is_wrapped(user, "_before_spmm"):
                user.replace_input_with(efeat, efeat.args[0])
    return dce(gm)


def fuse_div_and_sum(gm: fx.GraphModule) -> fx.GraphModule:
    """q = e / u[t] (an SDDMM with targets (e, t) and operator "div", or "mul"
    with 1.0 / u as its operand), then SpMM("copy_rhs", "sum", _, q)
    onto the other endpoint, q read by nothing else
        => FusedEDivUSum("div", "sum", u, e, ...): the quotient is never stored.
    The reference names this pass and leaves it empty
    (python/gs/jit/optimize.py:372-374)."""
    from ..ops.fused_op import _before_e_div_u_sum
    for spmm in list(gm.graph.nodes):
        if not _is_method(spmm, "_CAPI_SpMM"):
            continue
        if spmm.args[1] != "copy_rhs" or spmm.args[2] != "sum":
            continue
        quotient, u_target = spmm.args[4], spmm.args[8]
        v_item = spmm.args[5]
        if not (_is_wrapped(quotient, "_after_sddmm") and isinstance(v_item, fx.Node)
                and v_item.target is operator.getitem
                and _is_wrapped(v_item.args[0], "_before_spmm")):
            continue
        before_spmm = v_item.args[0]
        if set(quotient.users) != {spmm, before_spmm}:
            continue                      # the quotient itself is wanted as well
        out_item = quotient.args[0]
        if not (isinstance(out_item, fx.Node) and out_item.target is operator.getitem
                and _is_wrapped(out_item.args[0], "_before_sddmm")):
            continue
        before_sddmm = out_item.args[0]
        writers = [n for n in out_item.users if _is_method(n, "_CAPI_SDDMM")]
        if len(writers) != 1 or set(out_item.users) != {writers[0], quotient}:
            continue
        sddmm = writers[0]
        if not (sddmm.args[0] is spmm.args[0] and sddmm.args[4] is out_item
                and sddmm.args[5] == 1 and sddmm.args[6] == u_target and u_target in (0, 2)):
            continue
        op, e, rhs = before_sddmm.args[1], before_sddmm.args[2], before_sddmm.args[3]
        if op == "div":
            u = rhs
        elif (op == "mul" and isinstance(rhs, fx.Node) and rhs.op == "call_function"
              and rhs.target is operator.truediv and rhs.args[0] == 1.0):
            u = rhs.args[1]
        else:
            continue
        # the accumulator's users: the SpMM and the step that squeezes the result
        finish = [n for n in v_item.users if _is_wrapped(n, "_after_spmm")]
        if len(finish) != 1 or set(v_item.users) != {spmm, finish[0]}:
            continue
        with gm.graph.inserting_before(spmm):
            parts = gm.graph.call_function(
                _before_e_div_u_sum,
                args=(before_spmm.args[0], before_spmm.args[1], e, u, u_target))
            u2, e2, v, squeeze = (gm.graph.call_function(operator.getitem, args=(parts, i))
                                  for i in range(4))
            gm.graph.call_method("_CAPI_FusedEDivUSum",
                                 args=(spmm.args[0], "div", "sum", u2, e2, v, None, None,
                                       u_target, spmm.args[9]))
        finish[0].args = (v, squeeze)
        gm.graph.erase_node(spmm)
        gm.graph.erase_node(sddmm)
    return dce(gm)


def merge_u_mul_v(gm: fx.GraphModule) -> fx.GraphModule:
    """Two SDDMMs with targets (u, v), the same operator, graph and format
       => one FusedUOPV that sweeps the edges once."""
    groups: Dict[str, List[fx.Node]] = {}
    for node in gm.graph.nodes:
        if _is_method(node, "_CAPI_SDDMM") and node.args[5] == 0 and node.args[6] == 2:
            groups.setdefault(f"{node.args[0]}|{node.args[1]}|{node.args[7]}", []).append(node)
    order = {n: i for i, n in enumerate(gm.graph.nodes)}
    for pair in groups.values():
        if len(pair) != 2:
            continue
        first, second = sorted(pair, key=order.get)
        # The fused operator runs where the second product ran.  Readers of the
        # first output that sit in between (its squeeze step) move behind it;
        # that is only sound when their own users come later still.
        early = [u for u in first.args[4].users
                 if u is not first and order[u] < order[second]]
        if any(order[uu] < order[second] for u in early for uu in u.users):
            continue
        for u in sorted(early, key=order.get, reverse=True):
            second.append(u)
        with gm.graph.inserting_before(second):
            gm.graph.call_method(
                "_CAPI_FusedUOPV",
                args=(first.args[0], first.args[1], first.args[2], first.args[3], first.args[4],
                      second.args[2], second.args[3], second.args[4], second.args[7]))
        gm.graph.erase_node(first)
        gm.graph.erase_node(second)
    return dce(gm)


def read_column_slice_in_place(gm: fx.GraphModule) -> fx.GraphModule:
    """s = A._CAPI_Slicing(cols, axis=1, ...) whose matrix s[0] is only asked for its
    shape, summed by _CAPI_FusedESquareSum(copy_rhs, sum, e = w[s[1]]) onto rows, and
    row-sliced (s[0]._CAPI_Slicing(rows, axis=0, ...)), and whose edge index s[1] only
    gathers edge data that feeds those operators
        => A._CAPI_SlicedESquareSum(cols, w, out)
           A._CAPI_ColRowSlicing(cols, rows, on, out)   (edge index into A's edges)
    The slice -- row id, edge position and column of every edge, and every edge
    tensor gathered through it -- is then dead and is not computed: a layer-wise
    sampler slices a few hundred long columns, sums them onto rows, keeps a quarter
    of the edges and never looks at the rest again (examples/ladies/ladies.py:7-21 of
    the reference, which fuses neither step for a single matrix)."""
    for slicing in list(gm.graph.nodes):
        if not _is_method(slicing, "_CAPI_Slicing") or slicing.args[2] != 1:
            continue
        parent, cols = slicing.args[0], slicing.args[1]
        sliced = _getitem_users(slicing, 0)
        index = _getitem_users(slicing, 1)
        if len(sliced) != 1 or len(index) > 1 or len(slicing.users) != len(sliced) + len(index):
            continue
        g = sliced[0]
        gathered = list(index[0].users) if index else []
        if not all(_is_wrapped(n, "data_index") and n.args[1] is index[0] for n in gathered):
            continue
        sums, row_slices, shapes, ok = [], [], [], True
        for user in g.users:
            if (_is_method(user, "_CAPI_FusedESquareSum") and user.args[0] is g
                    and user.args[1] == "copy_rhs" and user.args[2] == "sum"
                    and user.args[8] == 2 and user.args[4] in gathered):
                sums.append(user)
            elif (_is_method(user, "_CAPI_Slicing") and user.args[0] is g
                  and user.args[2] == 0):
                row_slices.append(user)
            elif (_is_method(user, "_CAPI_GetNumRows") or _is_method(user, "_CAPI_GetNumCols")):
                shapes.append(user)
            else:
                ok = False
        if not ok or not row_slices:
            continue
        # what was gathered through the slice may only be summed, looked at for its
        # shape, or gathered again through the index of one of the row slices
        regather = []
        row_indices = [i for rs in row_slices for i in _getitem_users(rs, 1)]
        for w in gathered:
            for user in w.users:
                if user in sums and user.args[4] is w and list(user.all_input_nodes).count(w) == 1:
                    continue
                if _is_wrapped(user, "_before_spmm"):
                    continue
                if (_is_wrapped(user, "data_index") and user.args[0] is w
                        and user.args[1] in row_indices):
                    regather.append(user)
                    continue
                ok = False
        if not ok:
            continue
        for node in shapes:
            with gm.graph.inserting_before(node):
                if node.target == "_CAPI_GetNumRows":      # a column slice keeps the rows
                    fresh = gm.graph.call_method("_CAPI_GetNumRows", args=(parent,))
                else:
                    fresh = gm.graph.call_method("numel", args=(cols,))
            node.replace_all_uses_with(fresh)
        for node in sums:
            w = node.args[4]
            with gm.graph.inserting_before(node):
                gm.graph.call_method("_CAPI_SlicedESquareSum",
                                     args=(parent, cols, w.args[0], node.args[5]))
            gm.graph.erase_node(node)
        for w in gathered:
            for user in list(w.users):
                if _is_wrapped(user, "_before_spmm"):      # reads shape and dtype only
                    user.replace_input_with(w, w.args[0])
        for rs in row_slices:
            with gm.graph.inserting_before(rs):
                fused = gm.graph.call_method(
                    "_CAPI_ColRowSlicing", args=(parent, cols, rs.args[1], _CSC, rs.args[4]))
            rs.replace_all_uses_with(fused)
        for node in regather:                              # the new index addresses the parent
            node.replace_input_with(node.args[0], node.args[0].args[0])
    return dce(gm)


def sink_block_construction(gm: fx.GraphModule) -> fx.GraphModule:
    """Splitting results per batch and building blocks is host work (and, for the
    splits, a blocking read of the offsets).  Done where the sampler wrote it,
    it holds back the launches of the next layer; nothing on the device depends
    on it, so it moves to the end of the graph, in its original order."""
    host_functions = {"batch_gen_block", "batch_block_list", "create_block_from_coo", "create_block_from_csc",
                      "assign_block", "_CAPI_BatchSplitByOffset",
                      "_CAPI_BatchIndptrSplitByOffset"}

    def is_host_work(n: fx.Node) -> bool:
        if n.op == "call_method":
            return n.target == "_CAPI_BatchGetColCounts"
        if n.op != "call_function":
            return False
        name = getattr(n.target, "__name__", None) or str(n.target)
        return name.split(".")[-1] in host_functions

    output = next(n for n in gm.graph.nodes if n.op == "output")
    moving = set()
    for n in gm.graph.nodes:            # topological order: users come later
        if n.op == "output":
            continue
        if is_host_work(n) or any(a in moving for a in n.all_input_nodes):
            moving.add(n)
    for n in [n for n in gm.graph.nodes if n in moving]:
        output.prepend(n)
    return _finish(gm)


# --------------------------------------------------------------- formats
# operator -> (position of on_format, position of output_format or None); positions
# count the operator object itself as argument 0 (python/gs/jit/module.py:21-31).
FORMAT_ARGS = {
    "_CAPI_Slicing": (3, 4),
    "_CAPI_Sampling": (4, 5),
    "_CAPI_SamplingProbs": (5, 6),
    "_CAPI_SlicingSampling": (5, 6),
    "_CAPI_SlicingSamplingProbs": (6, 7),
    "_CAPI_SDDMM": (7, None),
    "_CAPI_SpMM": (9, None),
    "_CAPI_FusedUOPV": (8, None),
    "_CAPI_FusedESquareSum": (9, None),
    "_CAPI_FusedEDivUSum": (9, None),
    "_CAPI_ColRowSlicing": (3, 4),
}


def _preferred(node: fx.Node) -> List[int]:
    """Formats an operator can run on, best first.  Slicing prefers the format
    whose compressed axis is the sliced one (a gather), then the other
    compressed format (a filter pass, no sort), then COO."""
    t = node.target
    if t == "_CAPI_Slicing":
        return [_CSR, _CSC, _COO] if node.args[2] == 0 else [_CSC, _CSR, _COO]
    if t in ("_CAPI_Sampling", "_CAPI_SlicingSampling"):
        return [_CSR] if node.args[1] == 0 else [_CSC]
    if t in ("_CAPI_SamplingProbs", "_CAPI_SlicingSamplingProbs"):
        return [_CSR] if node.args[1] == 0 else [_CSC]
    if t in ("_CAPI_SpMM", "_CAPI_FusedESquareSum", "_CAPI_FusedEDivUSum"):
        return [_CSR, _COO] if node.args[8] == 2 else [_CSC, _COO]
    if t == "_CAPI_SDDMM":
        return [_COO, _CSC, _CSR]
    if t == "_CAPI_ColRowSlicing":
        return [_CSC]
    return [_COO, _CSC]


def select_formats(gm: fx.GraphModule, input_formats: int = _CSC) -> fx.GraphModule:
    """Deterministic format assignment: every operator runs on the best format
    its input already holds (no conversion), and producers materialise that
    format plus COO.  Input matrices hold `input_formats`; derived matrices hold
    what their producer was told to emit.  (The reference times every plan on
    the device and keeps the fastest, python/gs/jit/module.py:306-421.)"""
    holds: Dict[fx.Node, int] = {}

    def formats_of(graph_node: fx.Node) -> int:
        if graph_node in holds:
            return holds[graph_node]
        if (graph_node.op == "call_function" and graph_node.target is operator.getitem
                and graph_node.args[0] in holds):
            return holds[graph_node.args[0]]
        return input_formats

    for node in gm.graph.nodes:
        if node.op != "call_method" or node.target not in FORMAT_ARGS:
            continue
        on_pos, out_pos = FORMAT_ARGS[node.target]
        available = formats_of(node.args[0])
        choice: Optional[int] = next((f for f in _preferred(node) if f & available), None)
        if choice is None:                      # a conversion is unavoidable
            choice = _preferred(node)[0]
        node.update_arg(on_pos, choice)
        if out_pos is not None:
            out = choice | _COO if choice != _COO else _COO
            node.update_arg(out_pos, out)
            holds[node] = out
    return _finish(gm)
