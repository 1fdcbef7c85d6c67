"""gs.jit.compile: the rewrites are visible in the traced graph (no GPU needed
to trace), and compiled samplers return what eager execution returns (GPU)."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs


def graphsage_sampler(A, seeds, fanouts):
    input_node = seeds
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        sampleA = subA.individual_sampling(K, None, False)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    output_node = seeds
    return input_node, output_node, ret


def batch_graphsage_sampler(A, seeds, seeds_ptr, fanouts):
    ret = []
    for k in fanouts:
        subA = A[:, seeds::seeds_ptr]
        sampleA = subA.individual_sampling(k, None, False)
        seeds, seeds_ptr = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    return ret


def weighted_graphsage_sampler(A, seeds, fanouts):
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        sampleA = subA.individual_sampling(K, subA.edata["w"], False)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block(prefetch_edata={"w"}))
    return seeds, ret


def batch_weighted_graphsage_sampler(A, seeds, seeds_ptr, fanouts):
    ret = []
    for k in fanouts:
        subA = A[:, seeds::seeds_ptr]
        sampleA = subA.individual_sampling(k, subA.edata["w"], False)
        seeds, seeds_ptr = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    return ret


def ladies_sampler(A, seeds, fanouts):
    # examples/ladies/ladies.py:7-21 of the reference
    input_node = seeds
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        subA.edata["p"] = subA.edata["w"] ** 2
        prob = subA.sum("p", axis=1)
        sampleA, select_index = subA.collective_sampling(K, prob, False)
        sampleA = sampleA.div("w", prob[select_index], axis=1)
        out = sampleA.sum("w", axis=0)
        sampleA = sampleA.div("w", out, axis=0)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block(prefetch_edata={"w"}))
    output_node = seeds
    return input_node, output_node, ret


def pass_like_sampler(A, seeds, u1, v1, u2, v2):
    subA = A[:, seeds]
    a = gs.ops.u_mul_v(subA, u1, v1)
    b = gs.ops.u_mul_v(subA, u2, v2)
    return a + b


def targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_method"]


def test_graphsage_rewrites():
    m = gs.Matrix(gs.Graph(10, 10))
    c = gs.jit.compile(func=graphsage_sampler, args=(m, torch.arange(3), [25, 10]))
    t = targets(c.gm)
    assert t.count("_CAPI_SlicingSampling") == 2          # slice + sample fused
    assert "_CAPI_Slicing" not in t and "_CAPI_Sampling" not in t
    assert t.count("_CAPI_GraphRelabel") == 2 and "_CAPI_GetValidNodes" not in t
    fused = [n for n in c.gm.graph.nodes if n.target == "_CAPI_SlicingSampling"]
    assert [n.args[3] for n in fused] == [25, 10]         # fanouts are constants
    assert all(n.args[1] == 1 and n.args[5] == gs._CSC and n.args[6] == gs._CSC | gs._COO
               for n in fused)


def test_batch_graphsage_rewrites():
    m = gs.Matrix(gs.Graph(10, 10))
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    c = gs.jit.compile(func=batch_graphsage_sampler,
                       args=(bm, torch.arange(4), torch.tensor([0, 2, 4]), [5, 5, 5]),
                       try_compact=False, format_select=False)
    t = targets(c.gm)
    assert t.count("_CAPI_BatchFusedSlicingSampling") == 3
    # every layer's frontier is read off its block batch
    assert t.count("_CAPI_BatchBlocks") == 3 and "_CAPI_BatchGetValidNodes" not in t
    assert "_CAPI_BatchColSlicing" not in t and "_CAPI_BatchRowSampling" not in t
    # encoded batches are not fused (rows are renumbered between the two steps)
    bm2 = gs.BatchMatrix()
    bm2.load_from_matrix(m, True)
    c2 = gs.jit.compile(func=batch_graphsage_sampler,
                        args=(bm2, torch.arange(4), torch.tensor([0, 2, 4]), [5]))
    assert "_CAPI_BatchColSlicing" in targets(c2.gm)


def test_weighted_graphsage_rewrites():
    m = gs.Matrix(gs.Graph(10, 10))
    m.edata["w"] = torch.ones(5)
    c = gs.jit.compile(func=weighted_graphsage_sampler, args=(m, torch.arange(3), [15, 10]))
    t = targets(c.gm)
    # slice + weighted sample fused: the slice is never materialised
    assert t.count("_CAPI_SlicingSamplingProbs") == 2
    assert "_CAPI_Slicing" not in t and "_CAPI_SamplingProbs" not in t
    fused = [n for n in c.gm.graph.nodes if n.target == "_CAPI_SlicingSamplingProbs"]
    assert [n.args[4] for n in fused] == [15, 10]
    assert all(n.args[1] == 1 and n.args[6] == gs._CSC and n.args[7] == gs._CSC | gs._COO
               for n in fused)
    # both layers draw by the weights of the *input* matrix (its placeholder)
    assert fused[0].args[3] is fused[1].args[3] and fused[0].args[3].op == "placeholder"
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    cb = gs.jit.compile(func=batch_weighted_graphsage_sampler,
                        args=(bm, torch.arange(4), torch.tensor([0, 2, 4]), [5, 5]),
                        try_compact=False, format_select=False)
    tb = targets(cb.gm)
    assert tb.count("_CAPI_BatchFusedSlicingSamplingProbs") == 2
    assert "_CAPI_BatchColSlicing" not in tb and "_CAPI_BatchRowSamplingProbs" not in tb


def test_ladies_rewrites():
    m = gs.Matrix(gs.Graph(10, 10))
    m.edata["w"] = torch.rand(7)
    c = gs.jit.compile(func=ladies_sampler, args=(m, torch.arange(3), [4, 4]))
    t = targets(c.gm)
    # the column slice is only summed and row-sliced: it is read in place, never written
    assert t.count("_CAPI_SlicedESquareSum") == 2 and t.count("_CAPI_ColRowSlicing") == 2
    assert "_CAPI_Slicing" not in t and "_CAPI_FusedESquareSum" not in t
    import operator
    assert not any(n.target is operator.pow for n in c.gm.graph.nodes)   # the square itself is gone
    assert t.count("_CAPI_SpMM") == 2                     # the column sums stay
    assert t.count("_CAPI_SDDMM") == 4
    assert "_CAPI_GetValidNodes" not in t
    fused = [n for n in c.gm.graph.nodes if n.target == "_CAPI_ColRowSlicing"]
    for n in fused:
        # on the parent matrix (a run-time input), on its CSC, giving CSC + COO
        assert n.args[0].op == "call_function" and n.args[0].args[0].op == "placeholder"
        assert n.args[3] == gs._CSC and n.args[4] == gs._CSC | gs._COO
    # the weights of the kept edges are gathered from the parent's edge data with the
    # fused operator's index; nothing is gathered through a slice index any more
    gathers = [n for n in c.gm.graph.nodes
               if getattr(n.target, "__name__", "") == "data_index"]
    assert len(gathers) == 2 and all(g.args[0].op == "placeholder" for g in gathers)
    # edge data is a run-time input, not a baked constant
    assert not any(n.op == "get_attr" and "constant" in n.name and n.meta.get("val") is not None
                   for n in c.gm.graph.nodes)
    assert sum(n.op == "placeholder" for n in c.gm.graph.nodes) >= 3


def test_column_slice_stays_when_something_else_reads_it():
    """The rewrite must not fire when the slice, or edge data gathered through it, has a
    reader it cannot serve from the parent matrix."""
    def keeps_the_slice(A, seeds, K):
        subA = A[:, seeds]
        subA.edata["p"] = subA.edata["w"] ** 2
        prob = subA.sum("p", axis=1)
        sampleA, _ = subA.collective_sampling(K, prob, False)
        return sampleA.all_nodes(), subA.edata["w"]          # the slice's weights escape

    def sums_columns_too(A, seeds, K):
        subA = A[:, seeds]
        subA.edata["p"] = subA.edata["w"] ** 2
        prob = subA.sum("p", axis=1)
        extra = subA.sum("w", axis=0)                         # another reader of the slice
        sampleA, _ = subA.collective_sampling(K, prob, False)
        return sampleA.all_nodes(), extra

    for func in (keeps_the_slice, sums_columns_too):
        m = gs.Matrix(gs.Graph(10, 10))
        m.edata["w"] = torch.rand(7)
        c = gs.jit.compile(func=func, args=(m, torch.arange(3), 4))
        t = targets(c.gm)
        assert "_CAPI_ColRowSlicing" not in t and "_CAPI_SlicedESquareSum" not in t
        assert t.count("_CAPI_Slicing") == 2


def fastgcn_like_sampler(A, seeds, fanouts):
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        sampleA, _ = subA.collective_sampling(K, subA.row_ndata["deg"], False)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    return seeds, ret


def walks_twice(A, seeds):
    return A.random_walk(seeds, 3), A.random_walk(seeds, 3)


def test_identical_sampling_calls_are_not_merged():
    """Every layer of FastGCN samples the same list of row weights: the calls
    look alike but each draws its own sample (free operators and walks too)."""
    m = gs.Matrix(gs.Graph(10, 10))
    m.row_ndata["deg"] = torch.rand(10)
    c = gs.jit.compile(func=fastgcn_like_sampler, args=(m, torch.arange(3), [4, 4]))
    names = [str(n.target) for n in c.gm.graph.nodes if n.op == "call_function"]
    assert sum("ListSamplingWithProbs" in n for n in names) == 2
    c = gs.jit.compile(func=walks_twice, args=(m, torch.arange(3)))
    assert targets(c.gm).count("_CAPI_RandomWalk") == 2


def test_two_u_mul_v_are_merged():
    m = gs.Matrix(gs.Graph(10, 10))
    u, v = torch.rand(10), torch.rand(3)
    c = gs.jit.compile(func=pass_like_sampler, args=(m, torch.arange(3), u, v, u + 1, v + 1))
    t = targets(c.gm)
    assert t.count("_CAPI_FusedUOPV") == 1 and "_CAPI_SDDMM" not in t


def div_then_sum_sampler(A, seeds, col_scale):
    sub = A[:, seeds]
    return sub.div("w", col_scale, axis=0).sum("w", axis=1)


def div_then_sum_keeping_the_quotient(A, seeds, col_scale):
    q = A[:, seeds].div("w", col_scale, axis=0)
    return q.sum("w", axis=1), q.edata["w"]


def div_then_sum_on_the_same_axis(A, seeds, col_scale):
    return A[:, seeds].div("w", col_scale, axis=0).sum("w", axis=0)


def test_div_then_sum_is_fused_when_only_the_sum_is_wanted():
    m = gs.Matrix(gs.Graph(10, 10))
    m.edata["w"] = torch.rand(7)
    args = (m, torch.arange(3), torch.rand(3))
    t = targets(gs.jit.compile(func=div_then_sum_sampler, args=args).gm)
    assert t.count("_CAPI_FusedEDivUSum") == 1
    assert "_CAPI_SDDMM" not in t and "_CAPI_SpMM" not in t
    for kept in (div_then_sum_keeping_the_quotient, div_then_sum_on_the_same_axis):
        t = targets(gs.jit.compile(func=kept, args=args).gm)
        assert "_CAPI_FusedEDivUSum" not in t
        assert t.count("_CAPI_SDDMM") == 1 and t.count("_CAPI_SpMM") == 1


# ------------------------------------------------------------------- on the GPU
DEV = "cuda:0"


def _graph():
    from gsampler_amd.utils import rmat_csc
    indptr, indices = rmat_csc(5000, 150000, seed=1)
    m = gs.Matrix()
    m.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    g = torch.Generator().manual_seed(0)
    m.edata["w"] = (torch.rand(indices.numel(), generator=g) + 0.05).to(DEV)
    return m


def _blocks_equal(a, b):
    assert torch.equal(a.row, b.row) and torch.equal(a.col, b.col)
    assert (a.num_src, a.num_dst) == (b.num_src, b.num_dst)
    assert torch.equal(a.srcdata["_ID"], b.srcdata["_ID"])
    assert set(a.edata) == set(b.edata)
    for k in a.edata:
        assert torch.allclose(a.edata[k], b.edata[k], rtol=1e-5)


@pytest.mark.gpu
def test_compiled_graphsage_equals_eager():
    m = _graph()
    seeds = torch.randperm(5000, generator=torch.Generator().manual_seed(1))[:200].to(DEV)
    c = gs.jit.compile(func=graphsage_sampler, args=(m, seeds, [10, 5]))
    gs.manual_seed(3)
    e_in, e_out, e_blocks = graphsage_sampler(m, seeds, [10, 5])
    gs.manual_seed(3)
    c_in, c_out, c_blocks = c(m, seeds, [10, 5])
    assert torch.equal(e_in, c_in) and torch.equal(e_out, c_out)
    for a, b in zip(e_blocks, c_blocks):
        _blocks_equal(a, b)
    # other seeds through the same compiled object
    seeds2 = seeds.flip(0)[:100].contiguous()
    gs.manual_seed(4)
    want = graphsage_sampler(m, seeds2, [10, 5])
    gs.manual_seed(4)
    got = c(m, seeds2, [10, 5])
    assert torch.equal(want[1], got[1])


@pytest.mark.gpu
def test_compiled_batch_graphsage_equals_eager():
    from gsampler_amd.utils import batched_seeds
    m = _graph()
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    seeds, ptr = batched_seeds(5000, 4, 64, seed=2)
    seeds, ptr = seeds.to(DEV), ptr.to(DEV)
    c = gs.jit.compile(func=batch_graphsage_sampler, args=(bm, seeds, ptr, [10, 5]),
                       try_compact=False, format_select=False)
    gs.manual_seed(5)
    eager = batch_graphsage_sampler(bm, seeds, ptr, [10, 5])
    gs.manual_seed(5)
    comp = c(bm, seeds, ptr, [10, 5])
    for le, lc in zip(eager, comp):
        assert len(le) == len(lc) == 4
        for a, b in zip(le, lc):
            _blocks_equal(a, b)


@pytest.mark.gpu
def test_ladies_eager_compiled_and_invariants():
    m = _graph()
    seeds = torch.randperm(5000, generator=torch.Generator().manual_seed(6))[:128].to(DEV)
    c = gs.jit.compile(func=ladies_sampler, args=(m, seeds, [64, 64]))
    gs.manual_seed(7)
    e_in, e_out, e_blocks = ladies_sampler(m, seeds, [64, 64])
    gs.manual_seed(7)
    c_in, c_out, c_blocks = c(m, seeds, [64, 64])
    # The compiled graph slices rows on the CSC (edge order of the column slice)
    # where eager execution sorts into a CSR first, so edges and therefore the
    # first-occurrence frontier come in another order: compare order-free.  (The
    # two cannot be made to agree by running the eager slice on the CSC as well:
    # a slice along the compressed axis repeats a row that is asked for twice,
    # a slice across it cannot, so the format is part of the eager semantics.)
    assert torch.equal(e_out.sort().values, c_out.sort().values)

    def edge_list(blk, dst_ids):
        src = blk.srcdata["_ID"][blk.row].tolist()
        dst = dst_ids[blk.col].tolist()
        w = blk.edata["w"].tolist()
        return sorted(zip(src, dst, w))

    e_dst = c_dst = seeds
    for a, b in zip(e_blocks, c_blocks):
        assert (a.num_src, a.num_dst) == (b.num_src, b.num_dst)
        ea, eb = edge_list(a, e_dst), edge_list(b, c_dst)
        assert [(s, d) for s, d, _ in ea] == [(s, d) for s, d, _ in eb]
        assert np.allclose([w for _, _, w in ea], [w for _, _, w in eb], rtol=1e-5, atol=1e-8)
        e_dst, c_dst = a.srcdata["_ID"], b.srcdata["_ID"]
    blk = e_blocks[0]
    # at most K distinct source rows besides the seeds; weights normalised per column
    assert blk.num_dst == 128 and blk.num_src <= 128 + 64
    w = blk.edata["w"].double()
    col_sum = torch.zeros(blk.num_dst, dtype=torch.float64, device=DEV).index_add_(0, blk.col, w)
    has_edge = torch.zeros(blk.num_dst, dtype=torch.bool, device=DEV)
    has_edge[blk.col] = True
    assert torch.allclose(col_sum[has_edge], torch.ones_like(col_sum[has_edge]), atol=1e-5)
    # every block edge is an edge of the graph
    indptr, indices, _ = m.csc
    src = blk.srcdata["_ID"][blk.row]
    dst = seeds[blk.col]
    for s, d in list(zip(src.tolist(), dst.tolist()))[:300]:
        assert s in indices[indptr[d]:indptr[d + 1]].tolist()


@pytest.mark.gpu
def test_merged_u_mul_v_equals_eager():
    m = _graph()
    seeds = torch.arange(0, 900, 3, device=DEV)
    u, v = torch.rand(m.num_rows(), device=DEV), torch.rand(seeds.numel(), device=DEV)
    c = gs.jit.compile(func=pass_like_sampler, args=(m, seeds, u, v, u + 1, v + 1))
    assert torch.allclose(c(m, seeds, u, v, u + 1, v + 1),
                          pass_like_sampler(m, seeds, u, v, u + 1, v + 1))


@pytest.mark.gpu
def test_fused_div_then_sum_equals_eager():
    m = _graph()
    seeds = torch.arange(0, 900, 3, device=DEV)
    scale = torch.rand(seeds.numel(), device=DEV) + 0.5
    want = div_then_sum_sampler(m, seeds, scale)
    c = gs.jit.compile(func=div_then_sum_sampler, args=(m, seeds, scale))
    assert "_CAPI_FusedEDivUSum" in targets(c.gm)
    got = c(m, seeds, scale)
    assert got.shape == want.shape
    # the row sums accumulate in another order: 1e-5 relative
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    # against float64 arithmetic on the host
    sub = m[:, seeds]
    row, col = (t.cpu().numpy() for t in sub.coo[:2])
    w = sub.edata["w"].double().cpu().numpy()
    exact = np.zeros(sub._graph._CAPI_GetNumRows())
    np.add.at(exact, row, w / scale.double().cpu().numpy()[col])
    assert np.allclose(got.cpu().numpy(), exact, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_compiled_weighted_graphsage_matches_the_cdf_oracle():
    """The fused weighted operator draws through the weight CDF of the input
    matrix: bit-exact against the oracle's CDF sampler with the same seed and
    call ids; the eager path (slice, then key-based sampling) obeys the same
    invariants on the same seeds."""
    from oracle import binding as orc
    m = _graph()
    indptr, indices = m.csc[0].cpu().numpy(), m.csc[1].cpu().numpy()
    w = m.edata["w"].cpu().numpy()
    seeds = torch.randperm(5000, generator=torch.Generator().manual_seed(8))[:300].to(DEV)
    c = gs.jit.compile(func=weighted_graphsage_sampler, args=(m, seeds, [10, 5]))
    gs.manual_seed(21)
    _, blocks = c(m, seeds, [10, 5])
    cdf = orc.weight_cdf(indptr, w, indices, m.num_rows())   # the operator class packs the row ids
    s = seeds.cpu().numpy()
    for layer, (K, blk) in enumerate(zip([10, 5], blocks)):
        sub_indptr, col, rows, sel = orc.sample_weighted(indptr, indices, None, s, K, False,
                                                         seed=21, call_id=layer, cdf=cdf)
        uniq, _, r, cc = orc.unique_relabel(s, rows, edge_col=col)
        assert np.array_equal(blk.row.cpu().numpy(), r)
        assert np.array_equal(blk.col.cpu().numpy(), cc)
        assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq)
        assert np.array_equal(blk.edata["w"].cpu().numpy(), w[sel])
        s = uniq
    # eager: another algorithm, the same rules
    gs.manual_seed(21)
    _, eager = weighted_graphsage_sampler(m, seeds, [10, 5])
    deg = np.diff(indptr)
    s = seeds.cpu().numpy()
    blk = eager[0]
    counts = np.bincount(blk.col.cpu().numpy(), minlength=s.size)
    assert np.array_equal(counts, np.minimum(deg[s], 10))
    src = blk.srcdata["_ID"].cpu().numpy()[blk.row.cpu().numpy()]
    dst = s[blk.col.cpu().numpy()]
    edges = set(zip(np.repeat(np.arange(5000), deg).tolist(), indices.tolist()))
    assert all((int(d), int(u)) in edges for d, u in zip(dst, src))


def two_products_on_the_loaded_matrix(A, u1, v1, u2, v2):
    return gs.ops.u_mul_v(A, u1, v1), gs.ops.u_mul_v(A, u2, v2)


@pytest.mark.gpu
def test_merged_u_mul_v_keeps_the_edge_order_of_a_converted_format():
    """A matrix loaded as an edge list in arbitrary order: whatever format the
    compiled graph runs the merged operator on (a CSC derived from the edge list
    carries the edge ids of the sort), its outputs stay in the order of the
    loaded edges, as the two separate products give them."""
    g = torch.Generator().manual_seed(12)
    row = torch.randint(0, 40, (3000,), generator=g).to(DEV)
    col = torch.randint(0, 30, (3000,), generator=g).to(DEV)
    row[0], col[0] = 39, 29
    m = gs.Matrix()
    m.load_graph("COO", [row, col])
    u1, u2 = torch.rand(40, generator=g).to(DEV), torch.rand(40, generator=g).to(DEV)
    v1, v2 = torch.rand(30, generator=g).to(DEV), torch.rand(30, generator=g).to(DEV)
    c = gs.jit.compile(func=two_products_on_the_loaded_matrix, args=(m, u1, v1, u2, v2))
    assert targets(c.gm).count("_CAPI_FusedUOPV") == 1
    for fmt in (gs._COO, gs._CSC):
        o1, o2 = gs.ops.fused_u_mul_v(m, u1, v1, u2, v2, fmt)
        assert torch.equal(o1, u1[row] * v1[col]) and torch.equal(o2, u2[row] * v2[col])
    got = c(m, u1, v1, u2, v2)
    want = two_products_on_the_loaded_matrix(m, u1, v1, u2, v2)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    assert torch.equal(want[0], u1[row] * v1[col])


@pytest.mark.gpu
def test_try_compact_runs_the_search_and_leaves_the_random_state_alone():
    """try_compact=True builds and times both variants on the example arguments
    and keeps one of them; the sampler's (seed, next call id) is what it was, so
    the compiled function still draws the picks of an uncompiled run started
    from the same state when the plain variant won, and valid blocks either way."""
    m = _graph()
    seeds = torch.arange(0, 2000, 9, device=DEV)
    gs.manual_seed(31)
    before = gs.random_state()
    c = gs.jit.compile(func=graphsage_sampler, args=(m, seeds, [10, 5]), try_compact=True)
    assert gs.random_state() == before
    assert c.compact_search_ms is not None and len(c.compact_search_ms) == 2
    assert c.compact == (c.compact_search_ms[1] < c.compact_search_ms[0])
    out = c(m, seeds, [10, 5])
    assert gs.random_state() == (31, 2)
    blocks = out[-1]
    assert blocks[0].num_dst == seeds.numel() and blocks[1].num_dst == blocks[0].num_src
    indptr, indices, _ = m.csc
    src = blocks[0].srcdata["_ID"][blocks[0].row]
    dst = seeds[blocks[0].col]
    lo, hi = indptr[dst], indptr[dst + 1]
    # every block edge is an edge of the graph: its source occurs in the column of its target
    found = torch.zeros_like(src, dtype=torch.bool)
    for k in range(int((hi - lo).max())):
        pos = (lo + k).clamp(max=indices.numel() - 1)
        found |= (lo + k < hi) & (indices[pos] == src)
    assert bool(found.all())
    d = gs.jit.compile(func=graphsage_sampler, args=(m, seeds, [10, 5]))
    assert d.compact is False and d.compact_search_ms is None


@pytest.mark.gpu
def test_a_searched_compile_that_keeps_the_plain_variant_draws_the_same_samples(monkeypatch):
    """try_compact=True really runs both variants on the example arguments; when the
    plain one is kept, the compiled sampler returns what an unsearched compile
    returns from the same random state (nothing the search ran is left behind in
    the matrix's caches)."""
    m = _graph()
    seeds = torch.arange(3, 3000, 7, device=DEV)
    real = gs.jit.compile._time
    verdict = iter([1.0, 2.0])                     # plain, then compact: plain wins

    def timed(self, gm, args, runs=3):
        real(self, gm, args, runs)
        return next(verdict)

    monkeypatch.setattr(gs.jit.compile, "_time", timed)
    gs.manual_seed(77)
    c = gs.jit.compile(func=graphsage_sampler, args=(m, seeds, [10, 5]), try_compact=True)
    assert c.compact is False and c.compact_search_ms == (1.0, 2.0)
    assert gs.random_state() == (77, 0)
    s_in, s_out, s_blocks = c(m, seeds, [10, 5])
    monkeypatch.undo()
    gs.manual_seed(77)
    d = gs.jit.compile(func=graphsage_sampler, args=(m, seeds, [10, 5]))   # try_compact=None
    p_in, p_out, p_blocks = d(m, seeds, [10, 5])
    assert torch.equal(s_in, p_in) and torch.equal(s_out, p_out)
    for a, b in zip(s_blocks, p_blocks):
        _blocks_equal(a, b)


def _batch_relabel_graph(ids_for_blocks_late: bool, same_ids: bool):
    """A hand-made trace: all_nodes() first, the block builder after it, with the
    builder's id tensor either the same node or another one (made before or after
    the all_nodes() call)."""
    import operator
    from torch import fx
    g = fx.Graph()
    graph, seeds, rows = g.placeholder("graph"), g.placeholder("seeds"), g.placeholder("rows")
    other = seeds if same_ids else None
    if not same_ids and not ids_for_blocks_late:
        other = g.call_function(operator.add, args=(seeds, 1))
    valid = g.call_method("_CAPI_BatchGetValidNodes", args=(graph, seeds, rows))
    frontier = g.call_function(operator.getitem, args=(valid, 0))
    ptr = g.call_function(operator.getitem, args=(valid, 1))
    if other is None:
        other = g.call_function(operator.add, args=(seeds, 1))
    blocks = g.call_method("_CAPI_BatchBlocks", args=(graph, other, rows))
    g.output((frontier, ptr, blocks))
    return fx.GraphModule(torch.nn.Module(), g)


@pytest.mark.parametrize("late", [False, True])
def test_all_nodes_is_not_read_off_a_block_batch_built_from_other_ids(late):
    """The builder's frontier stands in for all_nodes() only when both were given the
    same id tensors; with other ids nothing moves (in particular not the builder in
    front of an argument that is made later) and the graph stays well-formed."""
    from gsampler_amd.jit import passes
    gm = passes.merge_relabel_and_all_nodes(_batch_relabel_graph(late, same_ids=False))
    gm.graph.lint()
    t = targets(gm)
    assert t == ["_CAPI_BatchGetValidNodes", "_CAPI_BatchBlocks"]


def test_all_nodes_is_read_off_the_block_batch_built_from_the_same_ids():
    from gsampler_amd.jit import passes
    gm = passes.merge_relabel_and_all_nodes(_batch_relabel_graph(False, same_ids=True))
    gm.graph.lint()
    t = targets(gm)
    assert "_CAPI_BatchGetValidNodes" not in t
    assert t == ["_CAPI_BatchBlocks", "frontier", "frontier_ptr"]   # the builder came first
