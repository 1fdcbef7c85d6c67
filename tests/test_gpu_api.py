"""The drop-in API (gs.Matrix / gs.BatchMatrix over gs_classes.Graph) against
the CPU oracle: the samplers below are the reference's example functions
(examples/graphsage/graphsage.py:7-28) run unchanged on `gsampler_amd`."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd.utils import batched_seeds, rmat_csc
from oracle import binding as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


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


@pytest.fixture(scope="module")
def graph():
    indptr, indices = rmat_csc(20000, 400000, seed=1)
    m = gs.Matrix()
    m.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    return m, indptr.numpy(), indices.numpy()


def oracle_layers(indptr, indices, seeds, ptr, fanouts, first_call):
    out = []
    for layer, fanout in enumerate(fanouts):
        s, c, rows, sel = orc.sample_uniform(indptr, indices, seeds, fanout, False, 0, 7777,
                                             first_call + layer)
        eptr = s[ptr] if ptr is not None else None
        uniq, uptr, r, cc = orc.unique_relabel(seeds, rows, ptr, eptr, c)
        out.append((uniq, uptr, r, cc, sel))
        seeds, ptr = uniq, (uptr if ptr is not None else None)
    return out


def test_load_graph_shape(graph):
    m, indptr, indices = graph
    assert m.num_cols() == 20000 and m.num_rows() == int(indices.max()) + 1
    assert m.num_edges() == indices.size
    assert torch.equal(m.csc[0].cpu(), torch.from_numpy(indptr))


def test_matrix_graphsage_matches_oracle(graph):
    m, indptr, indices = graph
    seeds = torch.randperm(20000, generator=torch.Generator().manual_seed(3))[:256]
    gs.manual_seed(7777)
    inp, outp, blocks = graphsage_sampler(m, seeds.to(DEV), [25, 10])
    want = oracle_layers(indptr, indices, seeds.numpy(), None, [25, 10], 0)
    assert torch.equal(inp.cpu(), seeds)
    for blk, (uniq, uptr, r, c, sel) in zip(blocks, want):
        assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq)
        assert np.array_equal(blk.row.cpu().numpy(), r)
        assert np.array_equal(blk.col.cpu().numpy(), c)
        assert blk.num_src == uniq.size
    assert np.array_equal(outp.cpu().numpy(), want[-1][0])
    assert blocks[0].num_dst == 256 and blocks[1].num_dst == want[0][0].size
    # distinct seeds lead the frontier
    assert np.array_equal(want[0][0][:256], seeds.numpy())


def test_fused_operator_equals_slice_then_sample(graph):
    """_CAPI_SlicingSampling (what the JIT emits) picks the same edges as
    _CAPI_Slicing + _CAPI_Sampling with the same call id."""
    m, indptr, indices = graph
    seeds = torch.arange(0, 3000, 7, device=DEV)
    gs.manual_seed(11)
    sub, _ = m._graph._CAPI_Slicing(seeds, 1, gs._CSC, gs._CSC | gs._COO)
    a, a_idx = sub._CAPI_Sampling(1, 10, False, gs._CSC, gs._CSC | gs._COO)
    gs.manual_seed(11)
    b, b_idx = m._graph._CAPI_SlicingSampling(1, seeds, 10, False, gs._CSC, gs._CSC | gs._COO)
    assert torch.equal(a._CAPI_GetCSCIndptr(), b._CAPI_GetCSCIndptr())
    assert torch.equal(a._CAPI_GetCSCIndices(), b._CAPI_GetCSCIndices())
    assert torch.equal(a._CAPI_GetCOOCols(), b._CAPI_GetCOOCols())
    # the fused operator's edge index addresses the parent matrix directly
    assert torch.equal(m.csc[1][b_idx], b._CAPI_GetCSCIndices())


def test_batch_matrix_graphsage_matches_oracle(graph):
    m, indptr, indices = graph
    seeds, ptr = batched_seeds(20000, 8, 128, seed=5)
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    gs.manual_seed(7777)
    blocks_per_layer = batch_graphsage_sampler(bm, seeds.to(DEV), ptr.to(DEV), [15, 10, 5])
    want = oracle_layers(indptr, indices, seeds.numpy(), ptr.numpy(), [15, 10, 5], 0)
    o_ptr = ptr.numpy()
    for blocks, (uniq, uptr, r, c, sel) in zip(blocks_per_layer, want):
        assert len(blocks) == 8
        s_counts = np.diff(o_ptr)
        for b, blk in enumerate(blocks):
            assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq[uptr[b]:uptr[b + 1]])
            assert blk.num_dst == s_counts[b] and blk.num_src == uptr[b + 1] - uptr[b]
        got_r = torch.cat([blk.row for blk in blocks]).cpu().numpy()
        got_c = torch.cat([blk.col for blk in blocks]).cpu().numpy()
        assert np.array_equal(got_r, r) and np.array_equal(got_c, c)
        o_ptr = uptr


def test_coo_and_csr_views_round_trip(graph):
    m, indptr, indices = graph
    sub = m[:, torch.arange(0, 500, device=DEV)]
    row, col, _ = sub.coo
    ci, cx, _ = sub.csc
    ri, rx, r_eids = sub.csr
    import scipy.sparse as sp
    a = sp.csc_matrix((np.ones(cx.numel()), cx.cpu().numpy(), ci.cpu().numpy()),
                      shape=(sub.num_rows(), sub.num_cols()))
    b = sp.csr_matrix((np.ones(rx.numel()), rx.cpu().numpy(), ri.cpu().numpy()),
                      shape=(sub.num_rows(), sub.num_cols()))
    assert (a != b).nnz == 0
    # CSR e_ids map CSR order back to the COO / CSC edge order
    assert torch.equal(col[r_eids], rx)


def test_errors_are_exceptions_not_aborts(graph):
    m, _, _ = graph
    with pytest.raises(RuntimeError, match="GPU"):
        m._graph._CAPI_Slicing(torch.arange(3), 1, gs._CSC, gs._COO)
    with pytest.raises(RuntimeError, match="int64"):
        m._graph._CAPI_Slicing(torch.arange(3, device=DEV, dtype=torch.int32), 1, gs._CSC, gs._COO)
    with pytest.raises(RuntimeError, match="cannot produce"):
        m._graph._CAPI_Slicing(torch.arange(3, device=DEV), 1, gs._CSC, gs._CSR)
    with pytest.raises(RuntimeError, match="not implemented"):
        m._graph._CAPI_Sampling(0, 3, False, gs._CSC, gs._COO)


def test_edge_operators_reject_operands_that_would_be_read_out_of_bounds(graph):
    """Feature tensors shorter than the axis they are indexed by, outputs that
    are too small and mixed element types raise before any kernel runs."""
    m, _, _ = graph
    sub = m[:, torch.arange(0, 300, device=DEV)]
    g = sub._graph
    R, C, E = g._CAPI_GetNumRows(), g._CAPI_GetNumCols(), g._CAPI_GetNumEdges()
    f = lambda n, dtype=torch.float32: torch.ones(n, device=DEV, dtype=dtype)
    out_e, out_c = f(E), torch.zeros(C, device=DEV)
    with pytest.raises(RuntimeError, match="lhs has"):
        g._CAPI_SDDMM("mul", f(R - 1), f(C), out_e, 0, 2, gs._COO)
    with pytest.raises(RuntimeError, match="rhs has"):
        g._CAPI_SDDMM("mul", f(R), f(C - 1), out_e, 0, 2, gs._CSC)
    with pytest.raises(RuntimeError, match="out has"):
        g._CAPI_SDDMM("mul", f(R), f(C), f(E - 1), 0, 2, gs._COO)
    with pytest.raises(RuntimeError, match="but out is"):
        g._CAPI_SDDMM("mul", f(R, torch.float64), f(C), out_e, 0, 2, gs._COO)
    with pytest.raises(RuntimeError, match="targets"):
        g._CAPI_SDDMM("mul", f(R), f(C), out_e, 0, 3, gs._COO)
    with pytest.raises(RuntimeError, match="efeat has"):
        g._CAPI_SpMM("copy_rhs", "sum", None, f(E - 1), out_c, None, None, 0, gs._CSC)
    with pytest.raises(RuntimeError, match="ufeat has"):
        g._CAPI_SpMM("mul", "sum", f(R - 1), f(E), out_c, None, None, 0, gs._CSC)
    with pytest.raises(RuntimeError, match="out has"):
        g._CAPI_SpMM("copy_rhs", "sum", None, f(E), out_c[:-1].contiguous(), None, None, 0, gs._CSC)
    with pytest.raises(RuntimeError, match="efeat has"):
        g._CAPI_FusedESquareSum("copy_rhs", "sum", None, f(E - 1), out_c, None, None, 0, gs._CSC)
    with pytest.raises(RuntimeError, match="ufeat has"):
        g._CAPI_FusedEDivUSum("div", "sum", f(R - 1), f(E), out_c, None, None, 0, gs._CSC)
    with pytest.raises(RuntimeError, match="lhs has"):
        g._CAPI_FusedUOPV("mul", f(R - 1), f(C), f(E), f(R - 1), f(C), f(E), gs._COO)
    # and the well-formed calls still work
    g._CAPI_SDDMM("mul", f(R), f(C), out_e, 0, 2, gs._COO)
    g._CAPI_SpMM("copy_rhs", "sum", None, f(E), out_c, None, None, 0, gs._CSC)
    assert float(out_c.sum()) == pytest.approx(E)


def test_malformed_matrices_are_refused_at_load():
    ok_ptr = torch.tensor([0, 2, 2, 5], device=DEV)
    ok_idx = torch.tensor([0, 3, 1, 2, 3], device=DEV)
    gs.Graph(4, 3)._CAPI_LoadCSC(ok_ptr, ok_idx)
    with pytest.raises(RuntimeError, match="entries for"):
        gs.Graph(4, 4)._CAPI_LoadCSC(ok_ptr, ok_idx)
    with pytest.raises(RuntimeError, match="must run from 0"):
        gs.Graph(4, 3)._CAPI_LoadCSC(torch.tensor([0, 2, 2, 6], device=DEV), ok_idx)
    with pytest.raises(RuntimeError, match="must not decrease"):
        gs.Graph(4, 3)._CAPI_LoadCSC(torch.tensor([0, 3, 2, 5], device=DEV), ok_idx)
    with pytest.raises(RuntimeError, match="indices must lie"):
        gs.Graph(3, 3)._CAPI_LoadCSC(ok_ptr, ok_idx)
    with pytest.raises(RuntimeError, match="indices must lie"):
        gs.Graph(4, 3)._CAPI_LoadCSR(torch.tensor([0, 2, 2, 4, 5], device=DEV), ok_idx)
    with pytest.raises(RuntimeError, match="column ids"):
        gs.Graph(4, 3)._CAPI_LoadCOO(ok_idx, torch.tensor([0, 0, 2, 2, 3], device=DEV), False, False)
    with pytest.raises(RuntimeError, match="row ids"):
        gs.Graph(4, 3)._CAPI_LoadCOO(ok_idx - 1, torch.tensor([0, 0, 2, 2, 2], device=DEV), False, False)


def test_batch_offsets_from_the_caller_are_checked(graph):
    m, _, _ = graph
    g = m._graph
    seeds = torch.arange(0, 600, device=DEV)
    good = torch.tensor([0, 200, 200, 600], device=DEV)
    g._CAPI_BatchFusedSlicingSampling(seeds, good, 5, False)
    for bad in ([0, 200, 700], [0, 300, 200, 600], [1, 200, 600], [0, 200, 500]):
        ptr = torch.tensor(bad, device=DEV)
        with pytest.raises(RuntimeError, match="batch offsets"):
            g._CAPI_BatchFusedSlicingSampling(seeds, ptr, 5, False)
        with pytest.raises(RuntimeError, match="batch offsets"):
            g._CAPI_BatchColSlicing(seeds, ptr, True)
        with pytest.raises(RuntimeError, match="batch offsets"):
            torch.ops.gs_ops._CAPI_BatchListSamplingWithProbs(
                torch.ones(600, device=DEV), 4, False, ptr)
    with pytest.raises(RuntimeError, match="batch offsets"):
        g._CAPI_BatchColRowSlcing(seeds, good, seeds, torch.tensor([0, 100, 200, 601], device=DEV))
    # an array changed in place after it was accepted is looked at again
    ptr = good.clone()
    g._CAPI_BatchFusedSlicingSampling(seeds, ptr, 5, False)
    ptr[3] = 900
    with pytest.raises(RuntimeError, match="batch offsets"):
        g._CAPI_BatchFusedSlicingSampling(seeds, ptr, 5, False)


def test_operators_follow_the_current_stream(graph):
    """Everything is launched on torch's current stream (counts travel on it
    too): a step issued on a side stream of default priority gives the same
    result as on the default stream, without any device-wide synchronisation in
    between."""
    from gsampler_amd import capi
    m, indptr, indices = graph
    g_indptr, g_indices = torch.tensor(indptr, device=DEV), torch.tensor(indices, device=DEV)
    seeds = torch.arange(0, 20000, 7, device=DEV)

    def step():
        gs.manual_seed(21)
        sub = m[:, seeds].individual_sampling(10, None, False)
        block = sub.to_dgl_block()
        raw = capi.sample_uniform(g_indptr, g_indices, seeds, 10, False, 0, 7777, 3)
        return sub.all_nodes(), block.row, block.col, raw[2]

    want = step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = step()
    side.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_super_batch_with_an_empty_batch(graph):
    """A mini-batch without seeds travels through the super-batched sampler as
    an empty block; its neighbours are unaffected."""
    m, _, _ = graph
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    first = torch.arange(0, 20000, 101, device=DEV)
    third = torch.arange(7, 20000, 131, device=DEV)
    seeds = torch.cat([first, third])
    ptr = torch.tensor([0, first.numel(), first.numel(), seeds.numel()], device=DEV)

    def sampler(A, seeds, seeds_ptr, fanouts):
        out = []
        for k in fanouts:
            sub = A[:, seeds::seeds_ptr].individual_sampling(k, None, False)
            seeds, seeds_ptr = sub.all_nodes()
            out.append(sub.to_dgl_block())
        return out

    gs.manual_seed(2)
    eager = sampler(bm, seeds, ptr, [6, 3])
    compiled = gs.jit.compile(func=sampler, args=(bm, seeds, ptr, [6, 3]))
    gs.manual_seed(2)
    jit = compiled(bm, seeds, ptr, [6, 3])
    for layers in (eager, jit):
        assert [len(per_batch) for per_batch in layers] == [3, 3]
        for per_batch in layers:
            empty = per_batch[1]
            assert empty.num_edges() == 0 and empty.num_src == 0 and empty.num_dst == 0
        assert torch.equal(layers[0][0].srcdata["_ID"][: first.numel()], first)
        assert torch.equal(layers[0][2].srcdata["_ID"][: third.numel()], third)
    for a, b in zip(eager, jit):
        for x, y in zip(a, b):
            assert torch.equal(x.row, y.row) and torch.equal(x.col, y.col)
            assert torch.equal(x.srcdata["_ID"], y.srcdata["_ID"])


def test_batch_pointer_is_bound_to_the_length_it_was_checked_for(graph):
    """An offsets array accepted for one id tensor is not accepted for a shorter
    one, and the batched relabel refuses seeds that do not match the batch
    pointer of the slice (the kernels would read past their end)."""
    m, _, _ = graph
    g = m._graph
    seeds = torch.arange(600, device=DEV)
    ptr = torch.tensor([0, 100, 200, 600], device=DEV)
    sub, _ = g._CAPI_BatchFusedSlicingSampling(seeds, ptr, 5, False)
    with pytest.raises(RuntimeError, match="batch offsets"):
        g._CAPI_BatchFusedSlicingSampling(seeds[:500], ptr, 5, False)
    with pytest.raises(RuntimeError, match="batch offsets"):
        sub._CAPI_BatchGraphRelabel(seeds[:590], torch.empty(0, dtype=torch.int64, device=DEV))
    with pytest.raises(RuntimeError, match="batch offsets"):
        sub._CAPI_BatchGetValidNodes(seeds[:590], torch.empty(0, dtype=torch.int64, device=DEV))
    uniq, uptr = sub._CAPI_BatchGetValidNodes(seeds, torch.empty(0, dtype=torch.int64, device=DEV))
    # the produced pointer is bound to the frontier it splits
    sub2, _ = g._CAPI_BatchFusedSlicingSampling(uniq, uptr, 5, False)
    with pytest.raises(RuntimeError, match="batch offsets"):
        g._CAPI_BatchFusedSlicingSampling(uniq[:-1], uptr, 5, False)


def test_block_batch_emits_edge_list_and_compressed_form(graph):
    """to_dgl_block of a super-batch: one operator call lays out every block; the
    compressed form by destination of each block equals SciPy's conversion of the
    block's edge list, the blocks equal the per-batch split of the relabelled
    super-batch, and per-edge data travels with the edges."""
    import scipy.sparse as sp
    m, indptr, indices = graph
    seeds, ptr = batched_seeds(20000, 6, 100, seed=9)
    seeds[150:200] = seeds[100:150]                 # repeated seeds inside batch 1
    ptr = torch.tensor([0, 100, 250, 250, 400, 401, 600])      # an empty batch, a batch of one
    w = torch.rand(indices.size, device=DEV)
    m2 = gs.Matrix(m._graph, {}, {}, {"w": w})
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m2, False)
    gs.manual_seed(3)
    sub = bm[:, seeds.to(DEV)::ptr.to(DEV)].individual_sampling(7, None, False)
    blocks = sub.to_dgl_block(prefetch_edata={"w"})
    frontier, fptr, row, col, eids, eptr = sub._graph._CAPI_BatchGraphRelabel(
        seeds.to(DEV), torch.empty(0, dtype=torch.int64))
    assert len(blocks) == 6 and blocks.totals() == (frontier.numel(), 600, row.numel())
    fptr, eptr = fptr.tolist(), eptr.tolist()
    whole_w = sub.edata["w"]
    listed = list(blocks)
    assert listed[2].num_edges() == 0 and listed[2].num_dst == 0 and listed[2].num_src == 0
    assert blocks[-1] is listed[5] and blocks[1:3] == listed[1:3]
    for b, blk in enumerate(listed):
        lo, hi = eptr[b], eptr[b + 1]
        assert torch.equal(blk.row, row[lo:hi]) and torch.equal(blk.col, col[lo:hi])
        assert torch.equal(blk.srcdata["_ID"], frontier[fptr[b]:fptr[b + 1]])
        assert torch.equal(blk.edata["w"], whole_w[lo:hi])
        assert blk.num_dst == int(ptr[b + 1] - ptr[b]) and blk.num_src == fptr[b + 1] - fptr[b]
        b_indptr, b_indices, _ = blk.csc()
        assert b_indptr.numel() == blk.num_dst + 1 and int(b_indptr[0]) == 0
        ones = np.ones(blk.num_edges())
        from_coo = sp.coo_matrix((ones, (blk.row.cpu().numpy(), blk.col.cpu().numpy())),
                                 shape=(max(blk.num_src, 1), max(blk.num_dst, 1))).tocsc()
        direct = sp.csc_matrix((ones, b_indices.cpu().numpy(),
                                np.concatenate([b_indptr.cpu().numpy(),
                                                [] if blk.num_dst else [0]]).astype(np.int64)),
                               shape=(max(blk.num_src, 1), max(blk.num_dst, 1)))
        assert (from_coo != direct).nnz == 0        # parallel edges add up on both sides
        # and entry by entry: offsets are the running count of edges per destination,
        # the indices are the edges' sources in their (destination-grouped) order
        counts = np.bincount(blk.col.cpu().numpy(), minlength=blk.num_dst)
        assert np.array_equal(b_indptr.cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
        mine = seeds[int(ptr[b]):int(ptr[b + 1])]
        distinct = torch.unique(mine).numel() == mine.numel()
        assert (b == 1) <= (not distinct)
        if not distinct:
            # repeated seeds share the label of their first occurrence: the offsets
            # by seed position do not describe this block, so none are handed out
            # and the compressed form is derived from the edge list
            assert blk.indptr is None
            assert counts[torch.unique(mine).numel():].sum() == 0
        else:
            assert blk.indptr is not None and torch.equal(b_indices, blk.row)
            assert bool((blk.col[1:] >= blk.col[:-1]).all())
    # a block asked for on its own, before anything else was materialised
    again = sub.to_dgl_block()
    one = again[3]
    assert torch.equal(one.row, listed[3].row) and "w" not in one.edata
    # a block built from an edge list alone derives its compressed form
    loose = gs.utils.block.Block(listed[0].row, listed[0].col, listed[0].num_src, listed[0].num_dst)
    li, lx, _ = loose.csc()
    assert torch.equal(li, listed[0].csc()[0]) and torch.equal(lx, listed[0].csc()[1])


def test_writes_that_go_around_torch_need_invalidate_caches():
    """A matrix of a million edges or more keeps an int32 copy of its row ids for the uniform
    sampler, keyed by the tensor's identity and version counter.  A write through a raw
    pointer moves neither: the sampler goes on reading the copy until
    _CAPI_InvalidateCaches() ages everything that was derived from tensor contents."""
    from gsampler_amd import capi
    nodes = 60_000
    indptr, indices = rmat_csc(nodes, 1_500_000, seed=3)
    indptr, indices = indptr.to(DEV), indices.to(DEV)
    m = gs.Matrix()
    m.load_graph("CSC", [indptr, indices])
    seeds = torch.arange(0, 4000, device=DEV)

    def sample():                                      # the fused operator reads the copy
        gs.manual_seed(11)
        sub, _ = m._graph._CAPI_SlicingSampling(1, seeds, 5, False, gs._CSC, gs._COO)
        return sub._CAPI_GetCOORows().clone()

    before = sample()
    other = (indices + 1) % nodes                      # another graph on the same offsets
    capi.probe_stream_copy(other, indices)             # raw pointers: no version bump
    torch.cuda.synchronize()
    assert torch.equal(indices, other)
    stale = sample()
    assert torch.equal(stale, before)                  # still the picks of the old ids
    torch.ops.gs_ops._CAPI_InvalidateCaches()
    fresh = sample()
    assert torch.equal(fresh, (before + 1) % nodes)    # same positions, the new ids


def test_the_int32_copy_of_the_ids_can_be_switched_off():
    """Same picks with and without the copy; without it a matrix keeps no extra array."""
    nodes = 60_000
    indptr, indices = rmat_csc(nodes, 1_500_000, seed=4)
    m = gs.Matrix()
    m.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    seeds = torch.arange(100, 3100, device=DEV)

    def sample():
        gs.manual_seed(5)
        sub, _ = m._graph._CAPI_SlicingSampling(1, seeds, 7, False, gs._CSC, gs._COO)
        return sub._CAPI_GetCOORows().clone()

    with_copy = sample()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.ops.gs_ops._CAPI_SetNarrowIds(False)
    try:
        without = sample()
        torch.cuda.synchronize()
        assert torch.equal(with_copy, without)
        # the 6 MB copy is gone (everything else the call allocated was released again)
        assert torch.cuda.memory_allocated() <= base - 4 * 1_500_000 + (1 << 20)
    finally:
        torch.ops.gs_ops._CAPI_SetNarrowIds(True)
