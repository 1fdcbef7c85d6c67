"""The headline workload at its full size (2.45 M nodes, 124 M edges, 64 x 1024
seeds, fan-outs 15/10/5) through the C ABI: size-independent properties checked
on the device for every layer, and the whole step compared bit for bit with the
CPU restatement (which finishes a step of this size in well under a second).
The weighted variant (persistent weight CDF) and node2vec on the same graph are
covered the same way."""
import numpy as np
import pytest
import torch

from gsampler_amd import capi
from oracle import binding as orc

pytestmark = pytest.mark.gpu

NODES, EDGES = 2_450_000, 124_000_000
FANOUTS = [15, 10, 5]


@pytest.fixture(scope="module")
def graph():
    from gsampler_amd.utils import batched_seeds, chung_lu_csc
    dev = torch.device("cuda:0")
    indptr, indices = chung_lu_csc(NODES, EDGES, seed=1, device=dev)
    seeds, ptr = batched_seeds(NODES, 64, 1024, seed=2, device=dev)
    return indptr, indices, seeds, ptr


def batch_of(ptr, n):
    """Batch index of every position 0..n-1 for an offsets array."""
    return torch.searchsorted(ptr, torch.arange(n, device=ptr.device), right=True) - 1


def check_sampled_layer(indptr, indices, seeds, fanout, out):
    sub_indptr, coo_col, rows, sel = out
    deg = indptr[seeds + 1] - indptr[seeds]
    assert torch.equal(sub_indptr[1:] - sub_indptr[:-1], deg.clamp(max=fanout))
    assert int(sub_indptr[0]) == 0 and int(sub_indptr[-1]) == rows.numel()
    assert bool((coo_col[1:] >= coo_col[:-1]).all())               # column-sorted
    col = seeds[coo_col]
    assert bool(((sel >= indptr[col]) & (sel < indptr[col + 1])).all())   # an edge of that column
    assert torch.equal(rows, indices[sel])
    # no edge twice within one requested column
    pair = coo_col * EDGES + sel
    assert torch.unique(pair).numel() == pair.numel()


def check_relabelled_layer(seeds, ptr, rows, edge_ptr, coo_col, out, nodes=NODES, batches=64):
    NODES = nodes
    uniq, uniq_ptr, out_row, out_col = out
    B = ptr.numel() - 1
    assert int(uniq_ptr[0]) == 0 and int(uniq_ptr[-1]) == uniq.numel()
    assert bool((uniq_ptr[1:] >= uniq_ptr[:-1]).all())
    ub = batch_of(uniq_ptr, uniq.numel())
    # a batch's frontier holds every id once ...
    assert torch.unique(ub * NODES + uniq).numel() == uniq.numel()
    # ... starts with its seeds (the seeds of this workload are distinct per batch) ...
    sb = batch_of(ptr, seeds.numel())
    local = torch.arange(seeds.numel(), device=seeds.device) - ptr[sb]
    assert torch.equal(uniq[uniq_ptr[sb] + local], seeds)
    # ... and is exactly the set of ids of seeds ++ rows
    eb = batch_of(edge_ptr, rows.numel())
    keys = torch.cat([sb * NODES + seeds, eb * NODES + rows])
    assert torch.unique(keys).numel() == uniq.numel()
    # relabelling round-trips
    assert torch.equal(uniq[uniq_ptr[eb] + out_row], rows)
    assert torch.equal(uniq[uniq_ptr[eb] + out_col], seeds[coo_col])
    assert B == batches


def same(gpu, cpu):
    for g, c in zip(gpu, cpu):
        assert np.array_equal(g.cpu().numpy(), c)


def test_graphsage_step_properties_and_oracle(graph):
    indptr, indices, seeds, ptr = graph
    h_indptr, h_indices = indptr.cpu().numpy(), indices.cpu().numpy()
    h_seeds, h_ptr = seeds.cpu().numpy(), ptr.cpu().numpy()
    total = 0
    for layer, fanout in enumerate(FANOUTS):
        out = capi.sample_uniform(indptr, indices, seeds, fanout, False, 0, 7777, layer)
        check_sampled_layer(indptr, indices, seeds, fanout, out)
        want = orc.sample_uniform(h_indptr, h_indices, h_seeds, fanout, False, 0, 7777, layer)
        same(out, want)
        sub_indptr, coo_col, rows, _ = out
        edge_ptr = sub_indptr[ptr]
        rel = capi.unique_relabel(seeds, rows, ptr, edge_ptr, coo_col)
        check_relabelled_layer(seeds, ptr, rows, edge_ptr, coo_col, rel)
        want_rel = orc.unique_relabel(h_seeds, want[2], h_ptr, want[0][h_ptr], want[1])
        same(rel, want_rel)
        total += rows.numel()
        seeds, ptr = rel[0], rel[1]
        h_seeds, h_ptr = want_rel[0], want_rel[1]
    assert total > 20_000_000          # the step really is the full-size one


def test_weighted_step_with_persistent_cdf(graph):
    indptr, indices, seeds, ptr = graph
    g = torch.Generator(device=indices.device)
    g.manual_seed(5)
    probs = torch.randn(indices.numel(), generator=g, device=indices.device).exp_().float()
    nodes = indptr.numel() - 1
    cdf = capi.weight_cdf(indptr, probs, indices, nodes)
    h_indptr, h_indices, h_probs = indptr.cpu().numpy(), indices.cpu().numpy(), probs.cpu().numpy()
    h_cdf = orc.weight_cdf(h_indptr, h_probs, h_indices, nodes)
    assert np.array_equal(cdf.cpu().numpy(), h_cdf)
    out = capi.sample_weighted(indptr, indices, probs, seeds, 15, False, 7777, 0, cdf=cdf)
    check_sampled_layer(indptr, indices, seeds, 15, out)
    want = orc.sample_weighted(h_indptr, h_indices, h_probs, seeds.cpu().numpy(), 15, False,
                               7777, 0, cdf=h_cdf)
    same(out, want)
    # a second, larger layer: the frontier of the first
    edge_ptr = out[0][ptr]
    rel = capi.unique_relabel(seeds, out[2], ptr, edge_ptr, out[1])
    out2 = capi.sample_weighted(indptr, indices, probs, rel[0], 10, False, 7777, 1, cdf=cdf)
    check_sampled_layer(indptr, indices, rel[0], 10, out2)
    want2 = orc.sample_weighted(h_indptr, h_indices, h_probs, rel[0].cpu().numpy(), 10, False,
                                7777, 1, cdf=h_cdf)
    same(out2, want2)


def _check_walk_trace(indptr, indices, start, trace, length, steps):
    """Properties of a walk trace that hold at any size: row 0 is the start nodes; every hop
    follows an edge of the matrix (columns hold in-neighbours and are sorted); a walk that
    stopped stays at -1."""
    walks = start.numel()
    assert trace.shape == (length + 1, walks) and torch.equal(trace[0], start)
    for step in steps:
        prev, cur = trace[step - 1], trace[step]
        alive = cur >= 0
        assert bool((prev[alive] >= 0).all())
        p, c = prev[alive], cur[alive]
        lo, hi = indptr[p], indptr[p + 1]
        # lower bound of c inside [lo, hi), all walks at once
        left, right = lo.clone(), hi.clone()
        for _ in range(24):                       # degrees stay below 2^24
            active = left < right
            mid = (left + right) // 2
            less = indices[mid.clamp(max=EDGES - 1)] < c
            left = torch.where(active & less, mid + 1, left)
            right = torch.where(active & ~less, mid, right)
        assert bool(((left < hi) & (indices[left.clamp(max=EDGES - 1)] == c)).all())
        dead = ~alive
        assert bool((trace[step:, dead] == -1).all())
        # a walk only stops at a node without in-neighbours
        stopped = (prev >= 0) & dead
        ps = prev[stopped]
        assert bool((indptr[ps + 1] == indptr[ps]).all())


def test_edge_list_sort_at_full_size(graph):
    """The 124 M column ids of the headline graph in shuffled order (15 137 tiles a pass, three
    passes): positions and ids against torch's stable sort, and what holds at any size --
    the positions are a permutation, ids ascend, equal ids keep their order."""
    indptr, _, _, _ = graph
    col = capi.csc2coo(indptr, EDGES)
    g = torch.Generator(device=col.device)
    g.manual_seed(9)
    shuffled = col[torch.randperm(EDGES, generator=g, device=col.device)]
    ids, perm = capi.coo_sort(shuffled, NODES)
    assert torch.equal(ids, col)                               # the ids in order are the CSC's columns
    assert torch.equal(shuffled[perm], ids)
    assert bool(((ids[1:] > ids[:-1]) | (perm[1:] > perm[:-1])).all())   # stable
    seen = torch.zeros(EDGES, dtype=torch.bool, device=col.device)
    seen[perm] = True
    assert bool(seen.all())
    want = torch.sort(shuffled, stable=True)
    assert torch.equal(perm, want.indices)


def test_node2vec_walks(graph):
    indptr, indices, _, _ = graph
    indices = capi.segment_sort(indptr, indices, NODES)
    g = torch.Generator(device=indices.device)
    g.manual_seed(3)
    walks, length = 200_000, 80
    start = torch.randint(0, NODES, (walks,), generator=g, device=indices.device)
    trace = capi.node2vec(indptr, indices, start, length, 2.0, 0.5, 7777, 0)
    _check_walk_trace(indptr, indices, start, trace, length, (1, 2, 40, 80))
    want = orc.node2vec(indptr.cpu().numpy(), indices.cpu().numpy(), start.cpu().numpy(),
                        length, 2.0, 0.5, 7777, 0)
    assert np.array_equal(trace.cpu().numpy(), want)


def test_node2vec_walks_at_the_configured_size(graph):
    """1 M walks of 80 steps, p = 2, q = 0.5 (648 MB of trace), through the properties alone;
    the first 20 000 walks also against the CPU walks bit for bit (a walk depends on its
    position among the start nodes only, so a prefix of the launch is a launch of its own).
    With p = 2 a step back to the previous node is accepted at both levels of the rejection
    rule and any other neighbour at one of two: the share of steps that return is therefore
    well above the share a first-order walk shows, which is checked as a sanity bound."""
    indptr, indices, _, _ = graph
    indices = capi.segment_sort(indptr, indices, NODES)
    g = torch.Generator(device=indices.device)
    g.manual_seed(3)
    walks, length = 1_000_000, 80
    start = torch.randint(0, NODES, (walks,), generator=g, device=indices.device)
    trace = capi.node2vec(indptr, indices, start, length, 2.0, 0.5, 7777, 0)
    _check_walk_trace(indptr, indices, start, trace, length, (1, 2, 3, 17, 40, 79, 80))
    n = 20_000
    want = orc.node2vec(indptr.cpu().numpy(), indices.cpu().numpy(), start[:n].cpu().numpy(),
                        length, 2.0, 0.5, 7777, 0)
    assert np.array_equal(trace[:, :n].cpu().numpy(), want)
    first_order = capi.random_walk(indptr, indices, start, length, 7777, 1)
    def returns(t):
        back = (t[2:] == t[:-2]) & (t[2:] >= 0)
        return float(back.sum()) / float((t[2:] >= 0).sum())
    assert returns(trace) > 1.5 * returns(first_order)


def test_largest_configuration_weighted_layers():
    """111 M nodes, 1.6 B edges (13 GB of int64 indices, positions beyond 2^30,
    prefix sums of quantised weights that pass 2^61 while the CDF is built): edge-list ingest, CDF build and the
    three weighted layers (fan-outs 15, 10, 5) of 128 x 1024 seeds, each followed
    by unique + relabel over the 128 mini-batches, checked through properties on
    the device."""
    from gsampler_amd.utils import batched_seeds, chung_lu_csc
    dev = torch.device("cuda:0")
    nodes, edges = 111_000_000, 1_600_000_000
    indptr, indices = chung_lu_csc(nodes, edges, seed=1, device=dev)
    assert int(indptr[-1]) == edges and indices.numel() == edges
    assert bool((indptr[1:] >= indptr[:-1]).all())
    assert int(indices.min()) >= 0 and int(indices.max()) < nodes
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    probs = torch.empty(edges, device=dev).normal_(generator=g).exp_()
    cdf = capi.weight_cdf(indptr, probs, indices, nodes)
    row_bits = int(cdf[0])
    assert row_bits == (nodes - 1).bit_length()
    share_bits = min(62, 64 - row_bits)
    # every entry carries its edge's row id ...
    assert bool(((cdf[1:] & ((1 << row_bits) - 1)) == indices).all())
    # ... and inside a column the shares rise to 2^share_bits - 1 (spot check on some columns;
    # entries are unsigned 64-bit words, so shift as such)
    for c in (0, 1, 77, 1_000_000, nodes - 1):
        lo, hi = int(indptr[c]), int(indptr[c + 1])
        if hi > lo:
            share = cdf[lo + 1:hi + 1].cpu().numpy().view(np.uint64) >> np.uint64(row_bits)
            assert int(share[-1]) == (1 << share_bits) - 1
            assert bool((share[1:] >= share[:-1]).all())
            # the edge with the largest weight owns the largest piece
            piece = np.diff(np.concatenate([[0], share.astype(np.int64)]))
            assert int(piece.argmax()) == int(torch.argmax(probs[lo:hi]))
    seeds, ptr = batched_seeds(nodes, 128, 1024, seed=2, device=dev)

    def check(seeds, fanout, out):
        sub_indptr, coo_col, rows, sel = out
        deg = indptr[seeds + 1] - indptr[seeds]
        assert torch.equal(sub_indptr[1:] - sub_indptr[:-1], deg.clamp(max=fanout))
        col = seeds[coo_col]
        assert bool(((sel >= indptr[col]) & (sel < indptr[col + 1])).all())
        assert torch.equal(rows, indices[sel])
        assert torch.unique(coo_col * edges + sel).numel() == sel.numel()
        # positive weights only, unless the column has fewer than fanout of them
        zero = probs[sel] <= 0
        assert int(zero.sum()) == 0

    # all three layers of 128 mini-batches: sample, then unique + relabel
    total = 0
    for layer, fanout in enumerate(FANOUTS):
        out = capi.sample_weighted(indptr, indices, probs, seeds, fanout, False, 7777, layer,
                                   cdf=cdf)
        check(seeds, fanout, out)
        sub_indptr, coo_col, rows, _ = out
        edge_ptr = sub_indptr[ptr]
        rel = capi.unique_relabel(seeds, rows, ptr, edge_ptr, coo_col)
        check_relabelled_layer(seeds, ptr, rows, edge_ptr, coo_col, rel, nodes=nodes, batches=128)
        total += rows.numel()
        seeds, ptr = rel[0], rel[1]
    assert total > 20_000_000 and ptr.numel() == 129


# ------------------------------------------------------------------ LADIES
def _ladies(A, seeds, fanouts):
    """examples/ladies/ladies.py:7-21 of the reference."""
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
    return seeds, ret


def test_ladies_layers_at_full_size_against_the_operator_chain_on_the_cpu():
    """The layer-wise configuration (233 K nodes, 115 M edges, 512 seeds, 512
    nodes per layer) through Matrix + gs.jit.compile against the CPU operators
    chained by hand.  Weights are 0.5 or 1 (the hub rows of this multigraph
    collect more than a million edges of the sliced columns), so the row sums of
    their squares are exact in float32 in any order of summation and both sides pick
    the same 512 nodes; the normalised weights are held to 1e-5 relative of the
    same chain in float64."""
    import gsampler_amd as gs
    from gsampler_amd.utils import chung_lu_csc
    dev = torch.device("cuda:0")
    nodes, edges, K = 233_000, 115_000_000, 512
    indptr, indices = chung_lu_csc(nodes, edges, seed=1, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    w = torch.randint(1, 3, (indices.numel(),), generator=g, device=dev).float() / 2.0
    seeds = torch.randperm(nodes, generator=g, device=dev)[:512]
    A = gs.Matrix()
    A.load_graph("CSC", [indptr, indices])
    A.edata["w"] = w
    compiled = gs.jit.compile(_ladies, (A, seeds, [K, K]))
    gs.manual_seed(99)
    frontier, blocks = compiled(A, seeds, [K, K])

    h_indptr, h_indices, h_w = indptr.cpu().numpy(), indices.cpu().numpy(), w.cpu().numpy()
    h_seeds = seeds.cpu().numpy()
    for layer, blk in enumerate(blocks):
        sub_indptr, coo_col, rows, sel = orc.col_slice(h_indptr, h_indices, h_seeds)
        w_sub = h_w[sel]
        prob = orc.e_square_sum(("coo", rows, coo_col), w_sub, 2, nodes)
        exact = np.zeros(nodes)
        np.add.at(exact, rows, w_sub.astype(np.float64) ** 2)
        assert np.array_equal(prob, exact.astype(np.float32))        # the sums are exact
        picked, _ = orc.list_sample_weighted(prob, K, seed=99, call_id=layer)
        out_indptr, major, minor, select = orc.minor_slice(rows, picked, indptr=sub_indptr)
        uniq, _, out_row, out_col = orc.unique_relabel(h_seeds, picked[minor], edge_col=major)
        assert blk.num_dst_nodes() == h_seeds.size and blk.num_src_nodes() == uniq.size
        assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq)
        assert np.array_equal(blk.row.cpu().numpy(), out_row)
        assert np.array_equal(blk.col.cpu().numpy(), out_col)
        # Values: a column of these blocks sums ten thousand and more quotients
        # (a sequential float32 sum of that length, which is what the CPU
        # operators do, is itself off by more than 1e-4), so the yardstick is
        # the same chain in float64.
        q = w_sub[select].astype(np.float64) / prob[picked].astype(np.float64)[minor]
        col64 = np.zeros(h_seeds.size)
        np.add.at(col64, major, q)
        truth = q / col64[major]
        assert np.allclose(blk.edata["w"].double().cpu().numpy(), truth, rtol=1e-5, atol=0)
        # the weights of every column of a block sum to one
        sums = np.zeros(h_seeds.size)
        np.add.at(sums, out_col, blk.edata["w"].double().cpu().numpy())
        assert np.allclose(sums[np.bincount(out_col, minlength=h_seeds.size) > 0], 1.0, atol=1e-5)
        h_seeds = uniq
    assert np.array_equal(frontier.cpu().numpy(), h_seeds)
    assert blocks[1].num_edges() > 1_000_000          # the second layer really is a large one


def _ladies_with_probabilities(A, seeds, fanouts):
    """The same sampler, also handing out each layer's row probabilities and picked rows."""
    ret, probs, picks = [], [], []
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
        probs.append(prob)
        picks.append(select_index)
    return seeds, ret, probs, picks


def test_ladies_layers_at_full_size_with_unit_interval_weights_through_the_compiled_sampler():
    """The layer-wise configuration with its stated weights, U(0, 1], through Matrix +
    gs.jit.compile (the column slice is read in place: no slice is written).  Sums of up to a
    million squared weights depend on the order of addition in their last bits, so the GPU's row
    probabilities are held to 1e-5 of float64 and then handed to the CPU pick: picked rows,
    frontier and block structure are compared bit for bit, the normalised weights to 1e-5 of
    the same chain in float64."""
    import gsampler_amd as gs
    from gsampler_amd.utils import chung_lu_csc
    dev = torch.device("cuda:0")
    nodes, edges, K = 233_000, 115_000_000, 512
    indptr, indices = chung_lu_csc(nodes, edges, seed=1, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    w = 1.0 - torch.rand(edges, generator=g, device=dev, dtype=torch.float32)    # (0, 1]
    seeds = torch.randperm(nodes, generator=g, device=dev)[:512]
    A = gs.Matrix()
    A.load_graph("CSC", [indptr, indices])
    A.edata["w"] = w
    compiled = gs.jit.compile(_ladies_with_probabilities, (A, seeds, [K, K]))
    targets = [n.target for n in compiled.gm.graph.nodes if n.op == "call_method"]
    assert targets.count("_CAPI_ColRowSlicing") == 2 and "_CAPI_Slicing" not in targets
    gs.manual_seed(99)
    frontier, blocks, probs, picks = compiled(A, seeds, [K, K])

    h_indptr, h_indices, h_w = indptr.cpu().numpy(), indices.cpu().numpy(), w.cpu().numpy()
    h_seeds = seeds.cpu().numpy()
    for layer, blk in enumerate(blocks):
        sub_indptr, coo_col, rows, sel = orc.col_slice(h_indptr, h_indices, h_seeds)
        w_sub = h_w[sel]
        exact = np.zeros(nodes)
        np.add.at(exact, rows, w_sub.astype(np.float64) ** 2)
        g_prob = probs[layer].cpu().numpy()
        assert np.allclose(g_prob, exact, rtol=1e-5, atol=0)
        picked, _ = orc.list_sample_weighted(g_prob, K, seed=99, call_id=layer)
        assert np.array_equal(picks[layer].cpu().numpy(), picked)
        out_indptr, major, minor, select = orc.minor_slice(rows, picked, indptr=sub_indptr)
        uniq, _, out_row, out_col = orc.unique_relabel(h_seeds, picked[minor], edge_col=major)
        assert blk.num_dst_nodes() == h_seeds.size and blk.num_src_nodes() == uniq.size
        assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq)
        assert np.array_equal(blk.row.cpu().numpy(), out_row)
        assert np.array_equal(blk.col.cpu().numpy(), out_col)
        q = w_sub[select].astype(np.float64) / g_prob[picked].astype(np.float64)[minor]
        col64 = np.zeros(h_seeds.size)
        np.add.at(col64, major, q)
        assert np.allclose(blk.edata["w"].double().cpu().numpy(), q / col64[major], rtol=1e-5,
                           atol=0)
        h_seeds = uniq
    assert np.array_equal(frontier.cpu().numpy(), h_seeds)
    assert blocks[1].num_edges() > 1_000_000
