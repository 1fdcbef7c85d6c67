"""The sampling algorithms of the reference's examples/ directory (FastGCN,
AS-GCN, PASS, ShaDow-GNN single and batched, GraphSAINT random-walk, KGCN),
written against this package the way a user of the reference writes them:
each must run eagerly and through gs.jit.compile with the same result, and its
blocks must only hold edges of the graph."""
import pytest
import torch
import torch.nn.functional as F

import gsampler_amd as gs
from gsampler_amd.format import _COO

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
N = 6000


@pytest.fixture(scope="module")
def world():
    from gsampler_amd.utils import rmat_csc
    indptr, indices = rmat_csc(N, 180000, seed=3)
    m = gs.Matrix()
    m.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    g = torch.Generator().manual_seed(1)
    m.edata["w"] = (torch.rand(indices.numel(), generator=g) + 0.1).to(DEV)
    m.row_ndata["deg"] = torch.bincount(indices, minlength=N).float().to(DEV) + 1.0
    feats = torch.randn(N, 16, generator=g).to(DEV)
    # dense adjacency (edge multiplicities) for "is an edge of the graph" checks
    adj = torch.zeros(N, N, dtype=torch.int32)
    col = torch.repeat_interleave(torch.arange(N), indptr[1:] - indptr[:-1])
    adj.index_put_((indices, col), torch.ones(indices.numel(), dtype=torch.int32), accumulate=True)
    return m, feats, adj.to(DEV)


def edges_exist(block, dst_ids, adj):
    """Block edges (local row -> local col) are edges of the graph."""
    src = block.srcdata["_ID"][block.row]
    dst = dst_ids[block.col]
    assert bool((adj[src, dst] > 0).all())


def same_blocks(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert torch.equal(x.row, y.row) and torch.equal(x.col, y.col)
        assert torch.equal(x.srcdata["_ID"], y.srcdata["_ID"])
        assert set(x.edata) == set(y.edata)
        for k in x.edata:
            assert torch.allclose(x.edata[k], y.edata[k], rtol=1e-5, atol=1e-7)


def both_ways(func, args, sampling_calls):
    gs.manual_seed(11)
    eager = func(*args)
    assert gs.random_state() == (11, sampling_calls)
    compiled = gs.jit.compile(func=func, args=args)
    gs.manual_seed(11)
    out = compiled(*args)
    assert gs.random_state() == (11, sampling_calls)     # no sampling call merged away
    return eager, out


def global_edges(block, dst_ids):
    """Sorted (source id, destination id) pairs of a block.  The order of the
    edges, and of the frontier behind the seeds, follows the sparse format an
    operator ran on, which eager code and the compiler may choose differently."""
    src = block.srcdata["_ID"][block.row]
    dst = dst_ids[block.col]
    return torch.unique(src * N + dst, return_counts=True)


def same_edge_sets(a, b, dst_ids):
    (ka, ca), (kb, cb) = global_edges(a, dst_ids), global_edges(b, dst_ids)
    assert torch.equal(ka, kb) and torch.equal(ca, cb)
    assert torch.equal(torch.sort(a.srcdata["_ID"])[0], torch.sort(b.srcdata["_ID"])[0])
    assert torch.equal(a.srcdata["_ID"][: dst_ids.numel()], dst_ids)
    assert torch.equal(b.srcdata["_ID"][: dst_ids.numel()], dst_ids)


# ------------------------------------------------------------------ FastGCN
def fastgcn_sampler(A, seeds, fanouts):
    blocks = []
    for K in fanouts:
        sub = A[:, seeds]
        picked, _ = sub.collective_sampling(K, sub.row_ndata["deg"], False)
        seeds = picked.all_nodes()
        blocks.append(picked.to_dgl_block())
    return seeds, blocks


def test_fastgcn(world):
    m, _, adj = world
    seeds = torch.arange(0, N, 23, device=DEV)
    (e_nodes, e_blocks), (c_nodes, c_blocks) = both_ways(
        fastgcn_sampler, (m, seeds, [400, 400]), sampling_calls=2)
    # the first layer sees the same inputs either way: same picks, same edges
    same_edge_sets(e_blocks[0], c_blocks[0], seeds)
    for nodes, blocks in ((e_nodes, e_blocks), (c_nodes, c_blocks)):
        edges_exist(blocks[0], seeds, adj)
        edges_exist(blocks[1], blocks[0].srcdata["_ID"], adj)
        assert torch.equal(nodes, blocks[1].srcdata["_ID"])
        assert blocks[0].num_dst == seeds.numel()
        for b in blocks:                     # at most K distinct rows survive a layer
            assert torch.unique(b.srcdata["_ID"][b.row]).numel() <= 400


# ------------------------------------------------------------------- AS-GCN
def asgcn_sampler(A, seeds, fanouts, features, W):
    blocks = []
    for K in fanouts:
        sub = A[:, seeds]
        sub.edata["w"] = sub.edata["w"] ** 2
        p = sub.sum("w", axis=1).sqrt()
        h_u = features[sub.rows()] @ W[:, 0]
        h_v = features[sub.cols()] @ W[:, 1]
        attention = torch.flatten((F.relu(h_u + torch.sum(h_v)) + 1) / K)
        g_u = torch.flatten(F.relu(h_u) + 1)
        q = F.normalize(p * attention * g_u, p=1.0, dim=0)
        picked, index = sub.collective_sampling(K, q, False)
        picked.edata["w"] = gs.ops.u_add_v(picked, h_u[index], h_v)
        picked.edata["w"] = (F.relu(picked.edata["w"]) + 1) / picked.num_rows()
        picked = picked.div("w", q[index], 1)
        seeds = picked.all_nodes()
        blocks.append(picked.to_dgl_block(prefetch_edata={"w"}))
    return seeds, blocks


def test_asgcn(world):
    m, feats, adj = world
    W = torch.randn(16, 2, generator=torch.Generator().manual_seed(2)).to(DEV)
    seeds = torch.arange(5, N, 31, device=DEV)
    (e_nodes, e_blocks), (c_nodes, c_blocks) = both_ways(
        asgcn_sampler, (m, seeds, [300, 300], feats, W), sampling_calls=2)
    same_edge_sets(e_blocks[0], c_blocks[0], seeds)
    assert torch.allclose(torch.sort(e_blocks[0].edata["w"])[0], torch.sort(c_blocks[0].edata["w"])[0],
                          rtol=1e-5)
    for nodes, blocks in ((e_nodes, e_blocks), (c_nodes, c_blocks)):
        edges_exist(blocks[0], seeds, adj)
        edges_exist(blocks[1], blocks[0].srcdata["_ID"], adj)
        assert torch.equal(nodes, blocks[1].srcdata["_ID"])
        assert all("w" in b.edata and bool(torch.isfinite(b.edata["w"]).all()) for b in blocks)


# --------------------------------------------------------------------- PASS
def pass_sampler(A, seeds, fanouts, features, W1, W2, W3):
    blocks = []
    for K in fanouts:
        sub = A[:, seeds]
        u_feats, v_feats = features[sub.rows()], features[sub.cols()]
        att1 = torch.sum(gs.ops.u_mul_v(sub, u_feats @ W1, v_feats @ W1, _COO), dim=1)
        att2 = torch.sum(gs.ops.u_mul_v(sub, u_feats @ W2, v_feats @ W2, _COO), dim=1)
        att3 = sub.div("w", sub.sum("w", axis=0), axis=0).edata["w"]
        att = torch.stack([att1, att2, att3], dim=1)
        att = F.relu(att @ F.softmax(W3, dim=0))
        att = att + 10e-10 * torch.ones_like(att)
        sub.edata["w"] = att
        picked = sub.individual_sampling(K, probs=att, replace=True)
        seeds = picked.all_nodes()
        blocks.append(picked.to_dgl_block(prefetch_edata={"w"}))
    return seeds, blocks


def test_pass(world):
    m, feats, adj = world
    g = torch.Generator().manual_seed(4)
    W1, W2 = torch.randn(16, 8, generator=g).to(DEV), torch.randn(16, 8, generator=g).to(DEV)
    W3 = torch.randn(3, generator=g).to(DEV)
    seeds = torch.arange(1, N, 41, device=DEV)
    (e_nodes, e_blocks), (c_nodes, c_blocks) = both_ways(
        pass_sampler, (m, seeds, [10, 5], feats, W1, W2, W3), sampling_calls=2)
    assert torch.equal(e_nodes, c_nodes)
    same_blocks(e_blocks, c_blocks)
    edges_exist(e_blocks[0], seeds, adj)
    # with replacement: exactly K picks for every seed that has a neighbour
    per_col = torch.bincount(e_blocks[0].col, minlength=seeds.numel())
    assert set(per_col.tolist()) <= {0, 10}


# --------------------------------------------------------------- ShaDow-GNN
def shadow_sampler(A, seeds, fanouts):
    for K in fanouts:
        seeds = A[:, seeds].individual_sampling(K, None, False).all_nodes()
    return seeds, A[seeds, seeds].to_dgl_block()


def batch_shadow_sampler(A, seeds, seeds_ptr, fanouts):
    for K in fanouts:
        seeds, seeds_ptr = A[:, seeds::seeds_ptr].individual_sampling(K, None, False).all_nodes()
    return A[seeds::seeds_ptr, seeds::seeds_ptr].to_dgl_block()


def test_shadowgnn(world):
    m, _, adj = world
    seeds = torch.arange(2, N, 53, device=DEV)
    (e_nodes, e_block), (c_nodes, c_block) = both_ways(shadow_sampler, (m, seeds, [10, 5]),
                                                       sampling_calls=2)
    assert torch.equal(e_nodes, c_nodes)
    same_edge_sets(e_block, c_block, e_nodes)
    # the induced subgraph on the sampled nodes: every edge among them, nothing else
    sub = adj[e_nodes][:, e_nodes]
    assert e_block.num_edges() == int(sub.sum())
    edges_exist(e_block, e_nodes, adj)


def test_batch_shadowgnn_equals_one_batch_at_a_time(world):
    m, _, adj = world
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    seeds = torch.cat([torch.arange(2, N, 211, device=DEV), torch.arange(7, N, 307, device=DEV)])
    first = torch.arange(2, N, 211).numel()
    ptr = torch.tensor([0, first, seeds.numel()], device=DEV)
    gs.manual_seed(11)
    blocks = batch_shadow_sampler(bm, seeds, ptr, [8, 4])
    compiled = gs.jit.compile(func=batch_shadow_sampler, args=(bm, seeds, ptr, [8, 4]))
    gs.manual_seed(11)
    again = compiled(bm, seeds, ptr, [8, 4])
    assert len(blocks) == 2 and len(again) == 2
    for block, other in zip(blocks, again):
        ids = block.srcdata["_ID"]
        assert torch.equal(ids, other.srcdata["_ID"])
        same_edge_sets(block, other, ids)
        assert block.num_edges() == int(adj[ids][:, ids].sum())


# ---------------------------------------------------------------- GraphSAINT
def graphsaint_sampler(A, seeds, walk_length):
    paths = A._graph._CAPI_RandomWalk(seeds, walk_length)
    nodes = paths.view(seeds.numel() * (walk_length + 1))
    nodes = torch.unique(nodes[nodes != -1], sorted=False)
    return nodes, A[nodes, nodes].to_dgl_block()


def test_graphsaint(world):
    m, _, adj = world
    seeds = torch.arange(3, N, 17, device=DEV)
    (e_nodes, e_block), (c_nodes, c_block) = both_ways(graphsaint_sampler, (m, seeds, 4),
                                                       sampling_calls=1)
    assert torch.equal(torch.sort(e_nodes)[0], torch.sort(c_nodes)[0])
    assert bool(torch.isin(seeds, e_nodes).all())
    assert e_block.num_edges() == int(adj[e_nodes][:, e_nodes].sum())
    assert c_block.num_edges() == e_block.num_edges()


# --------------------------------------------------------------------- KGCN
def kgcn_sampler(A, seeds, fanouts):
    layers = []
    for K in fanouts:
        picked = A[:, seeds].individual_sampling(K, None, True)
        seeds = picked.csc[1]
        layers.append(picked)
    return seeds, layers


def test_kgcn(world):
    m, _, adj = world
    seeds = torch.arange(9, N, 61, device=DEV)
    (e_out, e_layers), (c_out, c_layers) = both_ways(kgcn_sampler, (m, seeds, [6, 3]),
                                                     sampling_calls=2)
    assert torch.equal(e_out, c_out)
    indptr, rows, _ = e_layers[0].csc
    deg = indptr[1:] - indptr[:-1]
    assert set(deg.tolist()) <= {0, 6}                       # with replacement: K or nothing
    assert bool((adj[rows, torch.repeat_interleave(seeds, deg)] > 0).all())
    for a, b in zip(e_layers, c_layers):
        assert all(torch.equal(x, y) for x, y in zip(a.csc[:2], b.csc[:2]))


# ------------------------------------------------------------ batched LADIES
def batch_ladies_sampler(A, fanouts, seeds, seeds_ptr):
    blocks = []
    for K in fanouts:
        sub = A[:, seeds::seeds_ptr]
        sub.edata["p"] = sub.edata["w"] ** 2
        prob = sub.sum("p", axis=1)
        _, probs_ptr = sub.all_rows()
        picked, index = sub.collective_sampling(K, prob, probs_ptr, False)
        picked = picked.div("w", prob[index], axis=1)
        picked = picked.div("w", picked.sum("w", axis=0), axis=0)
        seeds, seeds_ptr = picked.all_nodes()
        blocks.append(picked.to_dgl_block(prefetch_edata={"w"}))
    return blocks


def test_batch_ladies(world):
    m, _, adj = world
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m)
    parts = [torch.arange(s, N, 97, device=DEV) for s in (0, 11, 50)]
    seeds = torch.cat(parts)
    ptr = torch.tensor([0] + list(torch.cumsum(torch.tensor([p.numel() for p in parts]), 0)),
                       device=DEV)
    K = 64
    gs.manual_seed(11)
    eager = batch_ladies_sampler(bm, [K, K], seeds, ptr)
    assert gs.random_state() == (11, 2)
    compiled = gs.jit.compile(func=batch_ladies_sampler, args=(bm, [K, K], seeds, ptr))
    gs.manual_seed(11)
    jit = compiled(bm, [K, K], seeds, ptr)
    assert gs.random_state() == (11, 2)
    for layers in (eager, jit):
        assert len(layers) == 2 and all(len(per_batch) == 3 for per_batch in layers)
        dst = parts
        for per_batch in layers:
            nxt = []
            for block, ids in zip(per_batch, dst):
                edges_exist(block, ids, adj)
                assert block.num_dst == ids.numel()
                assert torch.equal(block.srcdata["_ID"][: ids.numel()], ids)
                assert torch.unique(block.srcdata["_ID"][block.row]).numel() <= K
                # weights are normalised per destination node
                sums = torch.zeros(ids.numel(), device=DEV).index_add_(0, block.col, block.edata["w"])
                has = torch.bincount(block.col, minlength=ids.numel()) > 0
                assert torch.allclose(sums[has], torch.ones_like(sums[has]), rtol=1e-5)
                nxt.append(block.srcdata["_ID"])
            dst = nxt
    for a, b, ids in zip(eager[0], jit[0], parts):     # first layer: the same picks
        same_edge_sets(a, b, ids)


def test_compiled_with_compaction_describes_the_same_blocks(world):
    """must_compact renumbers the rows of every slice densely (the variant the
    reference's compiler may pick by timing): same edges, same data."""
    m, feats, adj = world
    seeds = torch.arange(4, N, 29, device=DEV)

    def ladies(A, seeds, fanouts):
        blocks = []
        for K in fanouts:
            sub = A[:, seeds]
            sub.edata["p"] = sub.edata["w"] ** 2
            prob = sub.sum("p", axis=1)
            picked, index = sub.collective_sampling(K, prob, False)
            picked = picked.div("w", prob[index], axis=1)
            picked = picked.div("w", picked.sum("w", axis=0), axis=0)
            seeds = picked.all_nodes()
            blocks.append(picked.to_dgl_block(prefetch_edata={"w"}))
        return seeds, blocks

    plain = gs.jit.compile(func=ladies, args=(m, seeds, [200, 200]))
    dense = gs.jit.compile(func=ladies, args=(m, seeds, [200, 200]), must_compact=True)
    gs.manual_seed(8)
    p_nodes, p_blocks = plain(m, seeds, [200, 200])
    gs.manual_seed(8)
    d_nodes, d_blocks = dense(m, seeds, [200, 200])
    for blocks in (p_blocks, d_blocks):
        edges_exist(blocks[0], seeds, adj)
        edges_exist(blocks[1], blocks[0].srcdata["_ID"], adj)
        for b in blocks:
            sums = torch.zeros(b.num_dst, device=DEV).index_add_(0, b.col, b.edata["w"])
            has = torch.bincount(b.col, minlength=b.num_dst) > 0
            assert torch.allclose(sums[has], torch.ones_like(sums[has]), rtol=1e-5)
            assert torch.unique(b.srcdata["_ID"][b.row]).numel() <= 200
    assert p_blocks[0].num_dst == d_blocks[0].num_dst == seeds.numel()
