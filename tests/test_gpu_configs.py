"""The benchmark configurations at their stated sizes that the full-size
GraphSAGE test does not cover: the small two-layer configuration (R-MAT 100 K
nodes / 2 M edges, 1024 seeds, fan-outs 25 and 10) through Matrix eagerly and
through gs.jit.compile, and the layer-wise configuration (233 K nodes / 115 M
edges, 512 seeds, 512 nodes per layer) with its configured fp32 weights
U(0, 1]."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd import capi
from gsampler_amd.utils import chung_lu_csc, rmat_csc
from oracle import binding as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def graphsage_sampler(A, seeds, fanouts):
    """examples/graphsage/graphsage.py:7-28 of the reference."""
    input_node = seeds
    ret = []
    for K in fanouts:
        subA = A[:, seeds]
        sampleA = subA.individual_sampling(K, None, False)
        seeds = sampleA.all_nodes()
        ret.append(sampleA.to_dgl_block())
    output_node = seeds
    return input_node, output_node, ret


def test_small_two_layer_configuration_at_its_stated_size():
    nodes, edges, fanouts = 100_000, 2_000_000, [25, 10]
    indptr, indices = rmat_csc(nodes, edges, seed=1)
    assert indices.numel() == edges
    seeds = torch.randperm(nodes, generator=torch.Generator().manual_seed(3))[:1024]
    m = gs.Matrix()
    m.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    h_indptr, h_indices = indptr.numpy(), indices.numpy()
    compiled = gs.jit.compile(func=graphsage_sampler, args=(m, seeds.to(DEV), fanouts))
    for run in (graphsage_sampler, compiled):
        gs.manual_seed(7777)
        inp, outp, blocks = run(m, seeds.to(DEV), fanouts)
        assert torch.equal(inp.cpu(), seeds)
        h_seeds = seeds.numpy()
        total = 0
        for layer, (blk, K) in enumerate(zip(blocks, fanouts)):
            s, c, rows, sel = orc.sample_uniform(h_indptr, h_indices, h_seeds, K, False, 0, 7777,
                                                 layer)
            uniq, _, r, cc = orc.unique_relabel(h_seeds, rows, None, None, c)
            assert blk.num_dst == h_seeds.size and blk.num_src == uniq.size
            assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), uniq)
            assert np.array_equal(blk.row.cpu().numpy(), r)           # per-layer sampled COO,
            assert np.array_equal(blk.col.cpu().numpy(), cc)          # relabelled
            assert np.array_equal(uniq[:h_seeds.size], h_seeds)       # distinct seeds lead
            # invariants against the graph itself
            deg = np.diff(h_indptr)[h_seeds]
            assert np.array_equal(np.bincount(cc, minlength=h_seeds.size), np.minimum(deg, K))
            src, dst = uniq[r], h_seeds[cc]
            assert np.array_equal(src, h_indices[sel])
            assert np.all((sel >= h_indptr[dst]) & (sel < h_indptr[dst + 1]))
            assert np.unique(cc * edges + sel).size == sel.size      # no edge twice in a column
            total += r.size
            h_seeds = uniq
        assert np.array_equal(outp.cpu().numpy(), h_seeds)
        assert total > 40_000


def test_layerwise_configuration_with_unit_interval_weights():
    """Row probabilities are sums of up to a million squared weights; the GPU's
    sums are held to 1e-5 of float64, then the GPU's own probabilities go into the
    CPU pick, so that the picked nodes, the row slice, the frontier and the
    relabelled block are compared bit for bit, and the normalised weights to 1e-5
    of the same chain in float64."""
    nodes, edges, K = 233_000, 115_000_000, 512
    dev = torch.device(DEV)
    indptr, indices = chung_lu_csc(nodes, edges, seed=1, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    w = 1.0 - torch.rand(edges, generator=g, device=dev, dtype=torch.float32)    # (0, 1]
    assert float(w.min()) > 0.0 and float(w.max()) <= 1.0
    seeds = torch.randperm(nodes, generator=g, device=dev)[:512]
    h_indptr, h_indices, h_w = indptr.cpu().numpy(), indices.cpu().numpy(), w.cpu().numpy()
    h_seeds = seeds.cpu().numpy()
    block_edges = []
    for layer in range(2):
        # ---- GPU, through the C ABI
        sub_indptr, coo_col, rows, sel = capi.col_slice(indptr, indices, seeds)
        w_sub = w[sel]
        prob = capi.e_square_sum(("coo", rows, coo_col), w_sub, 2, nodes)
        picked, _ = capi.list_sample_weighted(prob, K, False, None, 99, layer)
        out_indptr, major, minor, select = capi.minor_slice(rows, picked, indptr=sub_indptr)
        view = ("csc", out_indptr, minor)
        w2 = capi.sddmm(view, "div", w_sub[select], prob[picked], 1, 0)
        col_sum = capi.spmm(view, "copy_rhs", "sum", None, w2, 0, seeds.numel())
        w3 = capi.sddmm(view, "div", w2, col_sum, 1, 2)
        uniq, _, out_row, out_col = capi.unique_relabel(seeds, picked[minor], edge_col=major)
        # ---- CPU
        o_indptr, o_col, o_rows, o_sel = orc.col_slice(h_indptr, h_indices, h_seeds)
        for got, want in ((sub_indptr, o_indptr), (coo_col, o_col), (rows, o_rows), (sel, o_sel)):
            assert np.array_equal(got.cpu().numpy(), want)
        ow_sub = h_w[o_sel]
        exact = np.zeros(nodes)
        np.add.at(exact, o_rows, ow_sub.astype(np.float64) ** 2)
        g_prob = prob.cpu().numpy()
        assert np.allclose(g_prob, exact, rtol=1e-5, atol=0)
        if layer == 1:
            assert exact.max() > 1e5                       # hub rows collect a million terms
        o_picked, _ = orc.list_sample_weighted(g_prob, K, seed=99, call_id=layer)
        assert np.array_equal(picked.cpu().numpy(), o_picked)
        oo_indptr, o_major, o_minor, o_select = orc.minor_slice(o_rows, o_picked, indptr=o_indptr)
        for got, want in ((out_indptr, oo_indptr), (major, o_major), (minor, o_minor),
                          (select, o_select)):
            assert np.array_equal(got.cpu().numpy(), want)
        o_uniq, _, o_row, o_colr = orc.unique_relabel(h_seeds, o_picked[o_minor], edge_col=o_major)
        for got, want in ((uniq, o_uniq), (out_row, o_row), (out_col, o_colr)):
            assert np.array_equal(got.cpu().numpy(), want)
        q = ow_sub[o_select].astype(np.float64) / g_prob[o_picked].astype(np.float64)[o_minor]
        assert np.allclose(w2.cpu().numpy(), q, rtol=1e-5, atol=0)
        col64 = np.zeros(h_seeds.size)
        np.add.at(col64, o_major, q)
        has = np.bincount(o_major, minlength=h_seeds.size) > 0
        assert np.allclose(col_sum.cpu().numpy()[has], col64[has], rtol=1e-5, atol=0)
        assert np.allclose(w3.cpu().numpy(), q / col64[o_major], rtol=1e-5, atol=0)
        block_edges.append(int(minor.numel()))
        seeds, h_seeds = uniq, o_uniq
    assert block_edges[1] > 1_000_000


def test_layerwise_row_sums_through_matrix_at_full_size():
    """`A[:, seeds].sum(key, axis=1)` of the same configuration through the
    Matrix API (the drop-in path of the row probabilities) against float64."""
    nodes, edges = 233_000, 115_000_000
    dev = torch.device(DEV)
    indptr, indices = chung_lu_csc(nodes, edges, seed=1, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    w = 1.0 - torch.rand(edges, generator=g, device=dev, dtype=torch.float32)
    seeds = torch.arange(0, 1024, 2, device=dev)      # low ids: the longest columns
    A = gs.Matrix()
    A.load_graph("CSC", [indptr, indices])
    A.edata["w"] = w
    subA = A[:, seeds]
    subA.edata["p"] = subA.edata["w"] ** 2
    prob = subA.sum("p", axis=1)
    by_col = subA.sum("w", axis=0)
    rows, cols, _ = subA.coo
    assert rows.numel() > 10_000_000
    h_w = subA.edata["w"].double().cpu().numpy()
    exact = np.bincount(rows.cpu().numpy(), weights=h_w * h_w, minlength=subA.num_rows())
    assert np.allclose(prob.cpu().numpy(), exact, rtol=1e-5, atol=0)
    exact_c = np.bincount(cols.cpu().numpy(), weights=h_w, minlength=512)
    assert np.allclose(by_col.cpu().numpy(), exact_c, rtol=1e-5, atol=0)
