"""Walks, per-column sort, Compact and the batched column+row slice on the GPU."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd import capi
from gsampler_amd.utils import chung_lu_csc
from oracle import binding as orc
from tests.conftest import random_csc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int64), device=DEV)


@pytest.fixture(scope="module")
def graph():
    indptr, indices = chung_lu_csc(30000, 600000, seed=3, sort_rows=True)
    return indptr.numpy(), indices.numpy()


def test_random_walk_parity(graph):
    indptr, indices = graph
    seeds = np.random.default_rng(0).integers(0, 30000, size=5000)
    got = capi.random_walk(T(indptr), T(indices), T(seeds), 20, call_id=3)
    assert np.array_equal(got.cpu().numpy(), orc.random_walk(indptr, indices, seeds, 20, call_id=3))


@pytest.mark.parametrize("p,q", [(2.0, 0.5), (0.25, 4.0), (1.0, 1.0)])
def test_node2vec_parity(graph, p, q):
    indptr, indices = graph
    seeds = np.random.default_rng(1).integers(0, 30000, size=5000)
    got = capi.node2vec(T(indptr), T(indices), T(seeds), 30, p, q, call_id=1)
    assert np.array_equal(got.cpu().numpy(),
                          orc.node2vec(indptr, indices, seeds, 30, p, q, call_id=1))


def test_reference_dag_fixture_through_the_api():
    # tests/test_random_walk.cc:27-60, tests/test_node2vec.cc:27-60
    indptr, indices = T([0, 0, 1, 2, 3, 5]), T([0, 1, 1, 2, 3])
    A = gs.Graph(5, 5)
    A._CAPI_LoadCSC(indptr, indices)
    seeds = T([4, 2, 3, 1])
    for out in (A._CAPI_RandomWalk(seeds, 3), A._CAPI_Node2Vec(seeds, 3, 2.0, 0.5)):
        assert tuple(out.shape) == (4, 4)
        path = out.reshape(-1, 4).cpu().numpy()      # the reference's own reshape
        assert path[0].tolist() == [4, 2, 3, 1]
        assert path[:, 3].tolist() == [1, 0, -1, -1] and path[:, 1].tolist() == [2, 1, 0, -1]
        assert path[:, 0][1] in (2, 3) and path[:, 0][2] == 1 and path[:, 0][3] == 0


def test_sort_csc_indices_and_matrix_walks(graph):
    rng = np.random.default_rng(2)
    indptr, indices = random_csc(rng, 2000, 2000, 50, hub_deg=7000)
    indices[0] = 1999
    want = orc.segment_sort(indptr, indices)
    # without a key range: segmented sort over all bits; with one: column and
    # row id sorted as one word (2000 and 2^40 rows: 22 and 51 bits; 2^60: back
    # to the segmented sort, the word would not fit)
    for bound in (0, 2000, 1 << 40, 1 << 60):
        assert np.array_equal(capi.segment_sort(T(indptr), T(indices), bound).cpu().numpy(), want)
    big = indices.copy()
    big[::3] += (1 << 39)                                   # ids that need the wide key range
    assert np.array_equal(capi.segment_sort(T(indptr), T(big), 1 << 40).cpu().numpy(),
                          orc.segment_sort(indptr, big))
    empty = capi.segment_sort(T(np.zeros(5)), T(np.zeros(0)), 10)
    assert empty.numel() == 0
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    with pytest.raises(RuntimeError, match="SortCSCIndices"):
        m.node2vec(T(rng.integers(0, 2000, size=5)), 3, 2.0, 0.5)     # unsorted columns
    m._graph._CAPI_SortCSCIndices()
    srt = orc.segment_sort(indptr, indices)
    assert np.array_equal(m.csc[1].cpu().numpy(), srt)
    seeds = rng.integers(0, 2000, size=300)
    gs.manual_seed(5)
    tr = m.node2vec(T(seeds), 10, 2.0, 0.5)
    assert np.array_equal(tr.reshape(-1, 300).cpu().numpy(),
                          orc.node2vec(indptr, srt, seeds, 10, 2.0, 0.5, seed=5, call_id=0))
    tr = m.random_walk(T(seeds), 10)
    assert np.array_equal(tr.reshape(-1, 300).cpu().numpy(),
                          orc.random_walk(indptr, srt, seeds, 10, seed=5, call_id=1))


def test_compact_rows_and_columns():
    rng = np.random.default_rng(4)
    indptr, indices = random_csc(rng, 300, 5000, 20)
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    sub = m[:, T(np.arange(0, 300, 3))]
    rows_before = sub.coo[0].cpu().numpy()
    sub.compact(0)
    kept = sub.row_ndata["_ID"].cpu().numpy()
    assert np.array_equal(kept, np.unique(rows_before))
    assert sub.num_rows() == kept.size
    assert np.array_equal(kept[sub.coo[0].cpu().numpy()], rows_before)
    # all_nodes / to_dgl_block map the compacted rows back to global ids
    nodes = sub.all_nodes().cpu().numpy()
    want = orc.unique_relabel(np.arange(0, 300, 3), rows_before)[0]
    assert np.array_equal(nodes, want)
    blk = sub.to_dgl_block()
    assert np.array_equal(blk.srcdata["_ID"].cpu().numpy(), want)
    # compact=True matrices compact after every slice
    mc = gs.Matrix(m._graph, compact=True)
    s2 = mc[:, T(np.arange(0, 300, 3))]
    assert s2.num_rows() == kept.size and "_ID" in s2.row_ndata


def test_batch_col_row_slicing():
    rng = np.random.default_rng(5)
    indptr, indices = random_csc(rng, 400, 300, 40)
    indices[0] = 299
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    w = torch.as_tensor(rng.random(indices.size).astype(np.float32), device=DEV)
    m.edata["w"] = w
    bm = gs.BatchMatrix()
    bm.load_from_matrix(m, False)
    col_ptr, row_ptr = np.array([0, 30, 30, 80]), np.array([0, 50, 60, 160])
    cols = rng.integers(0, 400, size=80)
    rows = np.concatenate([rng.permutation(300)[:50], rng.permutation(300)[:10],
                           rng.permutation(300)[:100]])
    sub = bm[T(rows)::T(row_ptr), T(cols)::T(col_ptr)]
    ci, cx, _ = sub.csc
    ci, cx = ci.cpu().numpy(), cx.cpu().numpy()
    got_w = sub.edata["w"].cpu().numpy()
    k = 0
    for b in range(3):
        rpos = {int(v): row_ptr[b] + i for i, v in enumerate(rows[row_ptr[b]:row_ptr[b + 1]])}
        for j in range(col_ptr[b], col_ptr[b + 1]):
            c = cols[j]
            want = [(rpos[int(r)], float(w[e])) for e, r in
                    zip(range(indptr[c], indptr[c + 1]), indices[indptr[c]:indptr[c + 1]])
                    if int(r) in rpos]
            got = list(zip(cx[ci[j]:ci[j + 1]].tolist(), got_w[ci[j]:ci[j + 1]].tolist()))
            assert got == want
            k += len(want)
    assert k == cx.size and sub.num_rows() == 160 and sub.num_cols() == 80


def test_sampling_after_a_column_sort_reads_the_sorted_row_ids():
    """From 2^20 edges on the uniform sampler reads an int32 copy of the row
    ids; a sort of the columns replaces the array the copy was made from."""
    n = 60000
    indptr, indices = chung_lu_csc(n, 1300000, seed=9, sort_rows=False)
    indptr, indices = indptr.numpy(), indices.numpy()
    assert indices.size >= 1 << 20
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    seeds = np.random.default_rng(3).integers(0, n, size=3000)
    gs.manual_seed(4)
    CSC = 2
    sub, _ = m._graph._CAPI_SlicingSampling(1, T(seeds), 5, False, CSC, CSC)   # fused: reads m's own arrays
    want = orc.sample_uniform(indptr, indices, seeds, 5, False, 0, 4, 0)
    assert np.array_equal(sub._CAPI_GetCSCIndices().cpu().numpy(), want[2])
    m._graph._CAPI_SortCSCIndices()
    srt = orc.segment_sort(indptr, indices)
    assert not np.array_equal(srt, indices)
    sub, _ = m._graph._CAPI_SlicingSampling(1, T(seeds), 5, False, CSC, CSC)
    want = orc.sample_uniform(indptr, srt, seeds, 5, False, 0, 4, 1)
    assert np.array_equal(sub._CAPI_GetCSCIndices().cpu().numpy(), want[2])
