"""Oracle format conversions and super-batch bookkeeping against closed forms
(numpy / scipy.sparse)."""
import numpy as np
import pytest
import scipy.sparse as sp

from oracle import binding as orc
from tests.conftest import random_csc


@pytest.mark.parametrize("seed", range(3))
def test_csc2coo_is_repeat_of_column_ids(seed):
    rng = np.random.default_rng(seed)
    indptr, indices = random_csc(rng, 200, 500, 30, hub_deg=3000)
    col = orc.csc2coo(indptr)
    assert np.array_equal(col, np.repeat(np.arange(200), np.diff(indptr)))
    # scipy's own conversion agrees (CSC -> COO keeps the edge order)
    m = sp.csc_matrix((np.ones(indices.size), indices, indptr), shape=(500, 200)).tocoo()
    assert np.array_equal(col, m.col)
    assert np.array_equal(indices, m.row)


def test_csc2coo_empty_columns_and_empty_matrix():
    indptr = np.array([0, 0, 3, 3, 3, 5])
    assert orc.csc2coo(indptr).tolist() == [1, 1, 1, 4, 4]
    assert orc.csc2coo(np.zeros(4, dtype=np.int64)).size == 0


@pytest.mark.parametrize("seed", range(3))
def test_sorted_to_indptr_round_trip(seed):
    rng = np.random.default_rng(10 + seed)
    num_cols = 300
    ids = np.sort(rng.integers(0, num_cols, size=5000))
    indptr = orc.sorted_to_indptr(ids, num_cols)
    assert np.array_equal(indptr, np.searchsorted(ids, np.arange(num_cols + 1), side="left"))
    assert np.array_equal(orc.csc2coo(indptr), ids)       # inverse of csc2coo
    assert orc.sorted_to_indptr(np.empty(0, dtype=np.int64), 3).tolist() == [0, 0, 0, 0]


def test_coo_to_csc_matches_scipy():
    """COO -> CSC as the host layer does it: stable sort by column, then indptr."""
    rng = np.random.default_rng(5)
    pairs = rng.permutation(70 * 40)[:2000]          # distinct (row, col) pairs
    row, col = pairs // 40, pairs % 40
    perm = np.argsort(col, kind="stable")
    indptr = orc.sorted_to_indptr(col[perm], 40)
    m = sp.coo_matrix((np.arange(2000) + 1.0, (row, col)), shape=(70, 40)).tocsc()
    assert np.array_equal(indptr, m.indptr)
    for c in range(40):
        mine = sorted(zip(row[perm][indptr[c]:indptr[c + 1]], perm[indptr[c]:indptr[c + 1]] + 1))
        theirs = sorted(zip(m.indices[m.indptr[c]:m.indptr[c + 1]],
                            m.data[m.indptr[c]:m.indptr[c + 1]].astype(np.int64)))
        assert mine == theirs


def test_decode_batch_ids():
    rng = np.random.default_rng(6)
    stride = 1000
    orig = rng.integers(0, stride, size=500)
    batch = rng.integers(0, 17, size=500)
    got_orig, got_batch = orc.decode_batch_ids(orig + batch * stride, stride)
    assert np.array_equal(got_orig, orig) and np.array_equal(got_batch, batch)


def test_split_indptr_rebases_every_batch():
    indptr = np.array([0, 2, 5, 5, 9, 12, 12, 20])
    offset = np.array([0, 2, 2, 5, 7])              # columns per batch: 2, 0, 3, 2
    out = orc.split_indptr(indptr, offset)
    want = np.concatenate([indptr[a:b + 1] - indptr[a] for a, b in zip(offset[:-1], offset[1:])])
    assert np.array_equal(out, want)
    assert out.tolist() == [0, 2, 5, 0, 0, 0, 4, 7, 0, 0, 8]


def test_coo_sort_is_a_stable_argsort_and_builds_the_csc():
    rng = np.random.default_rng(11)
    C, E = 300, 20000
    col = rng.integers(0, C, size=E)
    row = rng.integers(0, 500, size=E)
    sorted_col, perm = orc.coo_sort(col)
    want = np.argsort(col, kind="stable")
    assert np.array_equal(perm, want) and np.array_equal(sorted_col, col[want])
    indptr, indices, eids = orc.coo_to_csc(row, col, C)
    assert np.array_equal(np.diff(indptr), np.bincount(col, minlength=C))
    for c in (0, 17, C - 1):                              # column contents in edge order
        assert np.array_equal(indices[indptr[c]:indptr[c + 1]], row[col == c])
    assert np.array_equal(eids, want)
