"""Oracle column slicing / counts against NumPy closed forms and the
reference's own known-answer cases."""
import numpy as np
import pytest

from oracle import binding as orc
from tests import numpy_ref as ref
from tests.conftest import golden, random_csc


def test_reference_colwise_slicing_known_answer():
    # tests/test_colwise_slicing.cc:7-21 of the reference
    fx = golden()["colwise_slicing"]
    indptr, indices = np.array(fx["indptr"]), np.array(fx["indices"])
    sub_indptr, coo_col, sub_indices, sel = orc.col_slice(indptr, indices, fx["column_ids"])
    assert np.array_equal(sub_indptr, fx["sub_indptr"])
    assert np.array_equal(sub_indices, fx["sub_indices"])
    assert np.array_equal(sel, np.arange(15))
    assert np.array_equal(coo_col, np.repeat(np.arange(3), 5))


@pytest.mark.parametrize("seed", range(4))
def test_col_slice_matches_numpy(seed):
    rng = np.random.default_rng(seed)
    indptr, indices = random_csc(rng, 300, 1000, 40, hub_deg=5000)
    cols = rng.integers(0, 300, size=257)  # repeats allowed
    got = orc.col_slice(indptr, indices, cols)
    want = ref.col_slice(indptr, indices, cols)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_col_slice_empty_and_out_of_range():
    indptr = np.array([0, 2, 2, 5])
    indices = np.array([7, 8, 1, 2, 3])
    s, c, i, sel = orc.col_slice(indptr, indices, np.empty(0, dtype=np.int64))
    assert s.tolist() == [0] and i.size == 0
    # ids outside [0, num_cols) behave as empty columns
    s, c, i, sel = orc.col_slice(indptr, indices, [5, 2, -1, 1])
    assert s.tolist() == [0, 0, 3, 3, 3]
    assert i.tolist() == [1, 2, 3] and c.tolist() == [1, 1, 1]


def test_batched_slice_encodes_rows():
    # src/cuda/batch/slicing.cu:25-27 : row id + batch * num_rows
    rng = np.random.default_rng(0)
    indptr, indices = random_csc(rng, 50, 77, 9)
    cols = rng.integers(0, 50, size=30)
    ptr = np.array([0, 7, 7, 20, 30])
    plain = orc.col_slice(indptr, indices, cols)
    enc = orc.col_slice(indptr, indices, cols, batch_ptr=ptr, encode_stride=77)
    batch_of_edge = np.searchsorted(ptr, plain[1], side="right") - 1
    assert np.array_equal(enc[2], plain[2] + 77 * batch_of_edge)
    assert np.array_equal(enc[3], plain[3]) and np.array_equal(enc[0], plain[0])


@pytest.mark.parametrize("fanout,replace", [(3, False), (3, True), (0, False), (100, True)])
def test_col_count_rule(fanout, replace):
    # src/cuda/sampling.cu:112-123
    rng = np.random.default_rng(3)
    indptr, _ = random_csc(rng, 200, 10, 8)
    cols = rng.integers(0, 200, size=99)
    deg = indptr[cols + 1] - indptr[cols]
    cnt = np.where(deg == 0, 0, fanout) if replace else np.minimum(deg, fanout)
    want = np.concatenate([[0], np.cumsum(cnt)])
    assert np.array_equal(orc.col_count(indptr, cols, fanout, replace), want)
    # column_ids = None means the matrix's own columns
    deg = np.diff(indptr)
    cnt = np.where(deg == 0, 0, fanout) if replace else np.minimum(deg, fanout)
    assert np.array_equal(orc.col_count(indptr, None, fanout, replace),
                          np.concatenate([[0], np.cumsum(cnt)]))


def test_exclusive_scan():
    rng = np.random.default_rng(1)
    x = rng.integers(0, 1000, size=5000)
    assert np.array_equal(orc.exclusive_scan(x), np.cumsum(x) - x)
