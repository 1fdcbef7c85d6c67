"""Oracle row slicing (across the compressed axis) and COO slicing."""
import numpy as np

from oracle import binding as orc
from tests.conftest import golden, random_csc


def test_reference_rowwise_slicing_known_answer():
    # tests/test_rowwise_slicing.cc:7-24 : CSR-style slicing of id 5 keeps 2 edges;
    # the reference asserts the kept *column* ids are [10, 11] -- the segments
    # that hold the two edges whose id is 5.
    fx = golden()["rowwise_slicing"]
    indptr, indices = np.array(fx["indptr"]), np.array(fx["indices"])
    out_indptr, major, minor, select = orc.minor_slice(indices, fx["row_ids"], indptr=indptr)
    assert major.tolist() == fx["kept_major_ids"]
    assert minor.tolist() == [0, 0] and select.tolist() == [0, 2]
    assert out_indptr.tolist() == [0] * 11 + [1, 2]


def test_matches_numpy_closed_form():
    rng = np.random.default_rng(0)
    indptr, indices = random_csc(rng, 200, 300, 40, hub_deg=3000)
    col = np.repeat(np.arange(200), np.diff(indptr))
    picked = rng.permutation(300)[:50]
    out_indptr, major, minor, select = orc.minor_slice(indices, picked, indptr=indptr)
    mask = np.isin(indices, picked)
    pos = {int(v): i for i, v in enumerate(picked)}
    assert np.array_equal(select, np.nonzero(mask)[0])
    assert np.array_equal(major, col[mask])
    assert np.array_equal(minor, [pos[int(v)] for v in indices[mask]])
    assert np.array_equal(out_indptr,
                          np.concatenate([[0], np.cumsum(np.bincount(col[mask], minlength=200))]))
    # coordinate form: the other axis is carried through
    _, other, m2, s2 = orc.minor_slice(indices, picked, edge_major=col * 7)
    assert np.array_equal(other, col[mask] * 7) and np.array_equal(m2, minor)


def test_repeated_and_absent_ids():
    indices = np.array([4, 9, 4, 7, 1])
    picked = np.array([9, 4, 9, 100])       # 9 twice: smallest position wins; 100 absent
    out_indptr, major, minor, select = orc.minor_slice(indices, picked,
                                                       indptr=np.array([0, 2, 2, 5]))
    assert minor.tolist() == [1, 0, 1] and select.tolist() == [0, 1, 2]
    assert major.tolist() == [0, 0, 2] and out_indptr.tolist() == [0, 2, 2, 3]
    e = np.empty(0, dtype=np.int64)
    out_indptr, major, minor, select = orc.minor_slice(indices, e, indptr=np.array([0, 2, 2, 5]))
    assert out_indptr.tolist() == [0, 0, 0, 0] and minor.size == 0
