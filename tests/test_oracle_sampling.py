"""Oracle uniform sampling: the reference's own invariant tests, structural
invariants, and distribution checks chosen so that an off-by-one in a draw
range or a wrong slot rule fails (a non-uniform subset distribution)."""
import itertools

import numpy as np
import pytest
from scipy import stats

from oracle import binding as orc
from tests.conftest import golden, random_csc

ALGOS = {"auto": 0, "reservoir": 1, "floyd": 2}


def _ref_graph():
    fx = golden()["colwise_sampling"]
    return np.array(fx["indptr"]), np.array(fx["indices"])


def test_reference_sampling_test1_copy_path():
    # tests/test_colwise_sampling.cc:7-23 : K=6 > deg=5, no replace -> identity
    indptr, indices = _ref_graph()
    for algo in ALGOS.values():
        s, c, i, sel = orc.sample_uniform(indptr, indices, None, 6, False, algo)
        assert np.array_equal(s, indptr) and np.array_equal(i, indices)
        assert np.array_equal(sel, np.arange(100))


@pytest.mark.parametrize("fanout", [6, 4])
def test_reference_sampling_test2_3_replace(fanout):
    # tests/test_colwise_sampling.cc:25-60
    indptr, indices = _ref_graph()
    s, c, i, sel = orc.sample_uniform(indptr, indices, None, fanout, True)
    assert np.array_equal(s, np.arange(21) * fanout)
    assert i.size == 20 * fanout and not np.array_equal(i, indices[:i.size])
    assert np.unique(i).size <= 100
    # every pick comes from its own column
    assert np.array_equal(sel // 5, np.repeat(np.arange(20), fanout))


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
@pytest.mark.parametrize("fanout", [1, 5, 16, 17, 64])
def test_invariants(algo, fanout):
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 400, 10**6, 60, hub_deg=3000)
    cols = rng.integers(0, 400, size=333)
    s, c, i, sel = orc.sample_uniform(indptr, indices, cols, fanout, False,
                                      ALGOS[algo], seed=5, call_id=2)
    deg = indptr[cols + 1] - indptr[cols]
    assert np.array_equal(np.diff(s), np.minimum(deg, fanout))      # count
    assert np.array_equal(i, indices[sel])                           # edge exists
    assert np.array_equal(c, np.repeat(np.arange(cols.size), np.diff(s)))
    lo, hi = indptr[cols][c], indptr[cols + 1][c]
    assert np.all((sel >= lo) & (sel < hi))                          # own column
    for k in range(cols.size):                                       # no duplicates
        seg = sel[s[k]:s[k + 1]]
        assert np.unique(seg).size == seg.size
        if deg[k] <= fanout:                                         # copy in order
            assert np.array_equal(seg, np.arange(indptr[cols[k]], indptr[cols[k] + 1]))


def test_reservoir_above_64_is_auto_choice():
    indptr = np.array([0, 500]); indices = np.arange(500)
    a = orc.sample_uniform(indptr, indices, None, 100, False, ALGOS["auto"])
    r = orc.sample_uniform(indptr, indices, None, 100, False, ALGOS["reservoir"])
    assert np.array_equal(a[3], r[3])
    a = orc.sample_uniform(indptr, indices, None, 10, False, ALGOS["auto"])
    f = orc.sample_uniform(indptr, indices, None, 10, False, ALGOS["floyd"])
    assert np.array_equal(a[3], f[3])


def test_determinism_and_stream_separation():
    rng = np.random.default_rng(0)
    indptr, indices = random_csc(rng, 100, 1000, 50)
    cols = np.arange(100)
    a = orc.sample_uniform(indptr, indices, cols, 5, seed=1, call_id=0)
    b = orc.sample_uniform(indptr, indices, cols, 5, seed=1, call_id=0)
    c = orc.sample_uniform(indptr, indices, cols, 5, seed=1, call_id=1)
    d = orc.sample_uniform(indptr, indices, cols, 5, seed=2, call_id=0)
    assert np.array_equal(a[3], b[3])
    assert not np.array_equal(a[3], c[3]) and not np.array_equal(a[3], d[3])


def test_pick_depends_on_position_not_on_batching():
    """A column's picks depend only on its position in the seed array, so a
    super-batch equals the concatenation of nothing but itself: slicing the
    seed array differently must not change position k's picks."""
    rng = np.random.default_rng(0)
    indptr, indices = random_csc(rng, 100, 1000, 50, empty_frac=0)
    cols = rng.integers(0, 100, size=64)
    full = orc.sample_uniform(indptr, indices, cols, 4)
    # same columns, but all moved to column 7's data except position 10
    cols2 = cols.copy(); cols2[:] = cols[10]
    part = orc.sample_uniform(indptr, indices, cols2, 4)
    seg_full = full[3][full[0][10]:full[0][11]]
    seg_part = part[3][part[0][10]:part[0][11]]
    assert np.array_equal(seg_full, seg_part)


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
@pytest.mark.parametrize("deg,fanout", [(5, 2), (6, 3), (7, 1), (4, 3)])
def test_subsets_are_uniform(algo, deg, fanout):
    """Brute force on a tiny column: all C(deg, K) subsets equally likely.
    One column repeated n times = n independent samples (position differs)."""
    n = 20000
    indptr = np.array([0, deg]); indices = np.arange(deg)
    cols = np.zeros(n, dtype=np.int64)
    s, c, i, sel = orc.sample_uniform(indptr, indices, cols, fanout, False, ALGOS[algo])
    picks = np.sort(sel.reshape(n, fanout), axis=1)
    subsets = list(itertools.combinations(range(deg), fanout))
    index = {t: k for k, t in enumerate(subsets)}
    counts = np.zeros(len(subsets))
    for row in picks:
        counts[index[tuple(row)]] += 1
    p = stats.chisquare(counts).pvalue
    assert p > 0.01, (p, counts)


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
def test_inclusion_frequencies_chi_square(algo):
    """Per-edge inclusion counts against K/deg on a mid-size column."""
    deg, fanout, n = 53, 15, 6000
    indptr = np.array([0, deg]); indices = np.arange(deg)
    s, c, i, sel = orc.sample_uniform(indptr, indices, np.zeros(n, dtype=np.int64),
                                      fanout, False, ALGOS[algo], seed=11)
    counts = np.bincount(sel, minlength=deg).astype(float)
    # inclusion indicators are negatively correlated; the statistic below is
    # (deg-1)/deg-scaled chi-square with deg-1 dof for fixed-size designs
    expected = n * fanout / deg
    stat = np.sum((counts - expected) ** 2 / expected) / (1 - fanout / deg)
    p = stats.chi2.sf(stat, deg - 1)
    assert p > 0.01, p


def test_replace_positions_are_uniform():
    deg, fanout, n = 7, 3, 20000
    indptr = np.array([0, deg]); indices = np.arange(deg)
    s, c, i, sel = orc.sample_uniform(indptr, indices, np.zeros(n, dtype=np.int64),
                                      fanout, True)
    assert np.all(np.diff(s) == fanout)
    p = stats.chisquare(np.bincount(sel, minlength=deg)).pvalue
    assert p > 0.01, p
