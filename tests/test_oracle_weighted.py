"""Oracle weighted sampling: key arithmetic against math.log2, A-Res against
the exact successive-sampling probabilities (brute force on tiny inputs),
integer-CDF picks against the weights, structural rules of the reference."""
import itertools
import math

import numpy as np
import pytest
from scipy import stats

from oracle import binding as orc


def test_neg_log2_matches_libm():
    rng = np.random.default_rng(0)
    for r in rng.integers(0, 2**64, size=2000, dtype=np.uint64):
        v = (int(r) >> 12) + 1
        want = 52 - math.log2(v)
        assert abs(orc.neg_log2_unit(int(r)) - want) <= 1e-13 * max(1.0, want)
    assert orc.neg_log2_unit(2**64 - 1) == 0.0           # u = 1
    assert orc.neg_log2_unit(0) == 52.0                  # smallest u = 2^-52
    assert orc.neg_log2_unit(((2**51 - 1) << 12)) == 1.0  # u = 1/2 exactly
    # monotone: a larger draw never gives a larger exponential clock
    xs = np.sort(rng.integers(0, 2**64, size=500, dtype=np.uint64))
    ks = [orc.neg_log2_unit(int(x)) for x in xs]
    assert all(a >= b for a, b in zip(ks, ks[1:]))


def test_key_definition():
    w = 0.37
    words = orc.stream_words(5, 2, 11, 3)
    r64 = (int(words[1]) << 32) | int(words[0])
    assert orc.weighted_key(5, 2, 11, 3, w) == pytest.approx(
        orc.neg_log2_unit(r64) / float(np.float32(w)), rel=1e-15)
    assert math.isinf(orc.weighted_key(5, 2, 11, 3, 0.0))
    assert math.isinf(orc.weighted_key(5, 2, 11, 3, -1.0))
    assert math.isinf(orc.weighted_key(5, 2, 11, 3, float("nan")))


def _successive_probs(w, k):
    """P(ordered k-tuple) under successive weighted sampling without replacement."""
    out = {}
    for tup in itertools.permutations(range(len(w)), k):
        p, rest = 1.0, sum(w)
        for i in tup:
            p *= w[i] / rest
            rest -= w[i]
        out[tup] = p
    return out


@pytest.mark.parametrize("w,k", [([1, 2, 3, 4], 2), ([5, 1, 1, 1, 2], 3), ([1, 1, 1], 1)])
def test_list_sampling_is_successive_weighted_sampling(w, k):
    n_trials = 30000
    probs = np.array(w, dtype=np.float32)
    counts = {}
    for t in range(n_trials):
        idx, _ = orc.list_sample_weighted(probs, k, call_id=t)
        counts[tuple(idx.tolist())] = counts.get(tuple(idx.tolist()), 0) + 1
    want = _successive_probs(w, k)
    assert set(counts) <= set(want)
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n_trials
    assert stats.chisquare(obs, exp).pvalue > 0.01


def test_column_sampling_is_successive_weighted_sampling():
    w, k, n = [3, 1, 2, 2, 1], 2, 30000
    indptr = np.array([0, len(w)]); indices = np.arange(len(w)) + 100
    probs = np.array(w, dtype=np.float32)
    s, c, rows, sel = orc.sample_weighted(indptr, indices, probs, np.zeros(n, dtype=np.int64), k)
    assert np.array_equal(rows, indices[sel])
    want = _successive_probs(w, k)
    picks = sel.reshape(n, k)
    counts = {}
    for row in picks:
        counts[tuple(row.tolist())] = counts.get(tuple(row.tolist()), 0) + 1
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n
    assert stats.chisquare(obs, exp).pvalue > 0.01


def test_structural_rules():
    probs = np.array([0.5, 0.0, 2.0, 0.0, 1.0], dtype=np.float32)
    # N <= K without replacement: arange(N)  (src/cuda/list_sampling_probs.cu:16-19)
    idx, rng_ = orc.list_sample_weighted(probs, 5)
    assert idx.tolist() == [0, 1, 2, 3, 4] and rng_.tolist() == [0, 5]
    # zero weights are never chosen while positive ones remain ...
    for t in range(200):
        idx, _ = orc.list_sample_weighted(probs, 3, call_id=t)
        assert sorted(idx.tolist()) == [0, 2, 4]
    # ... and come last, in index order, when they must be used
    idx, _ = orc.list_sample_weighted(probs, 4, call_id=1)
    assert sorted(idx[:3].tolist()) == [0, 2, 4] and idx[3] == 1
    # per column: deg <= K copies the column, zero weights included
    indptr = np.array([0, 5, 5, 7]); indices = np.arange(7)
    p7 = np.array([0.5, 0, 2, 0, 1, 0, 0], dtype=np.float32)
    s, c, rows, sel = orc.sample_weighted(indptr, indices, p7, None, 5)
    assert s.tolist() == [0, 5, 5, 7] and sel.tolist() == list(range(7))
    s, c, rows, sel = orc.sample_weighted(indptr, indices, p7, None, 2)
    assert s.tolist() == [0, 2, 2, 4] and set(sel[:2]) <= {0, 2, 4} and sel[2:].tolist() == [5, 6]


def test_batched_list_sampling_segments_are_independent():
    rng = np.random.default_rng(1)
    probs = rng.random(1000, dtype=np.float32)
    ranges = np.array([0, 100, 100, 105, 600, 1000])
    idx, out_range = orc.list_sample_weighted(probs, 50, range_=ranges)
    assert out_range.tolist() == [0, 50, 50, 55, 105, 155]
    for b in range(5):
        seg = idx[out_range[b]:out_range[b + 1]]
        assert np.all((seg >= ranges[b]) & (seg < ranges[b + 1]))
        assert np.unique(seg).size == seg.size
        # a segment's picks do not depend on the other segments: same stream positions
        alone, _ = orc.list_sample_weighted(
            np.concatenate([np.zeros(ranges[b], dtype=np.float32), probs[ranges[b]:ranges[b + 1]]]),
            50, range_=np.array([0, ranges[b], ranges[b + 1]]))
        assert np.array_equal(alone[min(50, ranges[b]):], seg)
    assert idx[50:55].tolist() == [100, 101, 102, 103, 104]   # n_b <= K keeps its order


def test_replace_frequencies_follow_weights():
    w = np.array([1, 0, 3, 6], dtype=np.float32)
    idx, out_range = orc.list_sample_weighted(w, 40000, replace=True)
    counts = np.bincount(idx, minlength=4)
    assert counts[1] == 0
    assert stats.chisquare(counts[[0, 2, 3]], 40000 * np.array([0.1, 0.3, 0.6])).pvalue > 0.01
    indptr = np.array([0, 4]); indices = np.arange(4)
    s, c, rows, sel = orc.sample_weighted(indptr, indices, w, np.zeros(2000, dtype=np.int64), 20,
                                          replace=True)
    counts = np.bincount(sel, minlength=4)
    assert counts[1] == 0 and np.all(np.diff(s) == 20)
    assert stats.chisquare(counts[[0, 2, 3]], 40000 * np.array([0.1, 0.3, 0.6])).pvalue > 0.01
    # all weights non-positive: the last item, like the reference's all-zero CDF
    s, c, rows, sel = orc.sample_weighted(indptr, indices, np.zeros(4, dtype=np.float32), None, 3,
                                          replace=True)
    assert sel.tolist() == [3, 3, 3]


def test_uniform_list_sampling():
    assert orc.list_sample_uniform(5, 9).tolist() == [0, 1, 2, 3, 4]
    for picks in (7, 100):       # Floyd and reservoir (picks > 64)
        out = orc.list_sample_uniform(1000, picks, call_id=3)
        assert out.size == picks and np.unique(out).size == picks and out.max() < 1000
    out = orc.list_sample_uniform(10, 500, replace=True)
    assert out.size == 500 and out.max() < 10
    counts = np.zeros(12)
    for t in range(6000):
        counts[orc.list_sample_uniform(12, 4, call_id=t)] += 1
    assert stats.chisquare(counts).pvalue > 0.001


# ------------------------------------------------ sampling through a persistent CDF
def test_weight_cdf_is_a_quantised_prefix_sum():
    rng = np.random.default_rng(3)
    deg = np.array([5, 0, 300, 1, 4, 0, 7])
    indptr = np.concatenate([[0], np.cumsum(deg)])
    w = rng.lognormal(size=int(deg.sum())).astype(np.float32)
    w[indptr[4]:indptr[5]] = [0.0, -1.0, 0.0, 0.0]      # a column without positive weights
    w[indptr[6] + 2] = 0.0
    cdf = orc.weight_cdf(indptr, w)
    q = np.diff(cdf)
    assert cdf[0] == 0 and np.all(q >= 0)
    for c in range(deg.size):
        lo, hi = indptr[c], indptr[c + 1]
        wc, qc = w[lo:hi].astype(np.float64), q[lo:hi]
        if hi == lo:
            continue
        if wc.max() <= 0:
            assert np.all(qc == 0)
            continue
        # the maximum maps to 2^31 (give or take a unit), everything else in proportion
        assert abs(int(qc[wc.argmax()]) - 2**31) <= 1
        assert np.all(qc[wc <= 0] == 0)
        want = np.where(wc > 0, wc / wc.max() * 2**31, 0)
        assert np.all(np.abs(qc - want) <= 1.0 + want * 2**-40)


@pytest.mark.parametrize("w,k", [([3, 1, 2, 2, 1], 2), ([5, 1, 0, 1, 2, 1], 3), ([1, 1, 1, 1], 3),
                                 ([1000, 1, 2, 3, 2], 3)])   # mass on one item: the sequential phase
def test_cdf_column_sampling_is_successive_weighted_sampling(w, k):
    """Ordered k-tuples drawn through the CDF against the exact law of successive
    weighted sampling without replacement (zero weights have probability 0)."""
    n = 40000
    indptr = np.array([0, len(w)]); indices = np.arange(len(w)) + 100
    probs = np.array(w, dtype=np.float32)
    cdf = orc.weight_cdf(indptr, probs)
    s, c, rows, sel = orc.sample_weighted(indptr, indices, None, np.zeros(n, dtype=np.int64), k,
                                          cdf=cdf)
    assert np.array_equal(rows, indices[sel]) and np.array_equal(s, np.arange(n + 1) * k)
    want = {t: p for t, p in _successive_probs(w, k).items() if p > 0}
    counts = {}
    for row in sel.reshape(n, k):
        counts[tuple(row.tolist())] = counts.get(tuple(row.tolist()), 0) + 1
    assert set(counts) <= set(want)
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n
    assert stats.chisquare(obs, exp).pvalue > 0.01


def test_cdf_sampling_structural_rules():
    indptr = np.array([0, 6, 6, 9, 14]); indices = np.arange(14)
    probs = np.array([0, 5, 0, 0, 0, 0,   1, 1, 1,   0, 0, 0, 0, 0], dtype=np.float32)
    cdf = orc.weight_cdf(indptr, probs)
    s, c, rows, sel = orc.sample_weighted(indptr, indices, None, None, 3, cdf=cdf)
    assert s.tolist() == [0, 3, 3, 6, 9]
    assert sel[:3].tolist() == [1, 0, 2]          # the only positive item, then zeros in order
    assert sel[3:6].tolist() == [6, 7, 8]         # deg <= K: the column in order
    assert sel[6:].tolist() == [9, 10, 11]        # no positive weight at all
    assert c.tolist() == [0, 0, 0, 2, 2, 2, 3, 3, 3]
    # with replacement: proportional to the weights; a column of zeros gives its last item
    probs = np.array([1, 3, 0, 4,   0, 0], dtype=np.float32)
    indptr = np.array([0, 4, 6])
    cdf = orc.weight_cdf(indptr, probs)
    n = 20000
    s, c, rows, sel = orc.sample_weighted(indptr, np.arange(6), None,
                                          np.zeros(n, dtype=np.int64), 2, replace=True, cdf=cdf)
    cnt = np.bincount(sel, minlength=4)
    assert cnt[2] == 0
    assert stats.chisquare(cnt[[0, 1, 3]], 2 * n * np.array([1, 3, 4]) / 8).pvalue > 0.01
    s, c, rows, sel = orc.sample_weighted(indptr, np.arange(6), None, np.array([1]), 3,
                                          replace=True, cdf=cdf)
    assert sel.tolist() == [5, 5, 5]


def test_cdf_sampling_agrees_with_key_sampling_in_distribution():
    """Inclusion frequencies of both weighted samplers on one skewed column."""
    rng = np.random.default_rng(9)
    deg, k, n = 40, 5, 20000
    w = rng.lognormal(sigma=1.5, size=deg).astype(np.float32)
    indptr = np.array([0, deg]); indices = np.arange(deg)
    cols = np.zeros(n, dtype=np.int64)
    a = orc.sample_weighted(indptr, indices, w, cols, k)[3]
    b = orc.sample_weighted(indptr, indices, None, cols, k, cdf=orc.weight_cdf(indptr, w))[3]
    ca, cb = np.bincount(a, minlength=deg), np.bincount(b, minlength=deg)
    keep = (ca + cb) >= 20
    assert stats.chi2_contingency(np.stack([ca[keep], cb[keep]]))[1] > 0.01
