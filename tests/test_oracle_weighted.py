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
def _unpack_cdf(cdf, indptr):
    """(row_bits, share bits, per-edge share, per-edge row) of a packed CDF."""
    words = cdf.view(np.uint64)
    row_bits = int(words[0])
    cb = min(62, 64 - row_bits)
    entries = words[1:]
    share = entries >> np.uint64(row_bits)
    rows = entries & np.uint64((1 << row_bits) - 1) if row_bits else None
    return row_bits, cb, share, rows


@pytest.mark.parametrize("num_rows", [None, 1000, 2**22, 2**32, 2**33])
def test_weight_cdf_holds_shares_of_the_column_mass_and_row_ids(num_rows):
    """Entry e = share(e) << row_bits | row: shares are non-decreasing inside a column, end at
    2^cb - 1, and an edge's piece is its weight's part of the column's weight (to the 31-bit
    quantisation of the weights and one unit of the share); rows come back unchanged."""
    rng = np.random.default_rng(3)
    deg = np.array([5, 0, 300, 1, 4, 0, 7, 70000])
    indptr = np.concatenate([[0], np.cumsum(deg)])
    nnz = int(deg.sum())
    w = rng.lognormal(size=nnz).astype(np.float32)
    w[indptr[4]:indptr[5]] = [0.0, -1.0, 0.0, 0.0]      # a column without positive weights
    w[indptr[6] + 2] = 0.0
    w[indptr[6] + 5:indptr[6] + 7] = 0.0                 # zeros after the last positive edge
    indices = None
    if num_rows is not None:
        indices = rng.integers(0, num_rows, size=nnz)
        indices[0] = num_rows - 1
    cdf = orc.weight_cdf(indptr, w, indices, num_rows)
    row_bits, cb, share, rows = _unpack_cdf(cdf, indptr)
    if num_rows is None or num_rows > 2**32:
        assert row_bits == 0 and cb == 62
    else:
        assert row_bits == max(1, int(num_rows - 1).bit_length()) and cb == min(62, 64 - row_bits)
        assert np.array_equal(rows.astype(np.int64), indices)
    full = (1 << cb) - 1
    for c in range(deg.size):
        lo, hi = indptr[c], indptr[c + 1]
        if hi == lo:
            continue
        wc = np.where(w[lo:hi] > 0, w[lo:hi], 0).astype(np.float64)
        sc = [int(v) for v in share[lo:hi]]
        if wc.max() <= 0:
            assert all(v == 0 for v in sc)
            continue
        assert sc[-1] == full and all(b >= a for a, b in zip(sc, sc[1:]))
        piece = np.diff(np.array([0] + sc, dtype=object)).astype(np.float64)
        assert np.all(piece[wc == 0] == 0)
        # from the last positive edge on the share is 2^cb - 1
        last_pos = int(np.nonzero(wc)[0][-1])
        assert all(v == full for v in sc[last_pos:])
        want = wc / wc.sum() * 2.0**cb
        # weights are cut to multiples of max / 2^31 first: relative error below deg / 2^31 on
        # the total and one such unit on the edge itself
        unit = wc.max() / 2**31 / wc.sum() * 2.0**cb
        assert np.all(np.abs(piece - want) <= 2.0 + unit + want * (hi - lo) * 2.0**-30)


def test_weight_cdf_shares_are_exact_integer_quotients():
    """share = floor(G * 2^cb / T) recomputed with Python integers from the quantised weights
    (weights that are powers of two times the maximum quantise exactly)."""
    w = np.array([1, 0.5, 0.25, 1, 0.125, 0.5, 0, 1], dtype=np.float32)
    indptr = np.array([0, 8])
    for num_rows, idx in ((None, None), (5, np.array([4, 3, 2, 1, 0, 1, 2, 3]))):
        cdf = orc.weight_cdf(indptr, w, idx, num_rows)
        row_bits, cb, share, rows = _unpack_cdf(cdf, indptr)
        q = [int(x * 2**31) for x in w.tolist()]
        total, g, want = sum(q), 0, []
        for x in q:
            g += x
            want.append((1 << cb) - 1 if g == total else (g << cb) // total)
        assert [int(v) for v in share] == want


@pytest.mark.parametrize("w,k", [([3, 1, 2, 2, 1], 2), ([5, 1, 0, 1, 2, 1], 3), ([1, 1, 1, 1], 3),
                                 ([1000, 1, 2, 3, 2], 3)])   # mass on one item: the sequential phase
@pytest.mark.parametrize("packed_rows", [False, True])
def test_cdf_column_sampling_is_successive_weighted_sampling(w, k, packed_rows):
    """Ordered k-tuples drawn through the CDF against the exact law of successive
    weighted sampling without replacement (zero weights have probability 0)."""
    n = 40000
    indptr = np.array([0, len(w)]); indices = np.arange(len(w)) + 100
    probs = np.array(w, dtype=np.float32)
    cdf = orc.weight_cdf(indptr, probs, indices if packed_rows else None)
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
    cdf = orc.weight_cdf(indptr, probs, indices + 7)
    s, c, rows, sel = orc.sample_weighted(indptr, indices + 7, None, None, 3, cdf=cdf)
    assert s.tolist() == [0, 3, 3, 6, 9] and np.array_equal(rows, sel + 7)
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
