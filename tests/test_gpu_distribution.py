"""Sampling laws of the DEVICE output (not of the CPU restatement): chi-square
tests at p > 0.01 of what the HIP kernels return through the C ABI, for the
Floyd and reservoir samplers, sampling with replacement, the key-weighted and
the CDF-weighted samplers and the collective (list) picks.  One requested
column repeated n times gives n independent samples (the stream position
differs), so a single launch produces a whole experiment.  Expected laws are
exact: uniform over the C(deg, K) subsets, K/deg inclusion, and successive
weighted sampling without replacement enumerated on tiny inputs."""
import itertools

import numpy as np
import pytest
import torch
from scipy import stats

from gsampler_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ALGOS = {"reservoir": capi.ALGO_RESERVOIR, "floyd": capi.ALGO_FLOYD}


def T(a, dtype=torch.int64):
    return torch.as_tensor(np.asarray(a), dtype=dtype, device=DEV)


def one_column(deg, n, fanout, algo, seed=7777, replace=False, offset=0):
    indptr, indices = T([0, deg]), T(np.arange(deg) + offset)
    s, c, rows, sel = capi.sample_uniform(indptr, indices, T(np.zeros(n, dtype=np.int64)), fanout,
                                          replace, algo, seed, 0)
    assert torch.equal(rows, indices[sel])
    return s.cpu().numpy(), sel.cpu().numpy()


def successive_probs(w, k):
    """P(ordered k-tuple) under successive weighted sampling without replacement."""
    out = {}
    for tup in itertools.permutations(range(len(w)), k):
        p, rest = 1.0, float(sum(w))
        for i in tup:
            p *= w[i] / rest
            rest -= w[i]
        out[tup] = p
    return out


def tuple_counts(picks):
    counts = {}
    for row in picks:
        t = tuple(row.tolist())
        counts[t] = counts.get(t, 0) + 1
    return counts


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
@pytest.mark.parametrize("deg,fanout", [(5, 2), (6, 3), (7, 1), (4, 3), (20, 17)])
def test_device_subsets_are_uniform(algo, deg, fanout):
    n = 20000 if deg < 10 else 60000
    s, sel = one_column(deg, n, fanout, ALGOS[algo])
    assert np.array_equal(s, np.arange(n + 1) * fanout)
    picks = np.sort(sel.reshape(n, fanout), axis=1)
    assert np.all(picks[:, 1:] > picks[:, :-1]) and picks.min() >= 0 and picks.max() < deg
    subsets = list(itertools.combinations(range(deg), fanout))
    index = {t: k for k, t in enumerate(subsets)}
    counts = np.zeros(len(subsets))
    for row in picks:
        counts[index[tuple(row)]] += 1
    p = stats.chisquare(counts).pvalue
    assert p > 0.01, (p, counts)


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
@pytest.mark.parametrize("deg,fanout,n", [(53, 15, 6000), (1000, 5, 40000), (97, 64, 3000)])
def test_device_inclusion_frequencies(algo, deg, fanout, n):
    """Per-edge inclusion counts against K/deg.  For a fixed-size design with
    equal inclusion probabilities sum((c - e)^2 / e) / (1 - K/deg) is chi-square
    with deg - 1 degrees of freedom."""
    _, sel = one_column(deg, n, fanout, ALGOS[algo], seed=11)
    counts = np.bincount(sel, minlength=deg).astype(float)
    expected = n * fanout / deg
    stat = np.sum((counts - expected) ** 2 / expected) / (1 - fanout / deg)
    p = stats.chi2.sf(stat, deg - 1)
    assert p > 0.01, p


def test_device_reservoir_above_64_slots():
    """Fan-outs beyond one wavefront go through the strided reservoir path."""
    deg, fanout, n = 400, 100, 2000
    s, sel = one_column(deg, n, fanout, capi.ALGO_AUTO, seed=5)
    picks = np.sort(sel.reshape(n, fanout), axis=1)
    assert np.all(picks[:, 1:] > picks[:, :-1])
    counts = np.bincount(sel, minlength=deg).astype(float)
    expected = n * fanout / deg
    stat = np.sum((counts - expected) ** 2 / expected) / (1 - fanout / deg)
    assert stats.chi2.sf(stat, deg - 1) > 0.01


def test_device_replace_positions_are_uniform():
    deg, fanout, n = 7, 3, 20000
    s, sel = one_column(deg, n, fanout, capi.ALGO_AUTO, replace=True)
    assert np.all(np.diff(s) == fanout)
    assert stats.chisquare(np.bincount(sel, minlength=deg)).pvalue > 0.01


def test_device_list_uniform_picks():
    counts = np.zeros(12)
    for t in range(3000):
        out = capi.list_sample_uniform(12, 4, call_id=t).cpu().numpy()
        assert np.unique(out).size == 4
        counts[out] += 1
    stat = np.sum((counts - 1000.0) ** 2 / 1000.0) / (1 - 4 / 12)
    assert stats.chi2.sf(stat, 11) > 0.01
    out = capi.list_sample_uniform(1000, 100, call_id=3).cpu().numpy()      # reservoir over the grid
    assert out.size == 100 and np.unique(out).size == 100 and out.max() < 1000


@pytest.mark.parametrize("w,k", [([3, 1, 2, 2, 1], 2), ([5, 1, 1, 1, 2], 3), ([1, 1, 1], 1)])
def test_device_key_weighted_columns_follow_successive_sampling(w, k):
    n = 30000
    indptr, indices = T([0, len(w)]), T(np.arange(len(w)) + 100)
    probs = T(w, torch.float32)
    s, c, rows, sel = capi.sample_weighted(indptr, indices, probs, T(np.zeros(n, dtype=np.int64)), k)
    assert torch.equal(rows, indices[sel])
    want = successive_probs(w, k)
    counts = tuple_counts(sel.cpu().numpy().reshape(n, k))
    assert set(counts) <= set(want)
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n
    assert stats.chisquare(obs, exp).pvalue > 0.01


@pytest.mark.parametrize("w,k", [([3, 1, 2, 2, 1], 2), ([5, 1, 0, 1, 2, 1], 3), ([1, 1, 1, 1], 3),
                                 ([1000, 1, 2, 3, 2], 3)])
def test_device_cdf_weighted_columns_follow_successive_sampling(w, k):
    n = 40000
    indptr, indices = T([0, len(w)]), T(np.arange(len(w)) + 100)
    probs = T(w, torch.float32)
    cdf = capi.weight_cdf(indptr, probs)
    s, c, rows, sel = capi.sample_weighted(indptr, indices, None, T(np.zeros(n, dtype=np.int64)), k,
                                           cdf=cdf)
    assert torch.equal(rows, indices[sel])
    assert np.array_equal(s.cpu().numpy(), np.arange(n + 1) * k)
    want = {t: p for t, p in successive_probs(w, k).items() if p > 0}
    counts = tuple_counts(sel.cpu().numpy().reshape(n, k))
    assert set(counts) <= set(want)
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n
    assert stats.chisquare(obs, exp).pvalue > 0.01


def test_device_weighted_samplers_agree_on_a_skewed_column():
    """Inclusion frequencies of the key sampler and of the CDF sampler on one
    log-normal column of 40 edges: the same law, so a contingency test between
    the two passes; zero-weight edges are never picked by either."""
    rng = np.random.default_rng(9)
    deg, k, n = 40, 5, 20000
    w = rng.lognormal(sigma=1.5, size=deg).astype(np.float32)
    w[[7, 19]] = 0.0
    indptr, indices, probs = T([0, deg]), T(np.arange(deg)), T(w, torch.float32)
    cols = T(np.zeros(n, dtype=np.int64))
    a = capi.sample_weighted(indptr, indices, probs, cols, k)[3].cpu().numpy()
    b = capi.sample_weighted(indptr, indices, None, cols, k,
                             cdf=capi.weight_cdf(indptr, probs))[3].cpu().numpy()
    ca, cb = np.bincount(a, minlength=deg), np.bincount(b, minlength=deg)
    assert ca[7] == ca[19] == cb[7] == cb[19] == 0
    keep = (ca + cb) >= 20
    assert stats.chi2_contingency(np.stack([ca[keep], cb[keep]]))[1] > 0.01


@pytest.mark.parametrize("w,k", [([1, 2, 3, 4], 2), ([5, 1, 1, 1, 2], 3)])
def test_device_collective_weighted_pick_follows_successive_sampling(w, k):
    """The list pick in one launch: 6000 segments that all hold the same weights."""
    n = 6000
    probs = T(np.tile(np.asarray(w, dtype=np.float32), n), torch.float32)
    range_ = T(np.arange(n + 1) * len(w))
    idx, out_range = capi.list_sample_weighted(probs, k, False, range_)
    assert np.array_equal(out_range.cpu().numpy(), np.arange(n + 1) * k)
    picks = idx.cpu().numpy().reshape(n, k) - (np.arange(n) * len(w))[:, None]
    want = successive_probs(w, k)
    counts = tuple_counts(picks)
    assert set(counts) <= set(want)
    obs = np.array([counts.get(t, 0) for t in want])
    exp = np.array([want[t] for t in want]) * n
    assert stats.chisquare(obs, exp).pvalue > 0.01


def test_device_replace_frequencies_follow_weights():
    w = np.array([1, 0, 3, 6], dtype=np.float32)
    idx, _ = capi.list_sample_weighted(T(w, torch.float32), 40000, True)
    counts = np.bincount(idx.cpu().numpy(), minlength=4)
    assert counts[1] == 0
    assert stats.chisquare(counts[[0, 2, 3]], 40000 * np.array([0.1, 0.3, 0.6])).pvalue > 0.01
    indptr, indices = T([0, 4]), T(np.arange(4))
    for cdf in (None, capi.weight_cdf(indptr, T(w, torch.float32))):
        s, c, rows, sel = capi.sample_weighted(indptr, indices, T(w, torch.float32),
                                               T(np.zeros(2000, dtype=np.int64)), 20, True, cdf=cdf)
        counts = np.bincount(sel.cpu().numpy(), minlength=4)
        assert counts[1] == 0
        assert stats.chisquare(counts[[0, 2, 3]], 40000 * np.array([0.1, 0.3, 0.6])).pvalue > 0.01


def test_device_random_walk_and_node2vec_transition_laws():
    """One-step laws on a small graph: a uniform step picks each in-neighbour
    with probability 1/deg; a second-order step weighs the return edge by p, a
    neighbour of the previous node by q and any other candidate by 1 (the
    acceptance rule with integer levels), here with p = 2, q = 0.5 as configured."""
    # columns: 0 <- {1,2,3,4}; 1 <- {0,2}; 2 <- {0}; 3 <- {0,4}; 4 <- {0,1,2,3}
    cols = [[1, 2, 3, 4], [0, 2], [0], [0, 4], [0, 1, 2, 3]]
    indptr = T(np.cumsum([0] + [len(c) for c in cols]))
    indices = T(np.concatenate(cols))
    n = 40000
    start = T(np.zeros(n, dtype=np.int64))
    tr = capi.random_walk(indptr, indices, start, 1, 7777, 0).cpu().numpy()
    assert stats.chisquare(np.bincount(tr[1], minlength=5)[1:]).pvalue > 0.01
    p_, q_ = 2.0, 0.5
    tr = capi.node2vec(indptr, indices, T(np.full(n, 1, dtype=np.int64)), 2, p_, q_, 7777, 1).cpu().numpy()
    # first hop from 1: uniform over {0, 2}; look at walks 1 -> 0 -> x
    first = tr[1]
    assert stats.chisquare(np.bincount(first, minlength=3)[[0, 2]]).pvalue > 0.01
    via0 = tr[2][first == 0]
    # candidates of column 0: 1 (the previous node: weight p), 2 (in column 1, a
    # neighbour of the previous node: q), 3 and 4 (strangers: 1).  With integer
    # levels y in {0, 1}: P(accept | candidate) = P(y < h) = 1 for h = 2, 1/2 for
    # h = 1 and 1/2 for h = 0.5 (y = 0 only), so the law is (2, 1, 1, 1) / 5.
    want = np.array([2.0, 1.0, 1.0, 1.0]) / 5.0
    obs = np.bincount(via0, minlength=5)[1:]
    assert stats.chisquare(obs, want * obs.sum()).pvalue > 0.01
