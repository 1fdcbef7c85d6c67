"""Oracle walks: the reference's own DAG fixtures, uniform next hops, and the
node2vec transition law derived from its acceptance rule."""
import numpy as np
from scipy import stats

from oracle import binding as orc
from tests.conftest import golden, random_csc

# tests/test_random_walk.cc:27-60 and tests/test_node2vec.cc:27-60
DAG = golden()["walk_dag"]
DAG_INDPTR = np.array(DAG["indptr"])
DAG_INDICES = np.array(DAG["indices"])


def _edge_exists(src, dst):
    return dst == -1 or dst in DAG_INDICES[DAG_INDPTR[src]:DAG_INDPTR[src + 1]]


def _check_dag(trace):
    assert trace.shape == (4, 4)               # [walk_length + 1, num_seeds]
    assert trace[0].tolist() == [4, 2, 3, 1]
    for j in range(4):
        path = trace[:, j]
        for a, b in zip(path, path[1:]):
            if a == -1:
                assert b == -1
            else:
                assert _edge_exists(a, b)
    # every walk ends in node 0 and then hits the dead end
    assert trace[:, 3].tolist() == [1, 0, -1, -1]
    assert trace[:, 1].tolist() == [2, 1, 0, -1]


def test_reference_dag_fixtures():
    for call in range(5):
        _check_dag(orc.random_walk(DAG_INDPTR, DAG_INDICES, [4, 2, 3, 1], 3, call_id=call))
        _check_dag(orc.node2vec(DAG_INDPTR, DAG_INDICES, [4, 2, 3, 1], 3, 2.0, 0.5, call_id=call))


def test_random_walk_next_hop_is_uniform_over_the_column():
    indptr = np.array([0, 4, 4, 4, 4, 4]); indices = np.array([1, 2, 2, 4])
    n = 20000
    tr = orc.random_walk(indptr, indices, np.zeros(n, dtype=np.int64), 2)
    counts = np.bincount(tr[1], minlength=5)
    assert counts[0] == 0 and counts[3] == 0
    assert stats.chisquare(counts[[1, 2, 4]], n * np.array([.25, .5, .25])).pvalue > 0.01
    assert np.all(tr[2] == -1)                     # columns 1, 2, 4 are empty
    tr = orc.random_walk(indptr, indices, [7, -1, 1], 2)   # ids outside the matrix
    assert np.all(tr[1:] == -1)


def test_node2vec_transition_law():
    """p = 2, q = 0.5: levels y in {0, 1} with probability 1/2 each.  y = 0 is
    accepted outright (0 < min(p, q, 1)); y = 1 is accepted only for a return to
    the previous node (1 < p) -- a neighbour of the previous node needs 1 < q and
    any other node 1 < 1.  So candidates are accepted with probability 1 for the
    previous node and 1/2 otherwise."""
    # undirected triangle 0-1-2 plus pendant 3 attached to 0 (rows sorted per column)
    adj = {0: [1, 2, 3], 1: [0, 2], 2: [0, 1], 3: [0]}
    indptr = np.concatenate([[0], np.cumsum([len(adj[i]) for i in range(4)])])
    indices = np.concatenate([adj[i] for i in range(4)])
    n = 60000
    tr = orc.node2vec(indptr, indices, np.full(n, 1), 2, 2.0, 0.5, seed=3)
    # first step: no previous node -> every candidate accepted with prob 1/2 -> uniform
    c1 = np.bincount(tr[1], minlength=4)
    assert stats.chisquare(c1[[0, 2]]).pvalue > 0.01
    # second step from node 0 (previous = 1): weights 1 (return to 1), 1/2 (2), 1/2 (3)
    at0 = tr[2][tr[1] == 0]
    c2 = np.bincount(at0, minlength=4)
    assert c2[0] == 0
    assert stats.chisquare(c2[[1, 2, 3]], at0.size * np.array([.5, .25, .25])).pvalue > 0.01
    # p = q = 1 accepts everything: a plain uniform walk
    tr = orc.node2vec(indptr, indices, np.zeros(n, dtype=np.int64), 1, 1.0, 1.0)
    assert stats.chisquare(np.bincount(tr[1], minlength=4)[1:]).pvalue > 0.01


def test_node2vec_neighbour_rule_uses_q():
    """q = 3, p = 1: levels y in {0, 1, 2}; y = 0 accepted outright; y = 1, 2 only
    when the candidate is a neighbour of the previous node (y < q = 3)."""
    adj = {0: [1, 2, 3], 1: [0, 2], 2: [0, 1], 3: [0]}
    indptr = np.concatenate([[0], np.cumsum([len(adj[i]) for i in range(4)])])
    indices = np.concatenate([adj[i] for i in range(4)])
    n = 60000
    tr = orc.node2vec(indptr, indices, np.full(n, 1), 2, 1.0, 3.0, seed=5)
    at0 = tr[2][tr[1] == 0]           # previous = 1 whose neighbours are {0, 2}
    c = np.bincount(at0, minlength=4)
    # candidate 1 (return): h = p = 1 -> accepted for y = 0 only: 1/3
    # candidate 2 (neighbour of 1): h = q = 3 -> always accepted: 1
    # candidate 3: h = 1 -> 1/3
    w = np.array([1 / 3, 1, 1 / 3])
    assert stats.chisquare(c[[1, 2, 3]], at0.size * w / w.sum()).pvalue > 0.01


def test_segment_sort():
    rng = np.random.default_rng(0)
    indptr, indices = random_csc(rng, 300, 1000, 40, hub_deg=5000)
    out = orc.segment_sort(indptr, indices)
    for c in range(300):
        assert np.array_equal(out[indptr[c]:indptr[c + 1]], np.sort(indices[indptr[c]:indptr[c + 1]]))
