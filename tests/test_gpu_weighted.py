"""Weighted sampling on the GPU vs the oracle: bit-exact keys and picks."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd import capi
from oracle import binding as orc
from tests.conftest import random_csc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return None if a is None else torch.as_tensor(np.asarray(a, dtype=np.int64), device=DEV)


def F(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32), device=DEV)


def same(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(g.cpu().numpy(), w)


def test_key_arithmetic_is_bit_identical():
    rng = np.random.default_rng(0)
    cases = [0, 2**64 - 1, (2**51 - 1) << 12, 1 << 12, 2**63] + \
        [int(x) for x in rng.integers(0, 2**64, size=300, dtype=np.uint64)]
    for i, r in enumerate(cases):
        w = float(np.float32(rng.random() * 3 + 1e-3))
        e, k = capi.weighted_key_probe(7, 3, 1000 + i, i, w, r)
        assert e == orc.neg_log2_unit(r)
        assert k == orc.weighted_key(7, 3, 1000 + i, i, w)
    assert np.isinf(capi.weighted_key_probe(7, 3, 1, 1, 0.0, 5)[1])
    assert np.isinf(capi.weighted_key_probe(7, 3, 1, 1, -2.0, 5)[1])


@pytest.mark.parametrize("fanout", [1, 5, 15, 32, 33, 64])
def test_column_sampling_parity(fanout):
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 3000, 10**6, 120, hub_deg=30000)
    probs = rng.lognormal(0, 1, size=indices.size).astype(np.float32)
    probs[rng.random(indices.size) < 0.05] = 0.0
    cols = rng.integers(0, 3000, size=2000)
    same(capi.sample_weighted(T(indptr), T(indices), F(probs), T(cols), fanout, call_id=2),
         orc.sample_weighted(indptr, indices, probs, cols, fanout, call_id=2))
    same(capi.sample_weighted(T(indptr), T(indices), F(probs), None, fanout),
         orc.sample_weighted(indptr, indices, probs, None, fanout))


@pytest.mark.parametrize("fanout", [3, 70])
def test_column_sampling_with_replacement_parity(fanout):
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 2000, 10**6, 80, hub_deg=9000)
    probs = rng.random(indices.size).astype(np.float32)
    probs[rng.random(indices.size) < 0.1] = 0.0
    probs[indptr[5]:indptr[6]] = 0.0            # a column without positive weight
    cols = rng.integers(0, 2000, size=1500)
    same(capi.sample_weighted(T(indptr), T(indices), F(probs), T(cols), fanout, True),
         orc.sample_weighted(indptr, indices, probs, cols, fanout, True))
    same(capi.sample_weighted(T(indptr), T(indices), F(probs), None, fanout, True),
         orc.sample_weighted(indptr, indices, probs, None, fanout, True))


def _weighted_case(seed, cols=3000, hub=30000):
    rng = np.random.default_rng(seed)
    indptr, indices = random_csc(rng, cols, 10**6, 120, hub_deg=hub)
    probs = rng.lognormal(0, 1, size=indices.size).astype(np.float32)
    probs[rng.random(indices.size) < 0.05] = 0.0
    probs[indptr[7]:indptr[8]] = 0.0             # a column without positive weight
    lo = indptr[11]                              # a column with a single positive weight
    probs[lo:indptr[12]] = 0.0
    if indptr[12] > lo:
        probs[lo] = 2.0
    for c in (20, 21, 22, 23):                   # nearly all mass on one or two items
        if indptr[c + 1] - indptr[c] > 2:
            probs[indptr[c]] = 1e7
            probs[indptr[c] + 2] = 3e6
    return rng, indptr, indices, probs


@pytest.mark.parametrize("num_rows", [None, 0, 2**22, 2**27, 2**32, 2**40])
def test_weight_cdf_is_bit_identical(num_rows):
    """None: no row ids packed; 0: the bits that the largest id needs; wider id spaces leave
    fewer bits to the shares; ids beyond 32 bits are not packed."""
    rng, indptr, indices, probs = _weighted_case(1)
    if num_rows is None:
        g, h = capi.weight_cdf(T(indptr), F(probs)), orc.weight_cdf(indptr, probs)
    else:
        ids = indices if num_rows == 0 else rng.integers(0, num_rows, size=indices.size)
        g = capi.weight_cdf(T(indptr), F(probs), T(ids), num_rows or None)
        h = orc.weight_cdf(indptr, probs, ids, num_rows or None)
    assert np.array_equal(g.cpu().numpy(), h)
    empty = capi.weight_cdf(T(np.zeros(4)), F(np.zeros(0)))
    assert empty.cpu().tolist() == [0]


def test_weight_cdf_of_one_long_column():
    """A column far longer than a tile: the shares of every tile refer to the same total."""
    rng = np.random.default_rng(8)
    deg = np.array([3, 300_000, 0, 5])
    indptr = np.concatenate([[0], np.cumsum(deg)])
    probs = rng.lognormal(size=int(deg.sum())).astype(np.float32)
    ids = rng.integers(0, 2_450_000, size=probs.size)
    assert np.array_equal(capi.weight_cdf(T(indptr), F(probs), T(ids), 2_450_000).cpu().numpy(),
                          orc.weight_cdf(indptr, probs, ids, 2_450_000))


@pytest.mark.parametrize("fanout", [1, 5, 15, 64])
@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("packed_rows", [False, True])
def test_cdf_column_sampling_parity(fanout, replace, packed_rows):
    rng, indptr, indices, probs = _weighted_case(fanout)
    cdf = orc.weight_cdf(indptr, probs, indices if packed_rows else None)
    g_cdf = capi.weight_cdf(T(indptr), F(probs), T(indices) if packed_rows else None)
    cols = np.concatenate([rng.integers(0, 3000, size=2000), [7, 11, 7, 20, 21, 22, 23, 20]])
    same(capi.sample_weighted(T(indptr), T(indices), None, T(cols), fanout, replace, call_id=4,
                              cdf=g_cdf),
         orc.sample_weighted(indptr, indices, None, cols, fanout, replace, call_id=4, cdf=cdf))
    same(capi.sample_weighted(T(indptr), T(indices), None, None, fanout, replace, cdf=g_cdf),
         orc.sample_weighted(indptr, indices, None, None, fanout, replace, cdf=cdf))


def test_cdf_sampling_with_replacement_beyond_the_register_budget():
    # fanouts above 64 are written pick by pick instead of being held in registers
    rng, indptr, indices, probs = _weighted_case(3)
    cdf = orc.weight_cdf(indptr, probs, indices)
    g_cdf = capi.weight_cdf(T(indptr), F(probs), T(indices))
    cols = rng.integers(0, 3000, size=500)
    for fanout in (65, 100):
        same(capi.sample_weighted(T(indptr), T(indices), None, T(cols), fanout, True, call_id=2,
                                  cdf=g_cdf),
             orc.sample_weighted(indptr, indices, None, cols, fanout, True, call_id=2, cdf=cdf))
    with pytest.raises(capi.GsError):
        capi.sample_weighted(T(indptr), T(indices), None, T(cols), 65, False, cdf=g_cdf)


@pytest.mark.parametrize("n,k", [(10, 20), (1000, 64), (233000, 512), (5000, 5000)])
def test_list_sampling_parity(n, k):
    rng = np.random.default_rng(n)
    probs = rng.random(n).astype(np.float32)
    probs[rng.random(n) < 0.2] = 0.0
    same(capi.list_sample_weighted(F(probs), k, call_id=4),
         orc.list_sample_weighted(probs, k, call_id=4))
    same(capi.list_sample_weighted(F(probs), k, replace=True, call_id=4),
         orc.list_sample_weighted(probs, k, replace=True, call_id=4))
    for replace in (False, True):
        for algo in (0, 1):
            got = capi.list_sample_uniform(n, k, replace, algo, call_id=9)
            assert np.array_equal(got.cpu().numpy(),
                                  orc.list_sample_uniform(n, k, replace, algo, call_id=9))


def test_batched_list_sampling_parity():
    rng = np.random.default_rng(5)
    sizes = np.array([0, 700, 3, 20000, 0, 512, 513])
    ranges = np.concatenate([[0], np.cumsum(sizes)])
    probs = rng.random(ranges[-1]).astype(np.float32)
    probs[rng.random(probs.size) < 0.3] = 0.0
    same(capi.list_sample_weighted(F(probs), 512, range_=T(ranges)),
         orc.list_sample_weighted(probs, 512, range_=ranges))
    same(capi.list_sample_weighted(F(probs), 100, replace=True, range_=T(ranges)),
         orc.list_sample_weighted(probs, 100, replace=True, range_=ranges))


@pytest.mark.parametrize("case", ["few_positive", "all_zero", "repeated_weights", "one_heavy",
                                  "k_limits"])
def test_list_selection_cases(case):
    """The K smallest keys by selection (up to 2048 picks): cells of equal keys far larger
    than the pick count, weights that repeat, one dominant weight, pick counts at and
    around the limit of the selection path."""
    rng = np.random.default_rng(len(case))
    n = 300_000
    probs = rng.random(n).astype(np.float32)
    ks = [512]
    if case == "few_positive":        # fewer positive weights than picks: the rest by index
        probs[rng.permutation(n)[300:]] = 0.0
    elif case == "all_zero":
        probs[:] = 0.0
    elif case == "repeated_weights":  # many equal weights (keys still differ: other draws)
        probs = rng.choice(np.array([0.25, 0.5, 1.0], dtype=np.float32), size=n)
    elif case == "one_heavy":
        probs *= 1e-6
        probs[12345] = 1e6
    else:
        ks = [1, 2047, 2048, 2049]
    for k in ks:
        same(capi.list_sample_weighted(F(probs), k, call_id=2),
             orc.list_sample_weighted(probs, k, call_id=2))


def test_batched_list_selection_parity():
    """Segments long enough for the selection path, ragged, one of them empty, one taken
    whole, one with fewer positive weights than picks."""
    rng = np.random.default_rng(8)
    sizes = np.array([60000, 0, 300, 4097, 150000, 33000])
    ranges = np.concatenate([[0], np.cumsum(sizes)])
    probs = rng.random(ranges[-1]).astype(np.float32)
    probs[rng.random(probs.size) < 0.3] = 0.0
    probs[ranges[5]:ranges[6]] = 0.0
    probs[ranges[5] + 100:ranges[5] + 200] = 0.5
    for k in (64, 512):
        same(capi.list_sample_weighted(F(probs), k, range_=T(ranges), call_id=3),
             orc.list_sample_weighted(probs, k, range_=ranges, call_id=3))


def test_operators_through_the_api():
    rng = np.random.default_rng(6)
    indptr, indices = random_csc(rng, 500, 400, 60)
    indices[0] = 399
    probs = rng.random(indices.size).astype(np.float32)
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    m.edata["w"] = F(probs)
    gs.manual_seed(99)
    s = m.individual_sampling(7, m.edata["w"], False)
    want = orc.sample_weighted(indptr, indices, probs, None, 7, seed=99, call_id=0)
    assert np.array_equal(s.csc[1].cpu().numpy(), want[2])
    assert np.array_equal(s.edata["w"].cpu().numpy(), probs[want[3]])
    p = rng.random(400).astype(np.float32)
    sub, picked = m.collective_sampling(50, F(p), False)          # call id 1
    want_idx, _ = orc.list_sample_weighted(p, 50, seed=99, call_id=1)
    assert np.array_equal(picked.cpu().numpy(), want_idx)
    assert sub.num_rows() == 50
    u = torch.ops.gs_ops._CAPI_ListSampling(400, 30, False)          # call id 2
    assert np.array_equal(u.cpu().numpy(), orc.list_sample_uniform(400, 30, seed=99, call_id=2))
    ranges = np.array([0, 100, 400])
    idx, ptr = torch.ops.gs_ops._CAPI_BatchListSamplingWithProbs(F(p), 20, False, T(ranges))
    w_idx, w_ptr = orc.list_sample_weighted(p, 20, range_=ranges, seed=99, call_id=3)
    assert np.array_equal(idx.cpu().numpy(), w_idx) and np.array_equal(ptr.cpu().numpy(), w_ptr)
    idx, ptr = torch.ops.gs_ops._CAPI_BatchListSampling(20, False, T(ranges))
    w_idx, w_ptr = orc.list_sample_weighted(np.ones(400, dtype=np.float32), 20, range_=ranges,
                                            seed=99, call_id=4)
    assert np.array_equal(idx.cpu().numpy(), w_idx)
