"""Differential test over many small random cases: every operator of the path
on randomly shaped inputs (empty columns, one hub, duplicate and out-of-range
seeds, empty batches, sizes next to tile and chunk boundaries) against the CPU
restatement, bit for bit.  All inputs are valid ones; sizes are drawn so that
the cases straddle the work-group tiles (256, 1024, 2048, 4096, 8192) of the
kernels."""
import numpy as np
import pytest
import torch

from gsampler_amd import capi
from oracle import binding as orc
from tests.conftest import random_csc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
EDGY = [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096,
        4097, 8191, 8192, 8193]


def T(a, dtype=np.int64):
    return None if a is None else torch.as_tensor(np.asarray(a, dtype=dtype), device=DEV)


def same(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(g.cpu().numpy(), np.asarray(w))


def draw_size(rng, hi):
    return int(rng.choice(EDGY)) if rng.random() < 0.5 else int(rng.integers(0, hi))


def random_ptr(rng, total, batches):
    cuts = np.sort(rng.integers(0, total + 1, size=batches - 1)) if batches > 1 else np.zeros(0, int)
    return np.concatenate([[0], cuts, [total]]).astype(np.int64)


@pytest.mark.parametrize("seed", range(120))
def test_random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    C = max(1, draw_size(rng, 3000))
    R = max(1, draw_size(rng, 5000))
    indptr, indices = random_csc(rng, C, R, int(rng.integers(0, 40)), empty_frac=rng.random() * 0.6,
                                 hub_deg=int(rng.choice([0, 0, 300, 5000])))
    g_indptr, g_indices = T(indptr), T(indices)
    S = draw_size(rng, 4000)
    seeds = rng.integers(-2, C + 3, size=S)                 # some outside the matrix: empty columns
    if S and rng.random() < 0.5:
        seeds[rng.integers(0, S, size=S // 3 + 1)] = seeds[0]    # repeats
    g_seeds = T(seeds)
    call = int(rng.integers(0, 1000))

    # column slice, plain and batched with encoding
    same(capi.col_slice(g_indptr, g_indices, g_seeds), orc.col_slice(indptr, indices, seeds))
    B = int(rng.integers(1, 9))
    ptr = random_ptr(rng, S, B)
    same(capi.col_slice(g_indptr, g_indices, g_seeds, batch_ptr=T(ptr), encode_stride=R),
         orc.col_slice(indptr, indices, seeds, batch_ptr=ptr, encode_stride=R))

    # uniform sampling: fused and on the whole matrix, with and without replacement
    K = int(rng.choice([1, 2, 5, 8, 9, 16, 17, 33, 64, 100]))
    replace = bool(rng.random() < 0.3)
    algo = int(rng.integers(0, 3)) if K <= 64 else int(rng.choice([0, 1]))
    got = capi.sample_uniform(g_indptr, g_indices, g_seeds, K, replace, algo, 7777, call)
    want = orc.sample_uniform(indptr, indices, seeds, K, replace, algo, 7777, call)
    same(got, want)
    same(capi.sample_uniform(g_indptr, g_indices, None, K, replace, algo, 7777, call + 1),
         orc.sample_uniform(indptr, indices, None, K, replace, algo, 7777, call + 1))

    # unique + relabel of the sampled layer, per batch (seeds clipped into the id range first)
    ok_seeds = np.clip(seeds, 0, C - 1)
    w_sub, w_col, w_rows, _ = orc.sample_uniform(indptr, indices, ok_seeds, K, replace, algo, 7777, call)
    eptr = w_sub[ptr]
    same(capi.unique_relabel(T(ok_seeds), T(w_rows), T(ptr), T(eptr), T(w_col)),
         orc.unique_relabel(ok_seeds, w_rows, ptr, eptr, w_col))

    # row slice by a random picked set (repeats, ids no edge carries)
    P = draw_size(rng, 600)
    picked = rng.integers(0, R + 5, size=P)
    same(capi.minor_slice(g_indices, T(picked), indptr=g_indptr),
         orc.minor_slice(indices, picked, indptr=indptr))
    col = orc.csc2coo(indptr)
    same(capi.minor_slice(g_indices, T(picked), edge_major=T(col)),
         orc.minor_slice(indices, picked, edge_major=col))
    assert np.array_equal(capi.csc2coo(g_indptr).cpu().numpy(), col)

    # weighted sampling by keys and through the CDF
    if indices.size:
        probs = rng.random(indices.size).astype(np.float32)
        probs[rng.random(indices.size) < 0.2] = 0.0
        g_probs = torch.as_tensor(probs, device=DEV)
        Kw = min(K, 64)
        same(capi.sample_weighted(g_indptr, g_indices, g_probs, T(ok_seeds), Kw, replace, 7777, call),
             orc.sample_weighted(indptr, indices, probs, ok_seeds, Kw, replace, 7777, call))
        packed = bool(call % 2)           # row ids inside the CDF's entries, or not
        cdf = capi.weight_cdf(g_indptr, g_probs, g_indices if packed else None)
        h_cdf = orc.weight_cdf(indptr, probs, indices if packed else None)
        assert np.array_equal(cdf.cpu().numpy(), h_cdf)
        same(capi.sample_weighted(g_indptr, g_indices, None, T(ok_seeds), Kw, replace, 7777, call,
                                  cdf=cdf),
             orc.sample_weighted(indptr, indices, None, ok_seeds, Kw, replace, 7777, call, cdf=h_cdf))
        # scalar sums onto columns and rows
        e = (rng.random(indices.size).astype(np.float32) + 0.25)
        for view_g, view_o in ((("csc", g_indptr, g_indices), ("csc", indptr, indices)),
                               (("coo", g_indices, T(col)), ("coo", indices, col))):
            got = capi.spmm(view_g, "copy_rhs", "sum", None, torch.as_tensor(e, device=DEV), 0, C)
            want = orc.spmm(view_o, "copy_rhs", "sum", None, e, 0, C)
            assert np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-6)   # fp32: 1e-5 relative
        got = capi.e_square_sum(("coo", g_indices, T(col)), torch.as_tensor(e, device=DEV), 2, R)
        want = orc.e_square_sum(("coo", indices, col), e, 2, R)
        assert np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-6)

    # list sampling and walks
    n = draw_size(rng, 6000)
    if n:
        lp = rng.random(n).astype(np.float32)
        k = int(rng.choice([1, 7, 64, 65, 500]))
        got = capi.list_sample_weighted(torch.as_tensor(lp, device=DEV), k, False, None, 7777, call)
        want = orc.list_sample_weighted(lp, k, False, None, 7777, call)
        same(got if isinstance(got, tuple) else (got,), want if isinstance(want, tuple) else (want,))
    walkers = np.clip(seeds[:200], 0, C - 1)
    if walkers.size:
        sq = min(C, R)          # walks need a square matrix: keep ids inside it
        w_indptr, w_indices = random_csc(rng, sq, sq, 6, empty_frac=0.3)
        assert np.array_equal(
            capi.random_walk(T(w_indptr), T(w_indices), T(walkers % sq), 5, 7777, call).cpu().numpy(),
            orc.random_walk(w_indptr, w_indices, walkers % sq, 5, 7777, call))
