"""Frontier and labels of a row-sliced matrix (rows = positions in a short list
of ids) in one launch, against the oracle's unique + relabel over all edges.
Integer work: bit-exact."""
import numpy as np
import pytest
import torch

from gsampler_amd import capi
from oracle import binding as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int64), device=DEV)


def _case(rng, S, R, E, id_range, repeat_seeds=False, repeat_list=False, unused=0.3):
    seeds = rng.integers(0, id_range, size=S) if repeat_seeds else rng.permutation(id_range)[:S]
    list_ids = rng.integers(0, id_range, size=R) if repeat_list else rng.permutation(id_range)[:R]
    live = np.flatnonzero(rng.random(R) >= unused)          # listed ids that some edge uses
    row = rng.choice(live, size=E) if live.size and E else np.empty(0, dtype=np.int64)
    col = rng.integers(0, max(S, 1), size=row.size)
    return seeds.astype(np.int64), list_ids.astype(np.int64), row.astype(np.int64), col


def _check(seeds, list_ids, row, col):
    first = capi.first_position(T(row), list_ids.size)
    frontier, list_label, seed_label = capi.list_labels(T(seeds), T(list_ids), first)
    want = orc.unique_relabel(seeds, list_ids[row], edge_col=col if seeds.size else None)
    assert np.array_equal(frontier.cpu().numpy(), want[0])
    assert np.array_equal(list_label.cpu().numpy()[row], want[2])
    if seeds.size:
        assert np.array_equal(seed_label.cpu().numpy()[col], want[3])
        # every seed's label is the place of its first occurrence among the frontier
        assert np.array_equal(want[0][seed_label.cpu().numpy()], seeds)


@pytest.mark.parametrize("S,R,E", [(512, 512, 200_000), (1, 1, 10), (0, 700, 50_000),
                                   (1000, 1048, 300_000), (2047, 1, 5), (3, 2045, 100_000),
                                   (100, 33, 0), (700, 1025, 4000)])
@pytest.mark.parametrize("mode", ["distinct", "overlap", "repeats"])
def test_list_labels_match_unique_over_the_edges(S, R, E, mode):
    rng = np.random.default_rng(S * 7 + R * 3 + len(mode))
    id_range = {"distinct": 10**6, "overlap": S + R + 5, "repeats": max(2, (S + R) // 3)}[mode]
    seeds, list_ids, row, col = _case(rng, S, R, E, id_range, repeat_seeds=mode == "repeats",
                                      repeat_list=mode == "repeats")
    _check(seeds, list_ids, row, col)


def test_list_labels_large_ids_and_all_used():
    rng = np.random.default_rng(5)
    seeds = rng.integers(2**40, 2**41, size=300)
    list_ids = np.concatenate([seeds[:100], rng.integers(-2**50, 2**62, size=400)])
    row = rng.integers(0, 500, size=100_000)
    row[:500] = rng.permutation(500)                          # every listed id is used
    col = rng.integers(0, 300, size=row.size)
    _check(seeds, list_ids, row, col)


def test_list_labels_refuses_what_does_not_fit():
    n = capi.LIST_LABELS_MAX_KEYS
    seeds, ids = T(np.arange(n // 2)), T(np.arange(n // 2 + 1))
    with pytest.raises(capi.GsError, match="exceed"):
        capi.list_labels(seeds, ids, torch.zeros(n // 2 + 1, dtype=torch.int64, device=DEV))
