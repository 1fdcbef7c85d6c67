"""Oracle unique/relabel against NumPy first-occurrence closed forms."""
import numpy as np
import pytest

from oracle import binding as orc
from tests import numpy_ref as ref


def test_single_batch_matches_numpy(rng):
    seeds = rng.permutation(500)[:100]
    rows = rng.integers(0, 500, size=3000)
    edge_col = rng.integers(0, 100, size=3000)
    uniq, uptr, out_row, out_col = orc.unique_relabel(seeds, rows, edge_col=edge_col)
    want = ref.first_occurrence_unique(np.concatenate([seeds, rows]))
    assert np.array_equal(uniq, want)
    assert uptr.tolist() == [0, want.size]
    assert np.array_equal(uniq[:100], seeds)          # distinct seeds lead the frontier
    assert np.array_equal(out_row, ref.relabel(want, rows))
    assert np.array_equal(out_col, edge_col)          # distinct seeds -> identity


def test_duplicate_seeds_map_to_first_copy():
    seeds = np.array([9, 4, 9, 7, 4])
    rows = np.array([7, 1, 9, 1])
    edge_col = np.array([0, 2, 4, 3])
    uniq, uptr, out_row, out_col = orc.unique_relabel(seeds, rows, edge_col=edge_col)
    assert uniq.tolist() == [9, 4, 7, 1]
    assert out_row.tolist() == [2, 3, 0, 3]
    assert out_col.tolist() == [0, 0, 1, 2]


def test_batches_are_independent(rng):
    B = 6
    s_sizes = rng.integers(0, 40, size=B); s_sizes[2] = 0
    r_sizes = rng.integers(0, 400, size=B); r_sizes[4] = 0
    sp = np.concatenate([[0], np.cumsum(s_sizes)])
    rp = np.concatenate([[0], np.cumsum(r_sizes)])
    seeds = rng.integers(0, 300, size=sp[-1])
    rows = rng.integers(0, 300, size=rp[-1])
    edge_col = np.concatenate([rng.integers(sp[b], max(sp[b + 1], sp[b] + 1), size=r_sizes[b])
                               if s_sizes[b] else np.zeros(0, dtype=np.int64)
                               for b in range(B)]).astype(np.int64)
    # batches without seeds cannot have edges pointing at a seed
    for b in range(B):
        if s_sizes[b] == 0:
            rows = np.delete(rows, slice(rp[b], rp[b + 1])); r_sizes[b] = 0
            rp = np.concatenate([[0], np.cumsum(r_sizes)])
    uniq, uptr, out_row, out_col = orc.unique_relabel(seeds, rows, sp, rp, edge_col)
    for b in range(B):
        keys = np.concatenate([seeds[sp[b]:sp[b + 1]], rows[rp[b]:rp[b + 1]]])
        want = ref.first_occurrence_unique(keys) if keys.size else keys
        assert np.array_equal(uniq[uptr[b]:uptr[b + 1]], want)
        assert np.array_equal(out_row[rp[b]:rp[b + 1]], ref.relabel(want, rows[rp[b]:rp[b + 1]]))
        assert np.array_equal(out_col[rp[b]:rp[b + 1]],
                              ref.relabel(want, seeds[edge_col[rp[b]:rp[b + 1]]]))


def test_empty_inputs():
    e = np.empty(0, dtype=np.int64)
    uniq, uptr, out_row, out_col = orc.unique_relabel(e, e)
    assert uniq.size == 0 and uptr.tolist() == [0, 0]
    uniq, uptr, out_row, _ = orc.unique_relabel(e, np.array([3, 3, 2]))
    assert uniq.tolist() == [3, 2] and out_row.tolist() == [0, 0, 1]
