"""Row ids of every column sorted (SortIndicesCUDA, src/cuda/sort_indices.cu:11-37):
the device kernels against numpy's sort of every segment, on shapes that reach each
of their paths -- short segments sorted in LDS tile by tile, long ones split by 11
bits of the ids once, twice or three times, bins that stay long because one id
repeats, segments of exactly the sizes where the paths change."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from gsampler_amd import capi  # noqa: E402


def T(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.int64, device="cuda:0")


def sorted_segments(indptr, keys):
    out = keys.copy()
    for c in range(indptr.size - 1):
        out[indptr[c]:indptr[c + 1]].sort()
    return out


def check(sizes, keys, bound):
    indptr = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    assert keys.size == indptr[-1]
    got = capi.segment_sort(T(indptr), T(keys), bound).cpu().numpy()
    assert np.array_equal(got, sorted_segments(indptr, keys))


@pytest.mark.parametrize("bits", [3, 11, 12, 22, 23, 32])
def test_short_and_long_segments_for_every_number_of_rounds(bits):
    """2^bits ids: one round of splitting up to 11 bits, two up to 22, three up to 32."""
    rng = np.random.default_rng(bits)
    sizes = np.concatenate([rng.integers(0, 40, size=3000), [2047, 2048, 2049, 0, 0, 4096, 4097, 1],
                            rng.integers(0, 3000, size=60), [70000, 5, 200000, 0]])
    rng.shuffle(sizes)
    keys = rng.integers(0, 2**bits, size=int(sizes.sum()))
    check(sizes, keys, 2**bits)
    if bits > 3:
        check(sizes, keys, 2**bits - 5 if bits < 32 else 2**32 - 1)   # a bound that is no power of two


def test_ids_that_repeat_keep_bins_long():
    """A hub column whose ids come from a power law: most of a split segment lands in
    one bin (the low ids), which is split again; single ids repeat tens of thousands of
    times, so some bins stay long until the last bits."""
    rng = np.random.default_rng(5)
    n_ids = 1 << 20
    sizes = np.array([300000, 10, 0, 2500, 150000, 1, 1, 5000])
    keys = np.minimum((rng.pareto(0.6, size=int(sizes.sum()))).astype(np.int64), n_ids - 1)
    check(sizes, keys, n_ids)
    check(sizes, np.full(int(sizes.sum()), 77777), n_ids)             # every id the same
    check(sizes, (n_ids - 1 - keys), n_ids)                           # mass at the top of the range


@pytest.mark.parametrize("shape", ["ones", "empties", "one_segment", "tile_edges"])
def test_segment_layouts_around_the_tile_windows(shape):
    rng = np.random.default_rng(len(shape))
    if shape == "ones":            # thousands of one-id segments in one window
        sizes = np.ones(10000, dtype=np.int64)
    elif shape == "empties":       # runs of empty segments, also first and last
        sizes = np.zeros(9000, dtype=np.int64)
        sizes[rng.choice(9000, size=400, replace=False)] = rng.integers(1, 600, size=400)
        sizes[0] = sizes[-1] = 0
    elif shape == "one_segment":
        sizes = np.array([123457])
    else:                          # segments that start at the last position of a window
        sizes = np.array([2047, 2048, 1, 2047, 2, 2048, 2048, 4095, 2049, 2047, 1])
    keys = rng.integers(0, 50000, size=int(sizes.sum()))
    check(sizes, keys, 50000)


def test_a_power_law_graph_at_size():
    from gsampler_amd.utils import chung_lu_csc
    indptr, indices = chung_lu_csc(300_000, 20_000_000, seed=4, device="cuda:0")
    got = capi.segment_sort(indptr, indices, 300_000)
    # sorted inside every column, and the same ids per column: sorting (column, id)
    # pairs as one word gives the same array
    col = capi.csc2coo(indptr, int(indices.numel()))
    want = torch.sort(col * 300_000 + indices).values - col * 300_000
    assert torch.equal(got, want)
