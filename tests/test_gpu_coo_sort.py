"""Stable sort of edge positions by column id (COOSort, src/cuda/format_transform.cu:65-84):
the device kernels against numpy's stable argsort, on id ranges that take one to four
passes of 8 bits, on sizes around the 8192-edge tiles, and on ids that all meet in
a few digit values.  capi.coo_sort raises when the sort's gave-up flag is set."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from gsampler_amd import capi  # noqa: E402


def T(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.int64, device="cuda:0")


def check(ids, num_ids):
    ids = np.asarray(ids, dtype=np.int64)
    out, perm = capi.coo_sort(T(ids), num_ids)
    want = np.argsort(ids, kind="stable")
    assert np.array_equal(perm.cpu().numpy(), want)
    assert np.array_equal(out.cpu().numpy(), ids[want])


@pytest.mark.parametrize("bits", [1, 5, 8, 9, 16, 17, 22, 24, 25, 32])
@pytest.mark.parametrize("n", [1, 63, 8191, 8192, 8193, 100_000])
def test_every_number_of_passes_and_sizes_around_a_tile(bits, n):
    rng = np.random.default_rng(bits * 1000 + n % 997)
    check(rng.integers(0, 2**bits, size=n), 2**bits)


def test_bound_that_is_no_power_of_two_and_empty_input():
    rng = np.random.default_rng(5)
    check(rng.integers(0, 2_450_000, size=300_000), 2_450_000)
    check(rng.integers(0, 3, size=50_000), 3)
    check(np.zeros(0, dtype=np.int64), 10)
    check(np.zeros(20_000, dtype=np.int64), 1)


@pytest.mark.parametrize("num_ids", [2_000, 3_000_000])
def test_many_tiles_with_ids_of_a_power_law(num_ids):
    """Two million edges (245 tiles): most ids are small, so a few digit values of the
    upper pass hold most edges, and every tile waits for the counts of the ones before."""
    rng = np.random.default_rng(num_ids)
    ids = np.minimum((num_ids * rng.random(2_000_000) ** 4).astype(np.int64), num_ids - 1)
    check(ids, num_ids)


def test_one_id_and_two_alternating_ids_over_many_tiles():
    check(np.full(500_000, 1234567), 2_000_000)
    check(np.tile(np.array([255, 256]), 300_000), 5000)
    check(np.arange(400_000)[::-1] % 70_000, 70_000)


def test_back_to_back_calls_share_nothing():
    """Two sorts in a row on one stream, workspaces from the same allocator."""
    rng = np.random.default_rng(11)
    a = rng.integers(0, 50_000, size=200_000)
    b = rng.integers(0, 50_000, size=150_000)
    ra = capi.coo_sort(T(a), 50_000)
    rb = capi.coo_sort(T(b), 50_000)
    assert np.array_equal(ra[1].cpu().numpy(), np.argsort(a, kind="stable"))
    assert np.array_equal(rb[1].cpu().numpy(), np.argsort(b, kind="stable"))


def test_wider_ids_and_the_flag_offset():
    """Ids beyond 32 bits go through the radix sort of the library this one replaces for
    narrower ids; the two agree, and only the native path has a gave-up flag."""
    rng = np.random.default_rng(3)
    ids = rng.integers(0, 5000, size=100_000)
    a = capi.coo_sort(T(ids), 5000)
    b = capi.coo_sort(T(ids), 1 << 40)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert capi.lib().gs_coo_sort_flag_offset(100_000, 5000) == 0
    assert capi.lib().gs_coo_sort_flag_offset(100_000, 1 << 40) == -1
    assert capi.lib().gs_coo_sort_flag_offset(1 << 32, 5000) == -1
