"""HIP kernels vs the CPU oracle on the same seeded inputs, called through the
C ABI.  Integer / index work: bit-exact."""
import numpy as np
import pytest
import torch

from gsampler_amd import capi
from oracle import binding as orc
from tests.conftest import random_csc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return None if a is None else torch.as_tensor(np.asarray(a, dtype=np.int64), device=DEV)


def N(t):
    return None if t is None else t.cpu().numpy()


def assert_same(got, want):
    assert len(got) == len(want)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(N(g), w)


@pytest.mark.parametrize("n", [0, 1, 255, 256, 2048, 2049, 1 << 20, (1 << 22) + 3, (1 << 23) + 4099])
def test_scan(n):
    rng = np.random.default_rng(n)
    x = rng.integers(0, 1000, size=n)
    assert np.array_equal(N(capi.exclusive_scan(T(x))), np.cumsum(x) - x)


def test_reference_known_answers():
    indptr, indices = np.arange(21) * 5, np.arange(100)
    s, c, i, sel = capi.col_slice(T(indptr), T(indices), T([0, 1, 2]))
    assert N(s).tolist() == [0, 5, 10, 15] and N(i).tolist() == list(range(15))
    # K > deg, no replace -> identity (tests/test_colwise_sampling.cc test1)
    s, c, i, sel = capi.sample_uniform(T(indptr), T(indices), None, 6, False)
    assert np.array_equal(N(s), indptr) and np.array_equal(N(i), indices)
    for fanout in (6, 4):  # test2 / test3
        s, c, i, sel = capi.sample_uniform(T(indptr), T(indices), None, fanout, True)
        assert np.array_equal(N(s), np.arange(21) * fanout)
        assert np.array_equal(N(sel) // 5, np.repeat(np.arange(20), fanout))


@pytest.mark.parametrize("seed", range(3))
def test_col_slice_parity(seed):
    rng = np.random.default_rng(seed)
    indptr, indices = random_csc(rng, 3000, 10**5, 60, hub_deg=50000)
    cols = rng.integers(-2, 3003, size=2500)  # a few out-of-range ids
    assert_same(capi.col_slice(T(indptr), T(indices), T(cols)),
                orc.col_slice(indptr, indices, cols))
    ptr = np.array([0, 100, 100, 1700, 2500])
    assert_same(capi.col_slice(T(indptr), T(indices), T(cols), batch_ptr=T(ptr),
                               encode_stride=10**5),
                orc.col_slice(indptr, indices, cols, batch_ptr=ptr, encode_stride=10**5))
    e = np.empty(0, dtype=np.int64)
    assert_same(capi.col_slice(T(indptr), T(indices), T(e)), orc.col_slice(indptr, indices, e))


@pytest.mark.parametrize("algo", [capi.ALGO_AUTO, capi.ALGO_RESERVOIR, capi.ALGO_FLOYD])
@pytest.mark.parametrize("fanout", [1, 5, 8, 10, 15, 16, 25, 33, 64])
def test_sample_uniform_parity(algo, fanout):
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 5000, 10**6, 90, hub_deg=20000)
    cols = rng.integers(0, 5000, size=4097)
    narrow = T(indices).to(torch.int32)      # the int32 copy of the row ids: same outputs
    for call_id in (0, 3):
        want = orc.sample_uniform(indptr, indices, cols, fanout, False, algo,
                                  seed=7777, call_id=call_id)
        for ids in (T(indices), narrow):
            assert_same(capi.sample_uniform(T(indptr), ids, T(cols), fanout, False, algo,
                                            seed=7777, call_id=call_id), want)


@pytest.mark.parametrize("fanout", [3, 20, 100])
def test_sample_replace_and_unfused_parity(fanout):
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 2000, 10**6, 50, hub_deg=3000)
    cols = rng.integers(0, 2000, size=1500)
    assert_same(capi.sample_uniform(T(indptr), T(indices), T(cols), fanout, True),
                orc.sample_uniform(indptr, indices, cols, fanout, True))
    assert_same(capi.sample_uniform(T(indptr), T(indices).to(torch.int32), T(cols), fanout, True),
                orc.sample_uniform(indptr, indices, cols, fanout, True))
    # column_ids = None: sample the matrix's own columns (un-fused Sampling)
    for replace in (False, True):
        assert_same(capi.sample_uniform(T(indptr), T(indices), None, fanout, replace),
                    orc.sample_uniform(indptr, indices, None, fanout, replace))
    # reservoir with fanout > 64 (the AUTO choice there)
    assert_same(capi.sample_uniform(T(indptr), T(indices), T(cols), 100, False),
                orc.sample_uniform(indptr, indices, cols, 100, False))


@pytest.mark.parametrize("dtype", [torch.float32, torch.int64, torch.float64, torch.int32])
def test_col_slice_values_equal_a_gather_by_the_edge_positions(dtype):
    """Edge data of A[:, cols] copied by column runs of the parent's array is what
    indexing the data with the slice's edge positions gives (the positions are the
    oracle-checked output of the column slice)."""
    rng = np.random.default_rng(3)
    indptr, indices = random_csc(rng, 4000, 3000, 60, hub_deg=30000)
    nnz = int(indptr[-1])
    data = torch.as_tensor(rng.integers(0, 1 << 20, size=nnz), device=DEV).to(dtype)
    for cols in (rng.integers(0, 4000, size=700), np.arange(4000), np.empty(0, dtype=np.int64),
                 np.full(5, int(np.argmax(np.diff(indptr))))):      # repeats of the hub column
        sub_indptr, _, _, sel = capi.col_slice(T(indptr), T(indices), T(cols))
        want = orc.col_slice(indptr, indices, cols)
        assert np.array_equal(N(sel), want[3])
        got = capi.col_slice_values(T(indptr), T(cols), sub_indptr, data)
        assert torch.equal(got, data[sel])
    whole = capi.col_slice_values(T(indptr), None, T(indptr), data)   # every column, in order
    assert torch.equal(whole, data)
    with pytest.raises(capi.GsError, match="4 or 8 bytes"):
        capi.col_slice_values(T(indptr), None, T(indptr), data.to(torch.float16))


def _batched_case(rng, B, max_seeds, max_rows, id_range):
    s_sizes = rng.integers(1, max_seeds, size=B)
    r_sizes = rng.integers(0, max_rows, size=B)
    r_sizes[B // 2] = 0
    sp = np.concatenate([[0], np.cumsum(s_sizes)])
    rp = np.concatenate([[0], np.cumsum(r_sizes)])
    seeds = rng.integers(0, id_range, size=sp[-1])
    rows = rng.integers(0, id_range, size=rp[-1])
    edge_col = np.concatenate(
        [rng.integers(sp[b], sp[b + 1], size=r_sizes[b]) for b in range(B)]).astype(np.int64)
    return seeds, rows, sp, rp, edge_col


@pytest.mark.parametrize("id_range", [50, 5000, 2**32 - 2])
def test_unique_relabel_single_parity(id_range):
    rng = np.random.default_rng(1)
    seeds = rng.integers(0, id_range, size=777)
    rows = rng.integers(0, id_range, size=50000)
    if id_range > 10**6:
        rows[:5] = id_range  # the largest admissible key
    edge_col = rng.integers(0, 777, size=50000)
    assert_same(capi.unique_relabel(T(seeds), T(rows), edge_col=T(edge_col)),
                orc.unique_relabel(seeds, rows, edge_col=edge_col))
    # no seeds / no rows / nothing
    e = np.empty(0, dtype=np.int64)
    assert_same(capi.unique_relabel(T(e), T(rows)), orc.unique_relabel(e, rows))
    assert_same(capi.unique_relabel(T(seeds), T(e)), orc.unique_relabel(seeds, e))
    assert_same(capi.unique_relabel(T(e), T(e)), orc.unique_relabel(e, e))


@pytest.mark.parametrize("B,id_range", [(2, 100), (7, 3000), (64, 10**5)])
def test_unique_relabel_batched_parity(B, id_range):
    rng = np.random.default_rng(B)
    seeds, rows, sp, rp, edge_col = _batched_case(rng, B, 300, 6000, id_range)
    assert_same(capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), T(edge_col)),
                orc.unique_relabel(seeds, rows, sp, rp, edge_col))


def test_unique_relabel_hubs_and_ragged_batches():
    """A few ids that repeat thousands of times (buckets far above the average
    size), batches from empty to tens of thousands of keys."""
    rng = np.random.default_rng(11)
    r_sizes = np.array([0, 1, 40000, 3, 0, 25000, 9000, 2, 60000, 0, 500])
    B = r_sizes.size
    s_sizes = rng.integers(1, 50, size=B)
    s_sizes[4] = 0                      # a batch with nothing at all
    sp = np.concatenate([[0], np.cumsum(s_sizes)])
    rp = np.concatenate([[0], np.cumsum(r_sizes)])
    seeds = rng.integers(0, 10**6, size=sp[-1])
    rows = rng.integers(0, 10**6, size=rp[-1])
    hub = rng.random(rows.size) < 0.5
    rows[hub] = rng.choice([7, 123456, 999999], size=int(hub.sum()))
    edge_col = np.concatenate(
        [rng.integers(sp[b], max(sp[b + 1], sp[b] + 1), size=r_sizes[b]) for b in range(B)]
    ).astype(np.int64)
    edge_col = np.minimum(edge_col, max(sp[-1] - 1, 0))
    assert_same(capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), T(edge_col)),
                orc.unique_relabel(seeds, rows, sp, rp, edge_col))


@pytest.mark.parametrize("B", [1, 3])
def test_unique_relabel_buckets_beyond_their_regions(B):
    """The partition pass gives every bucket a region of at most 8192 entries.  Ids
    that repeat 9000 to 150000 times in one batch run over it (several buckets of
    one batch at once), next to a million ordinary keys; a last batch is all one id."""
    rng = np.random.default_rng(40 + B)
    n_r = 1_200_000
    rows = rng.integers(0, 10**6, size=n_r)
    for hub, times in [(3, 9000), (77777, 30000), (999_999, 150000), (5, 8193), (123, 8192)]:
        rows[rng.choice(n_r, size=times, replace=False)] = hub
    seeds = rng.integers(0, 10**6, size=500 * B)
    sp = rp = None
    if B > 1:
        rows = np.concatenate([rows, np.full(20000, 42), rng.integers(0, 300, size=100000)])
        sp = np.arange(B + 1) * 500
        rp = np.array([0, n_r, n_r + 20000, rows.size])
        edge_col = np.concatenate([rng.integers(sp[b], sp[b + 1], size=rp[b + 1] - rp[b])
                                   for b in range(B)]).astype(np.int64)
    else:
        edge_col = rng.integers(0, seeds.size, size=rows.size)
    got = capi.unique_relabel(T(seeds), T(rows), T(sp) if B > 1 else None,
                              T(rp) if B > 1 else None, T(edge_col))
    assert_same(got, orc.unique_relabel(seeds, rows, sp, rp, edge_col))
    if B == 1:
        keys = np.concatenate([seeds, rows])
        _, idx = np.unique(keys, return_index=True)
        assert np.array_equal(N(got[0]), keys[np.sort(idx)])


@pytest.mark.parametrize("by_pointer", [False, True])
def test_unique_frontier_and_labels_from_one_launch(by_pointer):
    """gs_unique_fill_relabel writes what gs_unique_fill and gs_unique_relabel write."""
    rng = np.random.default_rng(77)
    counts = rng.integers(0, 9, size=30000)
    seeds, rows, sp, rp, edge_col, col_indptr = _grouped_case(rng, counts, 16, 10**5)
    how = dict(col_indptr=T(col_indptr)) if by_pointer else dict(edge_col=T(edge_col))
    one = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), fused=True, **how)
    two = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), fused=False, **how)
    assert_same(one, tuple(None if x is None else N(x) for x in two))
    assert_same(one, orc.unique_relabel(seeds, rows, sp, rp, edge_col))
    # rows only / no edges at all
    one = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), want_col=False, fused=True)
    assert_same(one, orc.unique_relabel(seeds, rows, sp, rp))
    e = np.empty(0, dtype=np.int64)
    assert_same(capi.unique_relabel(T(seeds[:50]), T(e), edge_col=T(e), fused=True),
                orc.unique_relabel(seeds[:50], e, edge_col=e))


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("fanout", [5, 70])
def test_samplers_write_the_place_of_a_column_inside_its_batch(weighted, fanout):
    """With the offsets of the batches of its columns a sampler stores, for every edge,
    its column's place inside the batch (the packed, the strided and the weighted
    kernels); without them the column's place in the call."""
    rng = np.random.default_rng(fanout + weighted)
    indptr, indices = random_csc(rng, 3000, 10**5, 40, hub_deg=4000)
    cols = rng.integers(0, 3000, size=900)
    ptr = np.array([0, 1, 1, 300, 640, 900])
    if weighted:
        probs = rng.random(indices.size).astype(np.float32)
        k = min(fanout, 64)
        cdf = capi.weight_cdf(T(indptr), torch.as_tensor(probs, device=DEV), T(indices), 3000)
        plain = capi.sample_weighted(T(indptr), T(indices), None, T(cols), k, cdf=cdf, call_id=3)
        local = capi.sample_weighted(T(indptr), T(indices), None, T(cols), k, cdf=cdf, call_id=3,
                                     col_batch_ptr=T(ptr))
    else:
        plain = capi.sample_uniform(T(indptr), T(indices), T(cols), fanout, call_id=3)
        local = capi.sample_uniform(T(indptr), T(indices), T(cols), fanout, call_id=3,
                                    col_batch_ptr=T(ptr))
    for a, b in zip((plain[0], plain[2], plain[3]), (local[0], local[2], local[3])):
        assert torch.equal(a, b)
    col = N(plain[1])
    batch = np.searchsorted(ptr, col, side="right") - 1
    assert np.array_equal(N(local[1]), col - ptr[batch])


@pytest.mark.parametrize("repeat_seeds_in", [(), (2,), (0, 1, 2, 3)])
def test_unique_relabel_with_column_labels_from_the_sampler(repeat_seeds_in):
    """out_col handed in with every column's place inside its batch: batches with
    distinct seeds keep it, batches in which a seed repeats are rewritten -- the
    result is what the pass computes on its own, and what the oracle computes."""
    rng = np.random.default_rng(len(repeat_seeds_in))
    counts = rng.integers(0, 7, size=6000)
    seeds, rows, sp, rp, edge_col, col_indptr = _grouped_case(rng, counts, 4, 10**5)
    for b in repeat_seeds_in:                       # a repeated seed: labels are no longer places
        if sp[b + 1] - sp[b] >= 2:
            seeds[sp[b + 1] - 1] = seeds[sp[b]]
    batch = np.searchsorted(sp, edge_col, side="right") - 1
    places = edge_col - sp[batch]
    own = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), col_indptr=T(col_indptr))
    for fused in (True, False):
        handed = T(places.copy())
        got = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), col_indptr=T(col_indptr),
                                  out_col=handed, fused=fused)
        assert got[3].data_ptr() == handed.data_ptr()            # written in place
        assert_same(got, tuple(N(x) for x in own))
    assert_same(own, orc.unique_relabel(seeds, rows, sp, rp, edge_col))


def _grouped_case(rng, counts, B, id_range):
    """Edges grouped by seed position: counts[c] edges for seed c, B batches of seeds."""
    S = counts.size
    col_indptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    cuts = np.sort(rng.integers(0, S + 1, size=B - 1)) if B > 1 else np.empty(0, np.int64)
    sp = np.concatenate([[0], cuts, [S]]).astype(np.int64)
    rp = col_indptr[sp]
    seeds = rng.permutation(id_range)[:S] if id_range >= S else rng.integers(0, id_range, size=S)
    rows = rng.integers(0, id_range, size=int(col_indptr[-1]))
    edge_col = np.repeat(np.arange(S, dtype=np.int64), counts)
    return seeds.astype(np.int64), rows, sp, rp, edge_col, col_indptr


@pytest.mark.parametrize("shape", ["ragged", "fives", "gaps", "giant", "exact_tiles", "one_edge",
                                   "repeated_seeds"])
@pytest.mark.parametrize("B", [1, 7, 64])
def test_unique_relabel_by_column_pointer(shape, B):
    """The column of an edge read off the column pointer of a matrix compressed by
    column gives the labels that an explicit column per edge gives."""
    rng = np.random.default_rng(sum(shape.encode()) * 100 + B)
    id_range = 10**5
    if shape == "ragged":
        counts = rng.integers(0, 11, size=5000)
    elif shape == "fives":
        counts = np.full(6000, 5)
    elif shape == "gaps":      # long runs of empty columns, also at both ends and across tiles
        counts = np.zeros(20000, dtype=np.int64)
        counts[[4000, 4001, 9000, 15000, 15002]] = [3000, 1, 2047, 1, 5000]
    elif shape == "giant":     # one column over many tiles
        counts = rng.integers(0, 4, size=3000)
        counts[1500] = 50000
    elif shape == "exact_tiles":
        counts = np.full(1024, 4)
    elif shape == "one_edge":
        counts = np.zeros(300, dtype=np.int64)
        counts[299] = 1
    else:                      # seeds that repeat: labels go through the first occurrence
        counts = rng.integers(0, 6, size=4000)
        id_range = 500
    seeds, rows, sp, rp, edge_col, col_indptr = _grouped_case(rng, counts, B, id_range)
    bp = (T(sp), T(rp)) if B > 1 else (None, None)
    got = capi.unique_relabel(T(seeds), T(rows), *bp, col_indptr=T(col_indptr))
    assert_same(got, orc.unique_relabel(seeds, rows, sp if B > 1 else None,
                                        rp if B > 1 else None, edge_col))
    other = capi.unique_relabel(T(seeds), T(rows), *bp, edge_col=T(edge_col))
    assert_same(got, tuple(None if x is None else N(x) for x in other))


def test_unique_relabel_column_arguments_are_checked():
    seeds, rows = T(np.arange(4)), T(np.arange(8))
    with pytest.raises(ValueError, match="not both"):
        capi.unique_relabel(seeds, rows, edge_col=T(np.zeros(8, np.int64)),
                            col_indptr=T(np.array([0, 2, 4, 6, 8])))
    with pytest.raises(ValueError, match="entries"):
        capi.unique_relabel(seeds, rows, col_indptr=T(np.array([0, 8])))


@pytest.mark.parametrize("B", [1023, 1024, 1025, 3000])
def test_unique_relabel_many_tiny_batches(B):
    """Around 1024 batches the batch walk moves from every work-group's LDS to a launch
    of its own."""
    rng = np.random.default_rng(12)
    s_sizes = rng.integers(0, 3, size=B)
    r_sizes = rng.integers(0, 6, size=B)
    sp = np.concatenate([[0], np.cumsum(s_sizes)])
    rp = np.concatenate([[0], np.cumsum(r_sizes)])
    seeds = rng.integers(0, 20, size=sp[-1])
    rows = rng.integers(0, 20, size=rp[-1])
    assert_same(capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp)),
                orc.unique_relabel(seeds, rows, sp, rp))


def test_unique_relabel_one_huge_batch():
    """More keys in one batch than its buckets can take at the usual size: every
    bucket is deduplicated in global memory."""
    rng = np.random.default_rng(13)
    seeds = rng.integers(0, 3 * 10**6, size=1000)
    rows = rng.integers(0, 3 * 10**6, size=7 * 10**6)
    edge_col = rng.integers(0, 1000, size=rows.size)
    assert_same(capi.unique_relabel(T(seeds), T(rows), edge_col=T(edge_col)),
                orc.unique_relabel(seeds, rows, edge_col=edge_col))


def test_graphsage_layers_end_to_end():
    """Three fused slice+sample + unique/relabel layers on an R-MAT graph, super-batch
    of 8, compared with the oracle layer by layer."""
    from gsampler_amd.utils import rmat_csc, batched_seeds
    indptr_t, indices_t = rmat_csc(20000, 400000, seed=1)
    seeds_t, ptr_t = batched_seeds(20000, 8, 128, seed=2)
    indptr, indices = indptr_t.numpy(), indices_t.numpy()
    seeds, ptr = seeds_t.numpy(), ptr_t.numpy()
    g_seeds, g_ptr = T(seeds), T(ptr)
    for layer, fanout in enumerate([15, 10, 5]):
        g = capi.sample_uniform(T(indptr), T(indices), g_seeds, fanout, call_id=layer)
        o = orc.sample_uniform(indptr, indices, seeds, fanout, call_id=layer)
        assert_same(g, o)
        g_eptr = g[0][g_ptr]
        o_eptr = o[0][ptr]
        gu = capi.unique_relabel(g_seeds, g[2], g_ptr, g_eptr, g[1])
        ou = orc.unique_relabel(seeds, o[2], ptr, o_eptr, o[1])
        assert_same(gu, ou)
        g_seeds, g_ptr = gu[0], gu[1]
        seeds, ptr = ou[0], ou[1]


def test_format_and_batch_helpers_parity():
    rng = np.random.default_rng(21)
    indptr, indices = random_csc(rng, 3000, 5000, 40, hub_deg=20000)
    assert np.array_equal(N(capi.csc2coo(T(indptr))), orc.csc2coo(indptr))
    assert capi.csc2coo(T(np.zeros(5, dtype=np.int64))).numel() == 0
    ids = np.sort(rng.integers(0, 777, size=100000))
    assert np.array_equal(N(capi.sorted_to_indptr(T(ids), 777)), orc.sorted_to_indptr(ids, 777))
    enc = rng.integers(0, 1000, size=5000) + rng.integers(0, 64, size=5000) * 1000
    for g, o in zip(capi.decode_batch_ids(T(enc), 1000), orc.decode_batch_ids(enc, 1000)):
        assert np.array_equal(N(g), o)
    offset = np.array([0, 100, 100, 1500, 3000])
    assert np.array_equal(N(capi.split_indptr(T(indptr), T(offset))),
                          orc.split_indptr(indptr, offset))


@pytest.mark.parametrize("B", [1, 5])
@pytest.mark.parametrize("shape", ["mixed", "tag_collisions", "hubs"])
def test_unique_relabel_with_ids_beyond_32_bits(B, shape):
    """Ids of 2^32 - 1 and above (up to 2^40, and negative ones) go through the
    same kernels; the packed entries then carry only a 32-bit tag and every tag
    match is confirmed against the keys themselves.  `tag_collisions`: many
    distinct ids that agree in their low 32 bits (and repeat), so that equal tags
    meet in one table; `hubs`: two wide ids that repeat tens of thousands of
    times (buckets beyond the LDS table's sure size)."""
    rng = np.random.default_rng(B + len(shape))
    n_s, n_r = 400 * B, 60000 * B
    if shape == "mixed":
        pool = np.concatenate([rng.integers(0, 1000, size=300),
                               rng.integers(2**32 - 3, 2**32 + 3, size=50),
                               rng.integers(2**32, 2**40, size=3000),
                               np.array([2**40, -5, -1, 2**32 - 1, 2**63 - 1])])
    elif shape == "tag_collisions":
        low = rng.integers(0, 40, size=4000)
        low[:10] = 2**32 - 1                       # the tag that has to be moved
        pool = low + rng.integers(0, 50, size=4000) * 2**32
    else:
        pool = np.concatenate([rng.integers(2**33, 2**34, size=20000),
                               np.full(30000, 2**35 + 7), np.full(30000, 2**35 + 7 + 2**32)])
    seeds = rng.choice(pool, size=n_s)
    rows = rng.choice(pool, size=n_r)
    sp = rp = None
    if B > 1:
        sp = np.arange(B + 1) * 400
        cuts = np.sort(rng.integers(0, n_r, size=B - 1))
        rp = np.concatenate([[0], cuts, [n_r]])
        edge_col = np.concatenate([rng.integers(sp[b], sp[b + 1], size=rp[b + 1] - rp[b])
                                   for b in range(B)]).astype(np.int64)
    else:
        edge_col = rng.integers(0, n_s, size=n_r)
    got = capi.unique_relabel(T(seeds), T(rows), T(sp) if B > 1 else None,
                              T(rp) if B > 1 else None, T(edge_col))
    want = orc.unique_relabel(seeds, rows, sp, rp, edge_col)
    assert_same(got, want)
    # independent closed form for one batch: first occurrences in order
    if B == 1:
        keys = np.concatenate([seeds, rows])
        _, idx = np.unique(keys, return_index=True)
        assert np.array_equal(N(got[0]), keys[np.sort(idx)])
    # narrow ids still work afterwards (the flag is per call)
    small = rng.integers(0, 500, size=5000)
    assert_same(capi.unique_relabel(T(small[:50]), T(small)), orc.unique_relabel(small[:50], small))


@pytest.mark.parametrize("num_ids", [1, 300, 4096, 5000])
def test_first_position(num_ids):
    rng = np.random.default_rng(num_ids)
    ids = rng.integers(0, num_ids + 3, size=200000)          # a few ids outside the range
    ids[rng.random(ids.size) < 0.3] = 0                      # one hot id
    if num_ids > 10:
        ids[ids == 7] = 8                                    # an id that never occurs
    got = capi.first_position(T(ids), num_ids).cpu().numpy()
    want = np.full(num_ids, np.iinfo(np.int64).max)
    inside = ids < num_ids
    np.minimum.at(want, ids[inside], np.nonzero(inside)[0])
    assert np.array_equal(got, want)
    empty = capi.first_position(T(np.empty(0, dtype=np.int64)), 4).cpu().tolist()
    assert empty == [np.iinfo(np.int64).max] * 4


@pytest.mark.parametrize("num_cols,nnz", [(1, 50), (300, 20000), (70000, 300000), (5, 0)])
def test_coo_to_csc_parity(num_cols, nnz):
    """Edge list -> CSC: stable sort over the id bits, indptr, gathers."""
    rng = np.random.default_rng(num_cols)
    col = rng.integers(0, num_cols, size=nnz)
    row = rng.integers(0, 1000, size=nnz)
    want = orc.coo_to_csc(row, col, num_cols)
    got = capi.coo_to_csc(T(row), T(col), num_cols)
    assert_same(got, want)


@pytest.mark.parametrize("n", [0, 1, 1023, 8190, 8191, 8192, 8193, 20000])
@pytest.mark.parametrize("fanout,replace", [(-1, False), (5, False), (3, True)])
def test_col_count_sizes_around_the_single_launch_path(n, fanout, replace):
    """Up to 8191 columns one work-group counts and scans in a single launch; beyond,
    tiles and a down sweep.  Both against the oracle, total in pinned host memory included."""
    rng = np.random.default_rng(n + 7)
    indptr, _ = random_csc(rng, 3000, 10**5, 30, hub_deg=5000)
    cols = rng.integers(-2, 3003, size=n)                   # a few ids outside the matrix
    count = capi._Count()
    got = capi.col_count(T(indptr), T(cols), fanout, replace, count=count)
    want = orc.col_count(indptr, cols, fanout, replace)
    assert np.array_equal(N(got), want)
    assert count.get() == want[-1]


def test_count_mirrors_in_pinned_host_memory():
    """The optional mirror arguments of the two count entry points: the kernel that
    computes the edge total / the per-batch offsets stores them to pinned host memory
    as well; with NULL nothing else changes."""
    rng = np.random.default_rng(21)
    indptr, indices = random_csc(rng, 4000, 10**5, 40, hub_deg=9000)
    cols = rng.integers(0, 4000, size=7000)
    l = capi.lib()
    d_indptr, d_cols = T(indptr), T(cols)
    n = cols.size
    ws = torch.empty(l.gs_scan_workspace_bytes(n + 1), dtype=torch.uint8, device=DEV)
    mirror = torch.full((4,), -7, dtype=torch.int64).pin_memory()
    outs = []
    for use_mirror in (True, False):
        sub = torch.empty(n + 1, dtype=torch.int64, device=DEV)
        capi.check(l.gs_csc_col_count(d_indptr.data_ptr(), indptr.size - 1, d_cols.data_ptr(), n, 5, 0,
                                      sub.data_ptr(), mirror.data_ptr() if use_mirror else None,
                                      None, ws.data_ptr(), ws.numel(), None))
        torch.cuda.synchronize()
        outs.append(sub.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    assert int(mirror[0]) == outs[0][-1] and mirror[1:].tolist() == [-7, -7, -7]
    want = orc.col_count(indptr, cols, 5, False)
    assert np.array_equal(outs[0], want)

    seeds, rows, sp, rp, _ = _batched_case(rng, 9, 50, 400, 300)
    B = sp.size - 1
    d = [T(x) for x in (seeds, rows, sp, rp)]
    uws = torch.empty(l.gs_unique_workspace_bytes(seeds.size, rows.size, B), dtype=torch.uint8, device=DEV)
    host = torch.full((B + 3,), -7, dtype=torch.int64).pin_memory()
    uptr = torch.empty(B + 1, dtype=torch.int64, device=DEV)
    capi.check(l.gs_unique_count(d[0].data_ptr(), d[2].data_ptr(), seeds.size, d[1].data_ptr(),
                                 d[3].data_ptr(), rows.size, B, uptr.data_ptr(), host.data_ptr(),
                                 uws.data_ptr(), uws.numel(), None))
    torch.cuda.synchronize()
    assert host[:B + 1].tolist() == uptr.cpu().tolist() and host[B + 1:].tolist() == [-7, -7]
    assert np.array_equal(uptr.cpu().numpy(), orc.unique_relabel(seeds, rows, sp, rp)[1])


def test_outputs_that_are_only_8_byte_aligned(monkeypatch):
    """The kernels that store 16 bytes per lane fall back to narrower stores when an
    output array does not allow it: every array the wrappers allocate here starts one
    element past a 16-byte boundary."""
    real_empty = torch.empty

    def shifted(*size, **kw):
        if len(size) == 1 and isinstance(size[0], int) and kw.get("dtype") in (torch.int64, torch.float32):
            return real_empty(size[0] + 1, **kw)[1:]
        return real_empty(*size, **kw)

    monkeypatch.setattr(torch, "empty", shifted)
    rng = np.random.default_rng(31)
    indptr, indices = random_csc(rng, 3000, 10**5, 60, hub_deg=50000)
    cols = rng.integers(0, 3000, size=2500)
    got = capi.col_slice(T(indptr), T(indices), T(cols))
    assert all(t.data_ptr() % 16 == 8 for t in got)
    assert_same(got, orc.col_slice(indptr, indices, cols))
    data = torch.as_tensor(rng.random(indices.size).astype(np.float32), device=DEV)
    vals = capi.col_slice_values(T(indptr), T(cols), got[0], data)
    assert vals.data_ptr() % 16 == 4 and torch.equal(vals, data[got[3]])
    x = rng.integers(0, 50, size=100001)
    assert np.array_equal(N(capi.exclusive_scan(T(x))), np.cumsum(x) - x)
    counts = rng.integers(0, 11, size=5000)
    counts[100] = 6000
    seeds, rows, sp, rp, edge_col, col_indptr = _grouped_case(rng, counts, 7, 10**5)
    want = orc.unique_relabel(seeds, rows, sp, rp, edge_col)
    by_pointer = capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), col_indptr=T(col_indptr))
    assert by_pointer[2].data_ptr() % 16 == 8 and by_pointer[3].data_ptr() % 16 == 8
    assert_same(by_pointer, want)
    assert_same(capi.unique_relabel(T(seeds), T(rows), T(sp), T(rp), edge_col=T(edge_col)), want)


@pytest.mark.parametrize("fanout,replace", [(5, False), (15, False), (3, True), (100, False)])
def test_samplers_read_column_spans_left_by_the_count_pass(fanout, replace):
    """The count pass can leave every column's start and degree in one word; the fill passes
    that take it give the picks they give from the column pointer (oracle included), for
    requested columns with repeats, empty columns and ids outside the matrix."""
    rng = np.random.default_rng(fanout)
    indptr, indices = random_csc(rng, 3000, 3000, 40)
    cols = rng.integers(-2, 3004, size=5000)
    args = (fanout, replace, 0, 11, 3)
    with_spans = capi.sample_uniform(T(indptr), T(indices), T(cols), *args, spans=True)
    without = capi.sample_uniform(T(indptr), T(indices), T(cols), *args, spans=False)
    want = orc.sample_uniform(indptr, indices, cols, *args)
    for a, b in zip(with_spans, without):
        assert torch.equal(a, b)
    assert_same(with_spans, want)
    if fanout <= 64:
        probs = rng.random(indices.size).astype(np.float32)
        cdf = capi.weight_cdf(T(indptr), torch.as_tensor(probs, device=DEV), T(indices), 3000)
        a = capi._sample_weighted_cdf(T(indptr), T(indices), cdf, T(cols), fanout, replace, 11, 3,
                                      True, spans=True)
        b = capi._sample_weighted_cdf(T(indptr), T(indices), cdf, T(cols), fanout, replace, 11, 3,
                                      True, spans=False)
        for x, y in zip(a, b):
            assert torch.equal(x, y)


def test_a_column_too_long_for_a_span_is_looked_up():
    """Degrees from 2^24 - 1 on do not fit a span word: the count pass writes the look-up mark
    and the fill pass reads the column pointer for that column, and only for it."""
    long_deg = (1 << 24) + 5
    indptr = np.array([0, 3, 3 + long_deg, 3 + long_deg + 4], dtype=np.int64)
    rng = np.random.default_rng(1)
    indices = rng.integers(0, 1000, size=int(indptr[-1]))
    cols = np.array([1, 0, 2, 1], dtype=np.int64)
    d_indptr, d_cols = T(indptr), T(cols)
    span = torch.empty(4, dtype=torch.int64, device=DEV)
    capi.col_count(d_indptr, d_cols, 5, False, col_span=span)
    assert span.cpu().tolist() == [-1, 3 << 40, (4 << 40) | (3 + long_deg), -1]
    got = capi.sample_uniform(d_indptr, T(indices), d_cols, 5, False, 0, 7, 1, spans=True)
    want = orc.sample_uniform(indptr, indices, cols, 5, False, 0, 7, 1)
    assert_same(got, want)
