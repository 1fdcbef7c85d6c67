"""Operators that read a column slice without writing it: A[rows, cols] in one
pass over the parent matrix and the row sums of squared edge values of A[:, cols].
Checked against the CPU operators chained by hand (column slice, then row slice or
sum over the slice): what the reference computes through the intermediate slice
(src/cuda/fusion/column_row_slicing.cu:148-217, src/graph.cc:457-480)."""
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


def same(got, want):
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(g.cpu().numpy(), w)


def chained_col_row_slice(indptr, indices, cols, rows, key_offset=None):
    """Column slice, then row slice of it, select index mapped back to the parent."""
    sub_indptr, coo_col, sub_rows, sel = orc.col_slice(indptr, indices, cols)
    if key_offset is not None:
        sub_rows = sub_rows + np.asarray(key_offset)[coo_col]
    out_indptr, major, minor, kept = orc.minor_slice(sub_rows, rows, indptr=sub_indptr)
    return out_indptr, major, minor, sel[kept]


@pytest.mark.parametrize("ncol,nrow", [(0, 5), (1, 1), (7, 0), (300, 64), (2000, 512), (512, 5000)])
def test_col_row_slice_parity(ncol, nrow):
    rng = np.random.default_rng(ncol * 7 + nrow)
    indptr, indices = random_csc(rng, 3000, 5000, 50, hub_deg=40000)
    cols = rng.integers(0, 3000, size=ncol)                 # repeats allowed
    if ncol > 5:
        cols[2] = int(np.argmax(np.diff(indptr)))           # the hub column
        cols[3] = cols[4]
    rows = rng.integers(0, 5200, size=nrow)                 # repeats and absent ids
    want = chained_col_row_slice(indptr, indices, cols, rows)
    same(capi.col_row_slice(T(indptr), T(indices), T(cols), T(rows)), want)
    # the row ids read from a 32-bit copy
    same(capi.col_row_slice(T(indptr), T(indices), T(cols), T(rows),
                            indices32=T(indices).to(torch.int32)), want)
    got = capi.col_row_slice(T(indptr), T(indices), T(cols), T(rows), with_major=False)
    assert got[1] is None
    same((got[0], got[2], got[3]), (want[0], want[2], want[3]))


def test_col_row_slice_of_long_columns():
    """Columns far longer than a work-group's run of edges (the layer-wise
    sampler's case), columns without edges in between, a column id outside the
    matrix (degree 0)."""
    rng = np.random.default_rng(11)
    deg = np.zeros(400, dtype=np.int64)
    deg[rng.choice(400, size=40, replace=False)] = rng.integers(20_000, 90_000, size=40)
    indptr = np.concatenate([[0], np.cumsum(deg)])
    indices = rng.integers(0, 100_000, size=int(deg.sum()))
    cols = np.concatenate([rng.integers(0, 400, size=300), [400, -1, 399]])
    rows = rng.choice(100_000, size=512, replace=False)
    same(capi.col_row_slice(T(indptr), T(indices), T(cols), T(rows)),
         chained_col_row_slice(indptr, indices, cols, rows))


def test_col_row_slice_with_per_column_key_offsets():
    """Mini-batches of a super-batch: the row ids of batch b's columns and its picked rows
    are both moved by b * stride, so a row only matches inside its own batch; ids beyond
    32 bits take the confirming look-ups."""
    rng = np.random.default_rng(5)
    indptr, indices = random_csc(rng, 2000, 3000, 40, hub_deg=9000)
    for stride in (3000, 2**33):
        col_ptr = np.array([0, 100, 100, 350, 600])
        cols = rng.integers(0, 2000, size=600)
        batch_of_col = np.repeat(np.arange(4), np.diff(col_ptr))
        key_offset = batch_of_col * stride
        picked = np.concatenate([rng.choice(3000, size=80, replace=False) + b * stride
                                 for b in range(4)])
        want = chained_col_row_slice(indptr, indices, cols, picked, key_offset)
        same(capi.col_row_slice(T(indptr), T(indices), T(cols), T(picked), T(key_offset)), want)
        same(capi.col_row_slice(T(indptr), T(indices), T(cols), T(picked), T(key_offset),
                                indices32=T(indices).to(torch.int32)), want)


@pytest.mark.parametrize("ncol,num_rows", [(0, 100), (3, 5000), (600, 5200), (512, 100_000)])
@pytest.mark.parametrize("use_workspace", [True, False])
def test_sliced_e_square_sum_parity(ncol, num_rows, use_workspace):
    """Row sums of w^2 over A[:, cols] against float64 sums over the written slice; the
    last case is long enough (2.8 M edges) for the sorting path when a workspace is given."""
    rng = np.random.default_rng(ncol + num_rows)
    if num_rows == 100_000:
        deg = rng.integers(3000, 8000, size=700)
        indptr = np.concatenate([[0], np.cumsum(deg)])
        indices = rng.integers(0, num_rows, size=int(deg.sum()))
        cols = rng.integers(0, 700, size=ncol)
    else:
        indptr, indices = random_csc(rng, 3000, 5000, 50, hub_deg=40000)
        cols = rng.integers(0, 3000, size=ncol)
        if ncol > 5:
            cols[1] = int(np.argmax(np.diff(indptr)))
    w = (rng.random(indices.size) + 0.05).astype(np.float32)
    _, _, sub_rows, sel = orc.col_slice(indptr, indices, cols)
    want = np.zeros(num_rows)
    ok = sub_rows < num_rows                                 # ids outside the output are skipped
    np.add.at(want, sub_rows[ok], w[sel][ok].astype(np.float64) ** 2)
    got = capi.sliced_e_square_sum(T(indptr), T(indices), T(cols),
                                   torch.as_tensor(w, device=DEV), num_rows,
                                   use_workspace=use_workspace).cpu().numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-30)
    got32 = capi.sliced_e_square_sum(T(indptr), T(indices), T(cols),
                                     torch.as_tensor(w, device=DEV), num_rows,
                                     use_workspace=use_workspace,
                                     indices32=T(indices).to(torch.int32)).cpu().numpy()
    assert np.allclose(got32, want, rtol=1e-5, atol=1e-30)
    # and the CPU operator over the written slice agrees with the same sums
    cpu = orc.e_square_sum(("coo", sub_rows[ok], np.zeros(int(ok.sum()), dtype=np.int64)),
                           w[sel][ok], 2, num_rows)
    assert np.allclose(cpu, want, rtol=1e-5, atol=1e-30)
