"""Row slicing across the compressed axis / COO slicing on the GPU vs the oracle
(bit-exact), plus the reference's row-slicing known answer through the API."""
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


def same(got, want):
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            assert np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("npick", [0, 1, 50, 4000])
def test_minor_slice_parity(npick):
    rng = np.random.default_rng(npick)
    indptr, indices = random_csc(rng, 3000, 5000, 50, hub_deg=40000)
    col = np.repeat(np.arange(3000), np.diff(indptr))
    picked = rng.integers(0, 5200, size=npick)  # repeats and absent ids
    same(capi.minor_slice(T(indices), T(picked), indptr=T(indptr)),
         orc.minor_slice(indices, picked, indptr=indptr))
    same(capi.minor_slice(T(indices), T(picked), edge_major=T(col)),
         orc.minor_slice(indices, picked, edge_major=col))
    same(capi.minor_slice(T(indices), T(picked), indptr=T(indptr), with_major=False),
         orc.minor_slice(indices, picked, indptr=indptr, with_major=False))


def test_reference_rowwise_slicing_through_the_api():
    # tests/test_rowwise_slicing.cc:7-24
    indptr = torch.cat([torch.zeros(10, dtype=torch.int64), torch.arange(3) * 2]).to(DEV)
    indices = torch.arange(5, 7).repeat(2).to(DEV)
    A = gs.Graph(12, 12)
    A._CAPI_LoadCSC(indptr, indices)
    sub, sel = A._CAPI_Slicing(torch.tensor([5], device=DEV), 0, gs._CSR, gs._CSR)
    assert sub._CAPI_GetCSRIndptr().numel() == 2
    assert sub._CAPI_GetCSRIndices().tolist() == [10, 11]
    # the same slice taken directly on the CSC (no CSR built)
    sub2, sel2 = A._CAPI_Slicing(torch.tensor([5], device=DEV), 0, gs._CSC, gs._CSC | gs._COO)
    assert sub2._CAPI_GetCOOCols().tolist() == [10, 11]
    assert sub2._CAPI_GetCOORows().tolist() == [0, 0]
    assert sub2._CAPI_GetNumRows() == 1 and sub2._CAPI_GetNumCols() == 12
    assert sel2.tolist() == [0, 2]


def test_matrix_row_and_column_slicing_with_edata():
    rng = np.random.default_rng(3)
    indptr, indices = random_csc(rng, 400, 300, 30)
    indices[0] = 299
    col = np.repeat(np.arange(400), np.diff(indptr))
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    w = rng.random(indices.size, dtype=np.float32)
    m.edata["w"] = torch.as_tensor(w, device=DEV)
    cols = rng.permutation(400)[:64]
    rows = rng.permutation(300)[:80]
    sub = m[T(rows), T(cols)]
    r, c, _ = sub.coo
    r, c = r.cpu().numpy(), c.cpu().numpy()
    # closed form: edges (row, col) with col in cols and row in rows
    cpos = {int(v): i for i, v in enumerate(cols)}
    rpos = {int(v): i for i, v in enumerate(rows)}
    want = sorted((rpos[int(a)], cpos[int(b)], float(x))
                  for a, b, x in zip(indices, col, w) if int(a) in rpos and int(b) in cpos)
    got = sorted(zip(r.tolist(), c.tolist(), sub.edata["w"].cpu().numpy().tolist()))
    assert got == want
    assert sub.num_rows() == 80 and sub.num_cols() == 64
    assert torch.equal(sub.row_ndata["_ID"].cpu(), torch.as_tensor(rows))
    # COO slicing operator
    g = m._graph
    subc, sel = g._CAPI_Slicing(T(rows), 0, gs._COO, gs._COO)
    mask = np.isin(indices, rows)
    assert np.array_equal(sel.cpu().numpy(), np.nonzero(mask)[0])
    assert np.array_equal(subc._CAPI_GetCOOCols().cpu().numpy(), col[mask])


@pytest.mark.parametrize("num_rows_picked,max_deg", [(6, 400), (40, 12)])
def test_relabel_of_a_row_sliced_matrix(num_rows_picked, max_deg):
    """After row slicing the rows of a matrix are positions in the list of picked
    rows.  With few picked rows and many edges the relabel works on that list
    (first edge per picked row) instead of hashing every edge; with more picked
    rows it hashes the edges.  Both must give the unique of
    seeds ++ picked[coo.row] in first-occurrence order, and the same labels."""
    rng = np.random.default_rng(num_rows_picked)
    indptr, indices = random_csc(rng, 60, 50, max_deg, empty_frac=0.0)
    indices[indices == 49] = 48   # row 49 has no edge
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    cols = rng.permutation(60)[:12]
    picked = rng.permutation(50)[:num_rows_picked]
    if num_rows_picked == 6:
        picked[2] = 49            # a picked row without any edge
    sub = m[T(picked), T(cols)]
    row, col, _ = sub.coo
    assert (row.numel() >= 8 * (num_rows_picked + 12)) == (num_rows_picked == 6)
    seeds = T(cols)
    uniq, out_row, out_col, _ = sub._graph._CAPI_GraphRelabel(seeds, T(picked))
    keys = picked[row.cpu().numpy()]
    want = orc.unique_relabel(cols, keys, edge_col=col.cpu().numpy())
    assert np.array_equal(uniq.cpu().numpy(), want[0])
    assert np.array_equal(out_row.cpu().numpy(), want[2])
    assert np.array_equal(out_col.cpu().numpy(), want[3])
    assert np.array_equal(sub.all_nodes().cpu().numpy(), want[0])
    # first_position itself
    first = capi.first_position(row, num_rows_picked).cpu().numpy()
    r = row.cpu().numpy()
    for l in range(num_rows_picked):
        hits = np.nonzero(r == l)[0]
        assert first[l] == (hits[0] if hits.size else np.iinfo(np.int64).max)
