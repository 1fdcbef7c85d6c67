"""One matrix loaded as CSC, as CSR and as an unsorted edge list: sums, quotients,
slices and blocks must describe the same weighted matrix whatever format an
operator runs on (edge data stays in the order the matrix was loaded in; the
operators follow it through the edge ids of converted formats).  Checked against
a dense float64 copy."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
R, C, E = 300, 200, 6000


@pytest.fixture(scope="module")
def loaded():
    rng = np.random.default_rng(5)
    pairs = rng.choice(R * C, size=E, replace=False)          # distinct (row, col) pairs
    row, col = pairs // C, pairs % C
    w = (rng.random(E) + 0.5).astype(np.float32)
    dense = np.zeros((R, C))
    dense[row, col] = w
    out = {}
    # edge list in random order
    m = gs.Matrix()
    m.load_graph("COO", [torch.tensor(row, device=DEV), torch.tensor(col, device=DEV)])
    m.edata["w"] = torch.tensor(w, device=DEV)
    out["coo"] = m
    # CSC: edges ordered by column
    order = np.argsort(col, kind="stable")
    indptr = np.concatenate([[0], np.cumsum(np.bincount(col, minlength=C))])
    m = gs.Matrix()
    m.load_graph("CSC", [torch.tensor(indptr, device=DEV), torch.tensor(row[order], device=DEV)])
    m.edata["w"] = torch.tensor(w[order], device=DEV)
    out["csc"] = m
    # CSR: edges ordered by row
    order = np.argsort(row, kind="stable")
    indptr = np.concatenate([[0], np.cumsum(np.bincount(row, minlength=R))])
    m = gs.Matrix()
    m.load_graph("CSR", [torch.tensor(indptr, device=DEV), torch.tensor(col[order], device=DEV)])
    m.edata["w"] = torch.tensor(w[order], device=DEV)
    out["csr"] = m
    return out, dense


def dense_of(m, key="w"):
    """Dense matrix from whatever the Matrix reports as its edge list + data."""
    row, col, eids = m.coo
    data = m.edata[key]
    if eids is not None and eids.numel() > 0:
        data = data[eids]
    out = np.zeros((m.num_rows(), m.num_cols()))
    np.add.at(out, (row.cpu().numpy(), col.cpu().numpy()), data.double().cpu().numpy())
    return out


@pytest.mark.parametrize("fmt", ["coo", "csc", "csr"])
def test_shape_sums_and_quotients(loaded, fmt):
    ms, dense = loaded
    m = ms[fmt]
    assert (m.num_rows(), m.num_cols(), m.num_edges()) == (R, C, E)
    assert np.allclose(dense_of(m), dense)
    assert np.allclose(m.sum("w", axis=0).cpu().numpy(), dense.sum(axis=0), rtol=1e-5)
    assert np.allclose(m.sum("w", axis=1).cpu().numpy(), dense.sum(axis=1), rtol=1e-5)
    by_col = m.div("w", m.sum("w", axis=0), axis=0)
    with np.errstate(invalid="ignore", divide="ignore"):
        want = np.nan_to_num(dense / dense.sum(axis=0, keepdims=True))
    assert np.allclose(dense_of(by_col), want, rtol=1e-5)
    by_row = m.div("w", m.sum("w", axis=1), axis=1)
    with np.errstate(invalid="ignore", divide="ignore"):
        want = np.nan_to_num(dense / dense.sum(axis=1, keepdims=True))
    assert np.allclose(dense_of(by_row), want, rtol=1e-5)


@pytest.mark.parametrize("fmt", ["coo", "csc", "csr"])
def test_slices_keep_their_edge_data(loaded, fmt):
    ms, dense = loaded
    m = ms[fmt]
    cols = torch.tensor([5, 7, 7, 150, 199, 0], device=DEV)
    rows = torch.tensor([299, 3, 44, 45, 46, 100, 3], device=DEV)
    sub = m[:, cols]
    assert np.allclose(dense_of(sub), dense[:, cols.cpu().numpy()])
    assert np.allclose(sub.sum("w", axis=1).cpu().numpy(), dense[:, cols.cpu().numpy()].sum(axis=1),
                       rtol=1e-5)
    sub = m[rows, :]
    assert np.allclose(dense_of(sub), dense[rows.cpu().numpy(), :])
    sub = m[rows, cols]
    assert np.allclose(dense_of(sub), dense[np.ix_(rows.cpu().numpy(), cols.cpu().numpy())])


@pytest.mark.parametrize("fmt", ["coo", "csc", "csr"])
def test_sampling_and_blocks(loaded, fmt):
    ms, dense = loaded
    m = ms[fmt]
    cols = torch.arange(0, C, 3, device=DEV)
    gs.manual_seed(3)
    picked = m[:, cols].individual_sampling(4, None, False)
    got = dense_of(picked)
    want = dense[:, cols.cpu().numpy()]
    assert np.all((got == 0) | np.isclose(got, want))                 # a subset, weights intact
    assert np.array_equal((got != 0).sum(axis=0), np.minimum((want != 0).sum(axis=0), 4))
    block = picked.to_dgl_block(prefetch_edata={"w"})
    src = block.srcdata["_ID"][block.row].cpu().numpy()
    dst = cols[block.col].cpu().numpy()
    assert np.allclose(block.edata["w"].cpu().numpy(), dense[src, dst])
    assert torch.equal(block.srcdata["_ID"][: cols.numel()], cols)
    assert torch.equal(torch.sort(picked.all_nodes())[0], torch.sort(block.srcdata["_ID"])[0])
    # weighted picks favour heavy edges: with the weight as probability and one
    # pick per column, the pick is an edge of that column with positive weight
    gs.manual_seed(4)
    sub = m[:, cols]
    one = sub.individual_sampling(1, sub.edata["w"], False)
    got = dense_of(one)
    assert np.all((got == 0) | np.isclose(got, want))
    assert np.array_equal((got != 0).sum(axis=0), np.minimum((want != 0).sum(axis=0), 1))
