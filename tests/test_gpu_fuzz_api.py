"""Random sequences of Matrix operations (column, row and two-sided slices with
repeated and empty id lists, sums, quotients, per-column and collective
sampling, the block hand-off) on random multigraphs loaded as edge list, CSC or
CSR, checked after every step against a dense float64 model.  Weights are
multiples of 1/8, so sums are exact in any order."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dense_of(m, key="w"):
    row, col, eids = m.coo
    data = m.edata[key]
    if eids is not None and eids.numel() > 0:
        data = data[eids]
    out = np.zeros((m.num_rows(), m.num_cols()))
    np.add.at(out, (row.cpu().numpy(), col.cpu().numpy()), data.double().cpu().numpy())
    return out

def load(fmt, row, col, w, R, C):
    m = gs.Matrix()
    if fmt == "coo":
        m.load_graph("COO", [torch.tensor(row, device=DEV), torch.tensor(col, device=DEV)])
        m.edata["w"] = torch.tensor(w, device=DEV)
    elif fmt == "csc":
        order = np.argsort(col, kind="stable")
        indptr = np.concatenate([[0], np.cumsum(np.bincount(col, minlength=C))])
        m.load_graph("CSC", [torch.tensor(indptr, device=DEV), torch.tensor(row[order], device=DEV)])
        m.edata["w"] = torch.tensor(w[order], device=DEV)
    else:
        order = np.argsort(row, kind="stable")
        indptr = np.concatenate([[0], np.cumsum(np.bincount(row, minlength=R))])
        m.load_graph("CSR", [torch.tensor(indptr, device=DEV), torch.tensor(col[order], device=DEV)])
        m.edata["w"] = torch.tensor(w[order], device=DEV)
    return m

def case(seed):
    rng = np.random.default_rng(seed)
    R, C = int(rng.integers(1, 400)), int(rng.integers(1, 300))
    E = int(rng.integers(0, 5000))
    E += 1
    row = rng.integers(0, R, size=E); col = rng.integers(0, C, size=E)
    row[-1], col[-1] = R - 1, C - 1          # shapes are inferred from the largest ids
    w = (rng.integers(1, 9, size=E) / 8.0).astype(np.float32)     # dyadic: sums exact
    dense = np.zeros((R, C)); np.add.at(dense, (row, col), w.astype(np.float64))
    fmt = ["coo", "csc", "csr"][seed % 3]
    m = load(fmt, row, col, w, R, C)
    assert (m.num_rows(), m.num_cols(), m.num_edges()) == (R, C, E)
    steps = int(rng.integers(1, 5))
    trail = [fmt]
    for _ in range(steps):
        op = rng.choice(["cols", "rows", "both", "sum", "div0", "div1", "sample", "collective"])
        trail.append(op)
        r_now, c_now = dense.shape
        if r_now == 0 or c_now == 0:
            break
        if op == "cols":
            cols = rng.integers(0, c_now, size=int(rng.integers(0, 60)))
            m = m[:, torch.tensor(cols, device=DEV, dtype=torch.int64)]
            dense = dense[:, cols]
        elif op == "rows":
            rows = rng.permutation(r_now)[: int(rng.integers(0, r_now + 1))]     # distinct rows
            m = m[torch.tensor(rows, device=DEV, dtype=torch.int64), :]
            dense = dense[rows, :]
        elif op == "both":
            cols = rng.integers(0, c_now, size=int(rng.integers(0, 60)))
            rows = rng.permutation(r_now)[: int(rng.integers(0, r_now + 1))]
            m = m[torch.tensor(rows, device=DEV, dtype=torch.int64), torch.tensor(cols, device=DEV, dtype=torch.int64)]
            dense = dense[np.ix_(rows, cols)]
        elif op == "sum":
            assert np.allclose(m.sum("w", axis=0).cpu().numpy(), dense.sum(axis=0), rtol=1e-5, atol=1e-6), trail
            assert np.allclose(m.sum("w", axis=1).cpu().numpy(), dense.sum(axis=1), rtol=1e-5, atol=1e-6), trail
        elif op in ("div0", "div1"):
            ax = 0 if op == "div0" else 1
            d = torch.tensor(rng.integers(1, 5, size=dense.shape[1 - ax]).astype(np.float32), device=DEV)
            m = m.div("w", d, axis=ax)
            dn = d.cpu().numpy().astype(np.float64)
            dense = dense / (dn[None, :] if ax == 0 else dn[:, None])
        elif op == "sample":
            k = int(rng.integers(1, 6))
            nz_before = None
            got_m = m.individual_sampling(k, None, False)
            got = dense_of(got_m) if got_m.num_edges() else np.zeros(dense.shape)
            # multigraph: a cell may hold several edges; sampled cell sums never exceed the original
            assert np.all(got <= dense + 1e-6), trail
            row_, col_, _ = m.coo
            deg = np.bincount(col_.cpu().numpy(), minlength=dense.shape[1]) if m.num_edges() else np.zeros(dense.shape[1], int)
            r2, c2, _ = got_m.coo
            deg2 = np.bincount(c2.cpu().numpy(), minlength=dense.shape[1]) if got_m.num_edges() else np.zeros(dense.shape[1], int)
            assert np.array_equal(deg2, np.minimum(deg, k)), trail
            m, dense = got_m, got
        elif op == "collective":
            k = int(rng.integers(1, 20))
            p = torch.tensor((rng.random(r_now) + 0.01).astype(np.float32), device=DEV)
            sub, picked = m.collective_sampling(k, p, False)
            pk = picked.cpu().numpy()
            assert pk.size == min(k, r_now) and np.unique(pk).size == pk.size, trail
            m, dense = sub, dense[pk, :]
        got = dense_of(m) if m.num_edges() else np.zeros(dense.shape)
        assert got.shape == dense.shape, (trail, got.shape, dense.shape)
        assert np.allclose(got, dense, rtol=1e-5, atol=1e-6), trail
    # hand-off: block edges describe the same matrix
    if m.num_cols() > 0 and "_ID" in m.col_ndata:
        blk = m.to_dgl_block(prefetch_edata={"w"})
        nodes = m.all_nodes()
        assert torch.equal(torch.sort(nodes)[0], torch.sort(blk.srcdata["_ID"])[0]), trail
        assert blk.num_edges() == m.num_edges(), trail


@pytest.mark.parametrize("block", range(4))
def test_random_operator_sequences(block):
    for seed in range(block * 100, block * 100 + 100):
        case(seed)
