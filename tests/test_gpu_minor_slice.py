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


@pytest.mark.parametrize("npick", [20000, 140000])
def test_minor_slice_with_a_table_outside_lds(npick):
    """Picked sets whose table lives in L2: behind the filter that is kept in LDS
    (up to 131 072 ids) and without it; 19 M edges, so that work-groups stride
    over several runs of chunks."""
    rng = np.random.default_rng(npick)
    indptr, indices = random_csc(rng, 20000, 400000, 2400, hub_deg=60000)
    picked = rng.integers(0, 410000, size=npick)  # repeats and absent ids
    same(capi.minor_slice(T(indices), T(picked), indptr=T(indptr)),
         orc.minor_slice(indices, picked, indptr=indptr))


@pytest.mark.parametrize("npick", [3, 700, 5000])
def test_minor_slice_with_ids_beyond_32_bits(npick):
    """Picked ids of 2^32 - 1 and above: ids that agree in their low 32 bits must
    not be taken for each other, repeated picked ids keep their smallest
    position, and a narrow picked set still ignores wide edge ids."""
    rng = np.random.default_rng(npick)
    indptr, _ = random_csc(rng, 2000, 10, 60, hub_deg=30000)
    nnz = int(indptr[-1])
    low = rng.integers(0, 3000, size=nnz)
    low[rng.random(nnz) < 0.01] = 2**32 - 1
    ids = low + rng.integers(0, 4, size=nnz) * 2**32          # four ids per low half
    ids[:7] = [-3, 2**40, 2**32 - 1, 2**32 - 2, 2**63 - 1, 0, 2**32]
    col = np.repeat(np.arange(2000), np.diff(indptr))
    picked = rng.choice(ids, size=npick)
    picked[: min(npick, 3)] = [2**40, 2**32 - 1, -3][: min(npick, 3)]
    if npick > 10:
        picked[5] = picked[9]                                  # a repeated picked id
        picked[7] = 2**50 + 11                                 # one that no edge carries
    got = capi.minor_slice(T(ids), T(picked), indptr=T(indptr))
    same(got, orc.minor_slice(ids, picked, indptr=indptr))
    same(capi.minor_slice(T(ids), T(picked), edge_major=T(col)),
         orc.minor_slice(ids, picked, edge_major=col))
    # closed form: kept edges and their positions in the picked list
    first = {}
    for i, v in enumerate(picked.tolist()):
        first.setdefault(v, i)
    keep = np.array([v in first for v in ids.tolist()])
    assert np.array_equal(got[3].cpu().numpy(), np.nonzero(keep)[0])
    assert np.array_equal(got[2].cpu().numpy(), np.array([first[v] for v in ids[keep].tolist()]))
    # a narrow picked set against the same wide edge ids
    narrow = rng.integers(0, 3000, size=50)
    same(capi.minor_slice(T(ids), T(narrow), indptr=T(indptr)),
         orc.minor_slice(ids, narrow, indptr=indptr))


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


def test_column_slice_carries_edge_data_of_any_shape():
    """Edge data of A[:, cols]: scalar data goes by column runs of the parent's
    array, anything else through the edge index; both are data[edge positions]."""
    rng = np.random.default_rng(9)
    indptr, indices = random_csc(rng, 500, 300, 40, hub_deg=5000)
    nnz = indices.size
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    data = {"f32": torch.as_tensor(rng.random(nnz, dtype=np.float32), device=DEV),
            "f64": torch.as_tensor(rng.random(nnz), device=DEV),
            "i64": T(rng.integers(0, 10**12, size=nnz)),
            "f16": torch.as_tensor(rng.random(nnz, dtype=np.float32), device=DEV).half(),
            "wide": torch.as_tensor(rng.random((nnz, 3), dtype=np.float32), device=DEV),
            "strided": torch.as_tensor(rng.random((nnz, 2), dtype=np.float32), device=DEV)[:, 0]}
    for key, value in data.items():
        m.edata[key] = value
    for cols in (rng.integers(0, 500, size=90), np.arange(500)):
        sub = m[:, T(cols)]
        want = orc.col_slice(indptr, indices, cols)
        sel = torch.as_tensor(want[3], device=DEV)
        assert np.array_equal(sub.csc[1].cpu().numpy(), want[2])
        for key, value in data.items():
            assert torch.equal(sub.edata[key], value[sel]), key
    # a second slice in between does not confuse the first one's edge index
    g = m._graph
    a, sel_a = g._CAPI_Slicing(T(np.arange(10)), 1, gs._CSC, gs._CSC)
    b, sel_b = g._CAPI_Slicing(T(np.arange(20, 60)), 1, gs._CSC, gs._CSC)
    for sel in (sel_a, sel_b):
        assert torch.equal(torch.ops.gs_ops._CAPI_GatherRows(data["f32"], sel), data["f32"][sel])


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


@pytest.mark.parametrize("num_rows_picked,num_cols_picked", [(1500, 800), (1200, 848), (1300, 700)])
def test_relabel_of_a_row_sliced_matrix_with_a_long_list(num_rows_picked, num_cols_picked):
    """Around the 2048 keys that one work-group relabels from the picked list
    (more: sort + the general unique path; exactly that many and fewer: one
    launch), with repeated seeds among the columns."""
    rng = np.random.default_rng(num_rows_picked)
    indptr, indices = random_csc(rng, 3000, 4000, 160, empty_frac=0.05)
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    cols = rng.integers(0, 3000, size=num_cols_picked)          # repeats allowed
    picked = rng.permutation(4000)[:num_rows_picked]
    sub = m[T(picked), T(cols)]
    row, col, _ = sub.coo
    assert row.numel() >= 8 * (num_rows_picked + num_cols_picked)   # the list path is taken
    uniq, out_row, out_col, _ = sub._graph._CAPI_GraphRelabel(T(cols), T(picked))
    keys = picked[row.cpu().numpy()]
    want = orc.unique_relabel(cols, keys, edge_col=col.cpu().numpy())
    assert np.array_equal(uniq.cpu().numpy(), want[0])
    assert np.array_equal(out_row.cpu().numpy(), want[2])
    assert np.array_equal(out_col.cpu().numpy(), want[3])
    assert np.array_equal(sub.all_nodes().cpu().numpy(), want[0])


def test_batched_column_and_row_slice_whose_encoded_ids_pass_32_bits():
    """_CAPI_BatchColRowSlcing encodes a row of batch b as id + b * num_rows
    (src/cuda/batch/slicing.cu:25-27).  With 2^30 + 5 rows and 8 batches the
    encoded ids reach 2^33: every batch must still keep exactly the edges of its
    columns whose row it picked, relabelled to positions in `row`."""
    rng = np.random.default_rng(8)
    num_rows, num_cols, B = 2**30 + 5, 300, 8
    deg = rng.integers(0, 40, size=num_cols)
    indptr = np.concatenate([[0], np.cumsum(deg)])
    pool = np.concatenate([rng.integers(0, num_rows, size=400), [num_rows - 1, 0, 2**30]])
    indices = rng.choice(pool, size=int(indptr[-1]))
    g = gs.Graph(num_rows, num_cols)
    g._CAPI_LoadCSC(T(indptr), T(indices))
    cols = np.concatenate([rng.permutation(num_cols)[:30] for _ in range(B)])
    col_bptr = np.arange(B + 1) * 30
    rows = np.concatenate([rng.choice(pool, size=120, replace=False) for _ in range(B)])
    row_bptr = np.arange(B + 1) * 120
    sub, edge_index = g._CAPI_BatchColRowSlcing(T(cols), T(col_bptr), T(rows), T(row_bptr))
    got_indptr = sub._CAPI_GetCSCIndptr().cpu().numpy()
    got_rows = sub._CAPI_GetCSCIndices().cpu().numpy()
    got_sel = edge_index.cpu().numpy()
    want_rows, want_sel, want_cnt = [], [], []
    for b in range(B):
        where = {int(v): row_bptr[b] + i for i, v in enumerate(rows[row_bptr[b]:row_bptr[b + 1]])}
        for c in cols[col_bptr[b]:col_bptr[b + 1]]:
            n = 0
            for e in range(indptr[c], indptr[c + 1]):
                if int(indices[e]) in where:
                    want_rows.append(where[int(indices[e])])
                    want_sel.append(e)
                    n += 1
            want_cnt.append(n)
    assert len(want_sel) > 500 and max(want_rows) >= 7 * 120       # the later batches kept theirs
    assert np.array_equal(got_indptr, np.concatenate([[0], np.cumsum(want_cnt)]))
    assert np.array_equal(got_rows, np.array(want_rows))
    assert np.array_equal(got_sel, np.array(want_sel))
