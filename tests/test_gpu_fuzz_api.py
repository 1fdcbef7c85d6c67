"""Random sequences of Matrix operations (column, row and two-sided slices with
repeated and empty id lists, sums, quotients, per-column and collective
sampling, the block hand-off) on random multigraphs loaded as edge list, CSC or
CSR, checked after every step against a dense float64 model.  Weights are
multiples of 1/8, so sums are exact in any order.
The super-batched API the same way: random mini-batches (some empty) through
BatchMatrix column slicing, per-column sampling, all_nodes and the per-batch
blocks, one or two layers, checked batch by batch against the matrix."""
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


# ------------------------------------------------------------ super-batches
def batch_case(seed):
    rng = np.random.default_rng(seed)
    N = int(rng.integers(2, 500))
    E = int(rng.integers(1, 6000))
    row = rng.integers(0, N, size=E); col = rng.integers(0, N, size=E)
    row[-1], col[-1] = N - 1, N - 1
    w = (rng.integers(1, 9, size=E) / 8.0).astype(np.float32)
    order = np.argsort(col, kind="stable")
    indptr = np.concatenate([[0], np.cumsum(np.bincount(col, minlength=N))])
    m = gs.Matrix()
    m.load_graph("CSC", [torch.tensor(indptr, device=DEV), torch.tensor(row[order], device=DEV)])
    m.edata["w"] = torch.tensor(w[order], device=DEV)
    count = np.zeros((N, N), dtype=np.int64); np.add.at(count, (row, col), 1)
    deg = count.sum(axis=0)
    encoding = bool(rng.integers(0, 2))
    bm = gs.BatchMatrix(); bm.load_from_matrix(m, encoding)
    B = int(rng.integers(1, 9))
    sizes = [int(rng.integers(0, 40)) if rng.random() > 0.15 else 0 for _ in range(B)]
    distinct = True          # seeds of a mini-batch are distinct (duplicates share one label)
    seeds_l = [rng.permutation(N)[:min(s, N)] if distinct else rng.integers(0, N, size=s) for s in sizes]
    ptr = np.concatenate([[0], np.cumsum([len(s) for s in seeds_l])]).astype(np.int64)
    seeds = np.concatenate(seeds_l).astype(np.int64) if ptr[-1] else np.zeros(0, np.int64)
    g_seeds, g_ptr = torch.tensor(seeds, device=DEV), torch.tensor(ptr, device=DEV)
    layers = int(rng.integers(1, 3))
    gs.manual_seed(seed)
    for layer in range(layers):
        k = int(rng.integers(1, 7))
        sub = bm[:, g_seeds::g_ptr]
        smp = sub.individual_sampling(k, None, False)
        nodes, nodes_ptr = smp.all_nodes()
        blocks = smp.to_dgl_block()
        assert len(blocks) == B, "blocks"
        nodes, nodes_ptr = nodes.cpu().numpy(), nodes_ptr.cpu().numpy()
        assert nodes_ptr[0] == 0 and nodes_ptr[-1] == nodes.size
        new_seeds = []
        for b, blk in enumerate(blocks):
            sb = seeds[ptr[b]:ptr[b + 1]]
            fr = blk.srcdata["_ID"].cpu().numpy()
            assert np.array_equal(fr, nodes[nodes_ptr[b]:nodes_ptr[b + 1]]), ("frontier", seed, b)
            assert blk.num_dst == sb.size and blk.num_src == fr.size
            r, c = blk.row.cpu().numpy(), blk.col.cpu().numpy()
            src, dst_pos = fr[r], c
            assert np.all((dst_pos >= 0) & (dst_pos < max(sb.size, 1))) or r.size == 0
            dst = sb[dst_pos] if r.size else dst_pos
            # counts per requested column (position), edges exist, no more copies than the matrix has
            per_col = np.bincount(dst_pos, minlength=sb.size) if r.size else np.zeros(sb.size, int)
            assert np.array_equal(per_col, np.minimum(deg[sb], k)), ("count", seed, b)
            got = {}
            for s_, p_ in zip(src.tolist(), dst_pos.tolist()):
                got[(s_, p_)] = got.get((s_, p_), 0) + 1
            for (s_, p_), n_ in got.items():
                assert n_ <= count[s_, sb[p_]], ("edge", seed, b)
            # frontier: unique of seeds ++ sources in first-occurrence order
            keys = np.concatenate([sb, src])
            # block edge order is the sampled edge order of this batch, so first occurrences follow it
            _, first = np.unique(keys, return_index=True)
            assert np.array_equal(fr, keys[np.sort(first)]), ("order", seed, b)
            new_seeds.append(fr)
        seeds_l = new_seeds
        ptr = np.concatenate([[0], np.cumsum([len(s) for s in seeds_l])]).astype(np.int64)
        seeds = np.concatenate(seeds_l).astype(np.int64) if ptr[-1] else np.zeros(0, np.int64)
        g_seeds, g_ptr = torch.tensor(seeds, device=DEV), torch.tensor(ptr, device=DEV)


@pytest.mark.parametrize("block", range(3))
def test_random_super_batches(block):
    for seed in range(block * 100, block * 100 + 100):
        batch_case(seed)
