"""Edge-wise operators on the GPU: C ABI vs the oracle (fp32 within 1e-5
relative; copies and fp64 products exactly), and the gs.ops / Matrix wrappers
(broadcast tables, format selection, e_ids of converted formats)."""
import numpy as np
import pytest
import torch

import gsampler_amd as gs
from gsampler_amd import capi
from oracle import binding as orc
from tests.conftest import random_csc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = 1e-5


def T(a):
    return None if a is None else torch.as_tensor(a, device=DEV)


def close(got, want, rtol=RTOL):
    got = got.cpu().numpy()
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=rtol, atol=1e-6), np.abs(got - want).max()


@pytest.fixture(scope="module")
def g():
    rng = np.random.default_rng(7)
    indptr, indices = random_csc(rng, 700, 500, 60, hub_deg=20000)
    col = np.repeat(np.arange(700), np.diff(indptr))
    return rng, indptr, indices, col


def views(indptr, indices, col):
    return {"coo": (("coo", indices, col), ("coo", T(indices), T(col))),
            "csc": (("csc", indptr, indices), ("csc", T(indptr), T(indices)))}


@pytest.mark.parametrize("fmt", ["coo", "csc"])
def test_sddmm_parity(g, fmt):
    rng, indptr, indices, col = g
    ov, gv = views(indptr, indices, col)[fmt]
    E = indices.size
    u = rng.random(500, dtype=np.float32) + 0.5
    v = rng.random(700, dtype=np.float32) + 0.5
    e = rng.random(E, dtype=np.float32) + 0.1
    for op in ("add", "sub", "mul", "div"):
        close(capi.sddmm(gv, op, T(u), T(v), 0, 2), orc.sddmm(ov, op, u, v, 0, 2))
    close(capi.sddmm(gv, "div", T(e), T(v), 1, 2), orc.sddmm(ov, "div", e, v, 1, 2))
    close(capi.sddmm(gv, "mul", T(e), T(u), 1, 0), orc.sddmm(ov, "mul", e, u, 1, 0))
    assert np.array_equal(capi.sddmm(gv, "copy_lhs", T(u), None, 0, 2).cpu().numpy(),
                          orc.sddmm(ov, "copy_lhs", u, None, 0, 2))
    U, V = rng.random((500, 6), dtype=np.float32), rng.random((700, 6), dtype=np.float32)
    close(capi.sddmm(gv, "dot", T(U), T(V), 0, 2), orc.sddmm(ov, "dot", U, V, 0, 2))
    close(capi.sddmm(gv, "mul", T(U), T(V), 0, 2), orc.sddmm(ov, "mul", U, V, 0, 2))
    perm = rng.permutation(E)
    e64 = rng.random(E)
    close(capi.sddmm(gv, "mul", T(e64), T(v.astype(np.float64)), 1, 2, edge_map=T(perm)),
          orc.sddmm(ov, "mul", e64, v.astype(np.float64), 1, 2, edge_map=perm), 1e-12)


@pytest.mark.parametrize("fmt", ["coo", "csc"])
def test_spmm_and_fusions_parity(g, fmt):
    rng, indptr, indices, col = g
    ov, gv = views(indptr, indices, col)[fmt]
    E = indices.size
    u = rng.random(500, dtype=np.float32) + 0.5
    e = rng.random(E, dtype=np.float32) + 0.1
    close(capi.spmm(gv, "copy_rhs", "sum", None, T(e), 0, 700),
          orc.spmm(ov, "copy_rhs", "sum", None, e, 0, 700))
    close(capi.spmm(gv, "mul", "sum", T(u), T(e), 0, 700),
          orc.spmm(ov, "mul", "sum", u, e, 0, 700))
    close(capi.e_square_sum(gv, T(e), 0, 700), orc.e_square_sum(ov, e, 0, 700))
    close(capi.e_div_u_sum(gv, T(u), T(e), 0, 700), orc.e_div_u_sum(ov, u, e, 0, 700))
    if fmt == "coo":
        close(capi.spmm(gv, "copy_rhs", "sum", None, T(e), 2, 500),
              orc.spmm(ov, "copy_rhs", "sum", None, e, 2, 500))
        close(capi.e_square_sum(gv, T(e), 2, 500), orc.e_square_sum(ov, e, 2, 500))
    F = rng.random((E, 5), dtype=np.float32)
    close(capi.spmm(gv, "copy_rhs", "sum", None, T(F), 0, 700),
          orc.spmm(ov, "copy_rhs", "sum", None, F, 0, 700))
    s = e - 0.4
    for red in ("max", "min"):
        got = capi.spmm(gv, "copy_rhs", red, None, T(s), 0, 700, want_arg=True)
        want = orc.spmm(ov, "copy_rhs", red, None, s, 0, 700, want_arg=True)
        assert np.array_equal(got[0].cpu().numpy(), want[0])
        hit = want[0] != 0
        assert np.array_equal(s[got[2].cpu().numpy()[hit]], want[0][hit])
    o1, o2 = capi.fused_u_op_v(gv, "mul", T(u), T(e[:700]), T(u * 2), T(e[:700] + 1))
    w1, w2 = orc.fused_u_op_v(ov, "mul", u, e[:700], u * 2, e[:700] + 1)
    close(o1, w1); close(o2, w2)


@pytest.mark.parametrize("shape", ["hubs", "row_ranges", "tiny_segments"])
def test_scalar_sums_on_skewed_matrices(shape):
    """The load-balanced sum kernels: a few segments that hold most of the edges
    (and rows that most edges point to), and thousands of segments with zero or
    one edge.  Sums of up to 10^6 fp32 terms are compared with a float64 sum at
    1e-5 relative (the order of additions is not fixed)."""
    rng = np.random.default_rng(31)
    if shape == "hubs":
        deg = np.full(40, 50)
        deg[[3, 17]] = [1200000, 400000]     # > 2^20 edges: per-die accumulators
        R = 3000
        w = 1.0 / np.arange(1, R + 1) ** 1.2
        indices = rng.choice(R, size=int(deg.sum()), p=w / w.sum())
    elif shape == "row_ranges":
        # several ranges of 8192 rows: one holds a hub row (many slices of one
        # range), one is empty, the last one is partial
        deg = np.full(300, 5000)
        R = 30000
        indices = rng.integers(0, R, size=int(deg.sum()))
        indices[(indices >= 8192) & (indices < 16384)] += 8192
        indices[rng.random(indices.size) < 0.4] = 20001
    else:
        deg = rng.integers(0, 2, size=9000)
        R = 500
        indices = rng.integers(0, R, size=int(deg.sum()))
    C = deg.size
    indptr = np.concatenate([[0], np.cumsum(deg)])
    col = np.repeat(np.arange(C), deg)
    e = rng.random(indices.size, dtype=np.float32) + 0.1
    u = rng.random(R, dtype=np.float32) + 0.5
    e64 = e.astype(np.float64)
    onto_cols = np.bincount(col, weights=e64, minlength=C)
    onto_rows = np.bincount(indices, weights=e64, minlength=R)
    sq_rows = np.bincount(indices, weights=e64 * e64, minlength=R)
    div_cols = np.bincount(col, weights=e64 / u[indices], minlength=C)
    coo, csc = ("coo", T(indices), T(col)), ("csc", T(indptr), T(indices))
    for view in (coo, csc):
        close(capi.spmm(view, "copy_rhs", "sum", None, T(e), 0, C), onto_cols.astype(np.float32))
        close(capi.e_div_u_sum(view, T(u), T(e), 0, C), div_cols.astype(np.float32))
    close(capi.spmm(coo, "copy_rhs", "sum", None, T(e), 2, R), onto_rows.astype(np.float32))
    close(capi.e_square_sum(coo, T(e), 2, R), sq_rows.astype(np.float32))
    # and the oracle agrees with the float64 sums as well
    assert np.allclose(orc.spmm(("csc", indptr, indices), "copy_rhs", "sum", None, e, 0, C),
                       onto_cols, rtol=1e-5)


def test_matrix_sum_div_and_ops_wrappers(g):
    rng, indptr, indices, col = g
    m = gs.Matrix()
    m.load_graph("CSC", [T(indptr), T(indices)])
    R = m.num_rows()
    E = indices.size
    w = rng.random(E, dtype=np.float32) + 0.1
    m.edata["w"] = T(w)
    col_sum = np.zeros(700); np.add.at(col_sum, col, w.astype(np.float64))
    row_sum = np.zeros(R); np.add.at(row_sum, indices, w.astype(np.float64))
    close(m.sum("w", 0), col_sum.astype(np.float32))
    close(m.sum("w", 1), row_sum.astype(np.float32))       # runs on a CSR built on demand
    d = rng.random(700, dtype=np.float32) + 0.5
    close(m.div("w", T(d), 0).edata["w"], w / d[col])       # div divides
    dr = rng.random(R, dtype=np.float32) + 0.5
    close(m.div("w", T(dr), 1).edata["w"], w / dr[indices])
    close(gs.ops.e_square_sum(m, "w", 1), (row_sum * 0 + np.bincount(
        indices, weights=w.astype(np.float64) ** 2, minlength=R)).astype(np.float32))
    close(gs.ops.e_square_sum(m, "w", 0), np.bincount(
        col, weights=w.astype(np.float64) ** 2, minlength=700).astype(np.float32))
    u = rng.random(R, dtype=np.float32) + 0.5
    close(gs.ops.e_div_u_sum(m, "w", T(u), 0), np.bincount(
        col, weights=(w / u[indices]).astype(np.float64), minlength=700).astype(np.float32))
    # broadcasting: [R, 3, 1] * [C, 1, 4] -> [E, 3, 4]
    A = rng.random((R, 3, 1), dtype=np.float32)
    B = rng.random((700, 1, 4), dtype=np.float32)
    close(gs.ops.u_mul_v(m, T(A), T(B)), A[indices] * B[col])
    close(gs.ops.u_add_v(m, T(A), T(B), gs._CSC), A[indices] + B[col])
    o1, o2 = gs.ops.fused_u_mul_v(m, T(u), T(d), T(u + 1), T(d + 1))
    close(o1, u[indices] * d[col]); close(o2, (u[indices] + 1) * (d[col] + 1))
    close(gs.ops.copy_e_sum(m, T(w)), col_sum.astype(np.float32))
