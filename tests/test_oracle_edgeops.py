"""Oracle edge-wise operators against NumPy closed forms (np.add.at /
broadcasting); fp32, tolerance 1e-5 relative as the summation order differs."""
import numpy as np
import pytest

from oracle import binding as orc
from tests.conftest import random_csc

RTOL = 1e-5


def _graph(seed=0, cols=120, rows=90, max_deg=30):
    rng = np.random.default_rng(seed)
    indptr, indices = random_csc(rng, cols, rows, max_deg, hub_deg=400)
    col = np.repeat(np.arange(cols), np.diff(indptr))
    return rng, indptr, indices, col, rows, cols


@pytest.mark.parametrize("fmt", ["coo", "csc"])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_sddmm_u_op_v(fmt, op):
    rng, indptr, indices, col, R, Cn = _graph()
    u = rng.random(R, dtype=np.float32) + 0.5
    v = rng.random(Cn, dtype=np.float32) + 0.5
    view = ("coo", indices, col) if fmt == "coo" else ("csc", indptr, indices)
    got = orc.sddmm(view, op, u, v, 0, 2)
    f = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}[op]
    assert np.allclose(got, f(u[indices], v[col]), rtol=RTOL)


def test_sddmm_edge_targets_and_copy_and_dot():
    rng, indptr, indices, col, R, Cn = _graph(1)
    E = indices.size
    e = rng.random(E, dtype=np.float32) + 0.1
    v = rng.random(Cn, dtype=np.float32) + 0.5
    view = ("coo", indices, col)
    # LADIES: edge weight divided by a per-column / per-row vector
    assert np.allclose(orc.sddmm(view, "div", e, v, 1, 2), e / v[col], rtol=RTOL)
    u = rng.random(R, dtype=np.float32) + 0.5
    assert np.allclose(orc.sddmm(view, "div", e, u, 1, 0), e / u[indices], rtol=RTOL)
    assert np.array_equal(orc.sddmm(view, "copy_lhs", u, None, 0, 2), u[indices])
    assert np.array_equal(orc.sddmm(view, "copy_rhs", None, v, 0, 2), v[col])
    U = rng.random((R, 8), dtype=np.float32)
    V = rng.random((Cn, 8), dtype=np.float32)
    assert np.allclose(orc.sddmm(("csc", indptr, indices), "dot", U, V, 0, 2)[:, 0],
                       np.einsum("ef,ef->e", U[indices], V[col]), rtol=1e-4)
    assert np.allclose(orc.sddmm(view, "mul", U, V, 0, 2), U[indices] * V[col], rtol=RTOL)
    # fp64 and an edge map (features stored in another edge order)
    perm = rng.permutation(E)
    e64 = rng.random(E)
    got = orc.sddmm(view, "mul", e64, v.astype(np.float64), 1, 2, edge_map=perm)
    want = np.zeros(E); want[perm] = e64[perm] * v[col]
    assert np.allclose(got, want)


@pytest.mark.parametrize("fmt", ["coo", "csc"])
def test_spmm_sum_onto_columns_and_rows(fmt):
    rng, indptr, indices, col, R, Cn = _graph(2)
    E = indices.size
    e = rng.random(E, dtype=np.float32)
    u = rng.random(R, dtype=np.float32)
    view = ("coo", indices, col) if fmt == "coo" else ("csc", indptr, indices)
    want = np.zeros(Cn); np.add.at(want, col, e.astype(np.float64))
    assert np.allclose(orc.spmm(view, "copy_rhs", "sum", None, e, 0, Cn), want, rtol=RTOL)
    want = np.zeros(Cn); np.add.at(want, col, (u[indices] * e).astype(np.float64))
    assert np.allclose(orc.spmm(view, "mul", "sum", u, e, 0, Cn), want, rtol=RTOL)
    if fmt == "coo":  # u_target 2: reduce onto rows
        want = np.zeros(R); np.add.at(want, indices, e.astype(np.float64))
        assert np.allclose(orc.spmm(view, "copy_rhs", "sum", None, e, 2, R), want, rtol=RTOL)


def test_spmm_max_min_start_from_zero():
    rng, indptr, indices, col, R, Cn = _graph(3)
    e = (rng.random(indices.size, dtype=np.float32) - 0.3)
    want = np.zeros(Cn, dtype=np.float32); np.maximum.at(want, col, e)
    for view in (("coo", indices, col), ("csc", indptr, indices)):
        out, au, ae = orc.spmm(view, "copy_rhs", "max", None, e, 0, Cn, want_arg=True)
        assert np.array_equal(out, want)
        hit = out > 0
        assert np.array_equal(e[ae[hit]], out[hit])
    want = np.zeros(Cn, dtype=np.float32); np.minimum.at(want, col, e)
    assert np.array_equal(orc.spmm(("csc", indptr, indices), "copy_rhs", "min", None, e, 0, Cn),
                          want)


def test_fused_operators():
    rng, indptr, indices, col, R, Cn = _graph(4)
    E = indices.size
    e = rng.random(E, dtype=np.float32) + 0.1
    u = rng.random(R, dtype=np.float32) + 0.5
    csc, coo = ("csc", indptr, indices), ("coo", indices, col)
    want = np.zeros(Cn); np.add.at(want, col, e.astype(np.float64) ** 2)
    assert np.allclose(orc.e_square_sum(csc, e, 0, Cn), want, rtol=RTOL)
    assert np.allclose(orc.e_square_sum(coo, e, 0, Cn), want, rtol=RTOL)
    want = np.zeros(R); np.add.at(want, indices, e.astype(np.float64) ** 2)
    assert np.allclose(orc.e_square_sum(coo, e, 2, R), want, rtol=RTOL)
    want = np.zeros(Cn); np.add.at(want, col, (e / u[indices]).astype(np.float64))
    assert np.allclose(orc.e_div_u_sum(csc, u, e, 0, Cn), want, rtol=RTOL)
    assert np.allclose(orc.e_div_u_sum(coo, u, e, 0, Cn), want, rtol=RTOL)
    v1, v2 = rng.random(Cn, dtype=np.float32), rng.random(Cn, dtype=np.float32)
    u2 = rng.random(R, dtype=np.float32)
    o1, o2 = orc.fused_u_op_v(csc, "mul", u, v1, u2, v2)
    assert np.allclose(o1, u[indices] * v1[col], rtol=RTOL)
    assert np.allclose(o2, u2[indices] * v2[col], rtol=RTOL)


def test_row_slice_csr_view_uses_edge_map():
    """Reducing onto rows through a CSR built from the COO: edge features stay
    in COO order and are reached through e_ids (the stable-sort permutation)."""
    rng, indptr, indices, col, R, Cn = _graph(5)
    E = indices.size
    e = rng.random(E, dtype=np.float32)
    perm = np.argsort(indices, kind="stable")
    r_indptr = np.concatenate([[0], np.cumsum(np.bincount(indices, minlength=R))])
    got = orc.spmm(("csc", r_indptr, col[perm]), "copy_rhs", "sum", None, e, 0, R, edge_map=perm)
    want = np.zeros(R); np.add.at(want, indices, e.astype(np.float64))
    assert np.allclose(got, want, rtol=RTOL)
