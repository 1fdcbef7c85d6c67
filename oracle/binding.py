"""numpy-facing ctypes binding of the CPU oracle (oracle/libgs_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The shipped package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgs_oracle.so")

_lib = None


def build() -> None:
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        src = os.path.join(_HERE, "gs_oracle.cpp")
        if (not os.path.exists(LIB_PATH)
                or os.path.getmtime(src) > os.path.getmtime(LIB_PATH)):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.gs_num_threads_cpu.restype = C.c_int
    return _lib


def _i64(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int64))


def _p(a):
    if a is None:
        return None
    return a.ctypes.data_as(C.c_void_p)


def num_threads() -> int:
    return lib().gs_num_threads_cpu()


def philox4x32_10(ctr, key) -> np.ndarray:
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    lib().gs_philox4x32_10_cpu(_p(c), _p(k), _p(out))
    return out


def stream_words(seed, call_id, pos, draw) -> np.ndarray:
    out = np.zeros(4, dtype=np.uint32)
    lib().gs_stream_words_cpu(C.c_uint64(seed), C.c_uint64(call_id),
                              C.c_uint64(pos), C.c_uint64(draw), _p(out))
    return out


def exclusive_scan(x) -> np.ndarray:
    x = _i64(x)
    out = np.empty_like(x)
    lib().gs_exclusive_scan_i64_cpu(_p(x), _p(out), C.c_int64(x.size))
    return out


def col_count(indptr, column_ids, fanout, replace, num_items=None) -> np.ndarray:
    indptr = _i64(indptr)
    num_cols = indptr.size - 1
    if column_ids is not None:
        column_ids = _i64(column_ids)
        num_items = column_ids.size
    elif num_items is None:
        num_items = num_cols
    out = np.empty(num_items + 1, dtype=np.int64)
    lib().gs_csc_col_count_cpu(_p(indptr), C.c_int64(num_cols), _p(column_ids),
                               C.c_int64(num_items), C.c_int64(fanout),
                               C.c_int(int(replace)), _p(out))
    return out


def col_slice(indptr, indices, column_ids, with_coo=True, batch_ptr=None,
              encode_stride=0):
    indptr, indices, column_ids = _i64(indptr), _i64(indices), _i64(column_ids)
    num_cols = indptr.size - 1
    n = column_ids.size
    sub_indptr = col_count(indptr, column_ids, -1, False)
    nnz = int(sub_indptr[-1])
    out_idx = np.empty(nnz, dtype=np.int64)
    out_sel = np.empty(nnz, dtype=np.int64)
    out_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    nb = 0
    if batch_ptr is not None:
        batch_ptr = _i64(batch_ptr)
        nb = batch_ptr.size - 1
    lib().gs_csc_col_slice_fill_cpu(
        _p(indptr), C.c_int64(num_cols), _p(indices), _p(column_ids),
        C.c_int64(n), _p(sub_indptr), C.c_int64(nnz), _p(batch_ptr),
        C.c_int64(nb), C.c_int64(encode_stride), _p(out_col), _p(out_idx),
        _p(out_sel))
    return sub_indptr, out_col, out_idx, out_sel


def sample_uniform(indptr, indices, column_ids, fanout, replace=False, algo=0,
                   seed=7777, call_id=0, with_coo=True):
    indptr, indices = _i64(indptr), _i64(indices)
    num_cols = indptr.size - 1
    if column_ids is not None:
        column_ids = _i64(column_ids)
        n = column_ids.size
    else:
        n = num_cols
    sub_indptr = col_count(indptr, column_ids, fanout, replace, n)
    nnz = int(sub_indptr[-1])
    out_idx = np.empty(nnz, dtype=np.int64)
    out_sel = np.empty(nnz, dtype=np.int64)
    out_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gs_csc_col_sample_uniform_fill_cpu(
        _p(indptr), C.c_int64(num_cols), _p(indices), _p(column_ids),
        C.c_int64(n), C.c_int64(fanout), C.c_int(int(replace)), C.c_int(algo),
        C.c_uint64(seed), C.c_uint64(call_id), _p(sub_indptr), _p(out_col),
        _p(out_idx), _p(out_sel))
    return sub_indptr, out_col, out_idx, out_sel


def unique_relabel(seeds, rows, seeds_ptr=None, rows_ptr=None, edge_col=None,
                   want_row=True, want_col=True):
    seeds, rows = _i64(seeds), _i64(rows)
    S, E = seeds.size, rows.size
    if seeds_ptr is not None:
        seeds_ptr, rows_ptr = _i64(seeds_ptr), _i64(rows_ptr)
        B = seeds_ptr.size - 1
    else:
        B = 1
    unique_ptr = np.empty(B + 1, dtype=np.int64)
    lib().gs_unique_count_cpu(_p(seeds), _p(seeds_ptr), C.c_int64(S), _p(rows),
                              _p(rows_ptr), C.c_int64(E), C.c_int64(B),
                              _p(unique_ptr))
    U = int(unique_ptr[-1])
    unique = np.empty(U, dtype=np.int64)
    want_col = want_col and edge_col is not None
    if edge_col is not None:
        edge_col = _i64(edge_col)
    out_row = np.empty(E, dtype=np.int64) if want_row else None
    out_col = np.empty(E, dtype=np.int64) if want_col else None
    lib().gs_unique_fill_cpu(_p(seeds), _p(seeds_ptr), C.c_int64(S), _p(rows),
                             _p(rows_ptr), C.c_int64(E), C.c_int64(B),
                             _p(unique_ptr), _p(unique))
    if want_row or want_col:
        lib().gs_unique_relabel_cpu(_p(seeds), _p(seeds_ptr), C.c_int64(S), _p(rows),
                                    _p(rows_ptr), C.c_int64(E), C.c_int64(B),
                                    _p(edge_col), _p(out_row), _p(out_col))
    return unique, unique_ptr, out_row, out_col


def csc2coo(indptr, nnz=None) -> np.ndarray:
    indptr = _i64(indptr)
    if nnz is None:
        nnz = int(indptr[-1])
    out = np.empty(nnz, dtype=np.int64)
    lib().gs_csc2coo_cpu(_p(indptr), C.c_int64(indptr.size - 1), C.c_int64(nnz), _p(out))
    return out


def sorted_to_indptr(sorted_ids, num_cols) -> np.ndarray:
    sorted_ids = _i64(sorted_ids)
    out = np.empty(num_cols + 1, dtype=np.int64)
    lib().gs_sorted_to_indptr_cpu(_p(sorted_ids), C.c_int64(sorted_ids.size),
                                  C.c_int64(num_cols), _p(out))
    return out


def decode_batch_ids(encoded, stride):
    encoded = _i64(encoded)
    orig, batch = np.empty_like(encoded), np.empty_like(encoded)
    lib().gs_decode_batch_ids_cpu(_p(encoded), C.c_int64(encoded.size),
                                  C.c_int64(stride), _p(orig), _p(batch))
    return orig, batch


def split_indptr(indptr, offset) -> np.ndarray:
    indptr, offset = _i64(indptr), _i64(offset)
    nb = offset.size - 1
    total = int(offset[-1] - offset[0]) + nb
    out = np.empty(total, dtype=np.int64)
    lib().gs_split_indptr_cpu(_p(indptr), _p(offset), C.c_int64(nb),
                              C.c_int64(total), _p(out))
    return out


# ------------------------------------------------------ edge-wise operators
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy_lhs": 4, "copy_rhs": 5, "dot": 6}
REDUCERS = {"sum": 0, "max": 1, "min": 2}


def _view(view):
    kind, a, b = view
    a, b = _i64(a), _i64(b)
    if kind == "coo":
        return 1, a, b, 0, a.size
    return 2, a, b, a.size - 1, b.size


def _feat(t):
    if t is None:
        return None, 0
    t = np.ascontiguousarray(t)
    return t, (1 if t.ndim == 1 else int(np.prod(t.shape[1:])))


def _em(edge_map):
    return None if edge_map is None else _i64(edge_map)


def sddmm(view, op, lhs, rhs, lhs_target, rhs_target, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    lhs, llen = _feat(lhs)
    rhs, rlen = _feat(rhs)
    ref = lhs if lhs is not None else rhs
    flen = llen if lhs is not None else rlen
    red = flen if op == "dot" else 1
    out_len = flen // red
    out = np.zeros((nnz,) if ref.ndim == 1 else (nnz, out_len), dtype=ref.dtype)
    em = _em(edge_map)
    lib().gs_sddmm_cpu(C.c_int(fmt), _p(a), _p(b), C.c_int64(nmaj), C.c_int64(nnz), _p(em),
                       C.c_int(OPS[op]), C.c_int(0 if ref.dtype == np.float32 else 1),
                       _p(lhs), _p(rhs), _p(out), C.c_int(lhs_target), C.c_int(rhs_target),
                       C.c_int64(llen), C.c_int64(rlen), C.c_int64(out_len), C.c_int64(red),
                       None, None)
    return out


def fused_u_op_v(view, op, lhs1, rhs1, lhs2, rhs2):
    fmt, a, b, nmaj, nnz = _view(view)
    lhs1, llen = _feat(lhs1)
    rhs1, rlen = _feat(rhs1)
    lhs2, _ = _feat(lhs2)
    rhs2, _ = _feat(rhs2)
    out1 = np.zeros((nnz,) if lhs1.ndim == 1 else (nnz, llen), dtype=lhs1.dtype)
    out2 = np.zeros_like(out1)
    lib().gs_fused_u_op_v_cpu(C.c_int(fmt), _p(a), _p(b), C.c_int64(nmaj), C.c_int64(nnz),
                              C.c_int(OPS[op]), C.c_int(0 if lhs1.dtype == np.float32 else 1),
                              _p(lhs1), _p(rhs1), _p(out1), _p(lhs2), _p(rhs2), _p(out2),
                              C.c_int64(llen), C.c_int64(rlen), C.c_int64(llen), C.c_int64(1),
                              None, None)
    return out1, out2


def spmm(view, op, reduce, ufeat, efeat, u_target, n_out, edge_map=None, want_arg=False):
    fmt, a, b, nmaj, nnz = _view(view)
    ufeat, ulen = _feat(ufeat)
    efeat, elen = _feat(efeat)
    ref = ufeat if (ufeat is not None and op != "copy_rhs") else efeat
    flen = ulen if ref is ufeat else elen
    shape = (n_out,) if ref.ndim == 1 else (n_out, flen)
    out = np.zeros(shape, dtype=np.float32)
    arg_u = np.zeros(shape, dtype=np.int64) if want_arg else None
    arg_e = np.zeros(shape, dtype=np.int64) if want_arg else None
    em = _em(edge_map)
    lib().gs_spmm_cpu(C.c_int(fmt), _p(a), _p(b), C.c_int64(nmaj), C.c_int64(nnz), _p(em),
                      C.c_int(OPS[op]), C.c_int(REDUCERS[reduce]), _p(ufeat), _p(efeat),
                      _p(out), _p(arg_u), _p(arg_e), C.c_int(u_target), C.c_int64(ulen),
                      C.c_int64(elen), C.c_int64(flen), None, None)
    return (out, arg_u, arg_e) if want_arg else out


def e_square_sum(view, efeat, u_target, n_out, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    efeat, elen = _feat(efeat)
    out = np.zeros((n_out,) if efeat.ndim == 1 else (n_out, elen), dtype=np.float32)
    em = _em(edge_map)
    lib().gs_e_square_sum_cpu(C.c_int(fmt), _p(a), _p(b), C.c_int64(nmaj), C.c_int64(nnz),
                              _p(em), _p(efeat), _p(out), C.c_int(u_target), C.c_int64(elen))
    return out


def e_div_u_sum(view, ufeat, efeat, u_target, n_out, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    ufeat, ulen = _feat(ufeat)
    efeat, elen = _feat(efeat)
    out = np.zeros((n_out,) if efeat.ndim == 1 else (n_out, elen), dtype=np.float32)
    em = _em(edge_map)
    lib().gs_e_div_u_sum_cpu(C.c_int(fmt), _p(a), _p(b), C.c_int64(nmaj), C.c_int64(nnz),
                             _p(em), _p(ufeat), _p(efeat), _p(out), C.c_int(u_target),
                             C.c_int64(elen))
    return out


def minor_slice(ids, picked, indptr=None, edge_major=None, with_major=True):
    ids, picked = _i64(ids), _i64(picked)
    nmaj = 0
    out_indptr = None
    if indptr is not None:
        indptr = _i64(indptr)
        nmaj = indptr.size - 1
        out_indptr = np.empty(nmaj + 1, dtype=np.int64)
    if edge_major is not None:
        edge_major = _i64(edge_major)
    total = np.zeros(1, dtype=np.int64)
    args = [_p(ids), C.c_int64(ids.size), _p(picked), C.c_int64(picked.size), _p(indptr),
            C.c_int64(nmaj), _p(edge_major), _p(out_indptr), _p(total)]
    lib().gs_minor_slice_cpu(*args, None, None, None)
    kept = int(total[0])
    out_minor = np.empty(kept, dtype=np.int64)
    out_select = np.empty(kept, dtype=np.int64)
    want_major = with_major and (indptr is not None or edge_major is not None)
    out_major = np.empty(kept, dtype=np.int64) if want_major else None
    lib().gs_minor_slice_cpu(*args, _p(out_major), _p(out_minor), _p(out_select))
    return out_indptr, out_major, out_minor, out_select


# --------------------------------------------------------- weighted sampling
def neg_log2_unit(r64) -> float:
    f = lib().gs_neg_log2_unit_cpu
    f.restype = C.c_double
    return f(C.c_uint64(r64))


def weighted_key(seed, call_id, pos, draw, w) -> float:
    f = lib().gs_weighted_key_cpu
    f.restype = C.c_double
    return f(C.c_uint64(seed), C.c_uint64(call_id), C.c_uint64(pos), C.c_uint64(draw),
             C.c_float(w))


def weight_cdf(indptr, probs, indices=None, num_rows=None) -> np.ndarray:
    indptr = _i64(indptr)
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    if indices is not None:
        indices = _i64(indices)
        if num_rows is None:
            num_rows = int(indices.max()) + 1 if indices.size else 0
    cdf = np.empty(probs.size + 1, dtype=np.int64)
    lib().gs_weight_cdf_build_cpu(_p(indptr), C.c_int64(indptr.size - 1), _p(indices),
                                  C.c_int64(num_rows or 0), _p(probs),
                                  C.c_int64(probs.size), _p(cdf))
    return cdf


def sample_weighted(indptr, indices, probs, column_ids, fanout, replace=False, seed=7777,
                    call_id=0, with_coo=True, cdf=None):
    indptr, indices = _i64(indptr), _i64(indices)
    if cdf is not None:
        cdf = _i64(cdf)
        num_cols = indptr.size - 1
        if column_ids is not None:
            column_ids = _i64(column_ids)
        n = column_ids.size if column_ids is not None else num_cols
        sub_indptr = col_count(indptr, column_ids, fanout, replace, n)
        nnz = int(sub_indptr[-1])
        out_idx, out_sel = np.empty(nnz, dtype=np.int64), np.empty(nnz, dtype=np.int64)
        out_col = np.empty(nnz, dtype=np.int64) if with_coo else None
        lib().gs_csc_col_sample_weighted_cdf_fill_cpu(
            _p(indptr), C.c_int64(num_cols), _p(indices), _p(cdf), _p(column_ids),
            C.c_int64(n), C.c_int64(fanout), C.c_int(int(replace)), C.c_uint64(seed),
            C.c_uint64(call_id), _p(sub_indptr), _p(out_col), _p(out_idx), _p(out_sel))
        return sub_indptr, out_col, out_idx, out_sel
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    num_cols = indptr.size - 1
    if column_ids is not None:
        column_ids = _i64(column_ids)
        n = column_ids.size
    else:
        n = num_cols
    sub_indptr = col_count(indptr, column_ids, fanout, replace, n)
    nnz = int(sub_indptr[-1])
    out_idx = np.empty(nnz, dtype=np.int64)
    out_sel = np.empty(nnz, dtype=np.int64)
    out_col = np.empty(nnz, dtype=np.int64) if with_coo else None
    lib().gs_csc_col_sample_weighted_fill_cpu(
        _p(indptr), C.c_int64(num_cols), _p(indices), _p(probs), _p(column_ids),
        C.c_int64(n), C.c_int64(fanout), C.c_int(int(replace)), C.c_uint64(seed),
        C.c_uint64(call_id), _p(sub_indptr), _p(out_col), _p(out_idx), _p(out_sel))
    return sub_indptr, out_col, out_idx, out_sel


def list_sample_uniform(n, num_picks, replace=False, algo=0, seed=7777, call_id=0):
    f = lib().gs_list_sample_uniform_cpu
    f.restype = C.c_int64
    args = [C.c_int64(n), C.c_int64(num_picks), C.c_int(int(replace)), C.c_int(algo),
            C.c_uint64(seed), C.c_uint64(call_id)]
    count = f(*args, None)
    out = np.empty(count, dtype=np.int64)
    f(*args, _p(out))
    return out


def list_sample_weighted(probs, num_picks, replace=False, range_=None, seed=7777, call_id=0):
    """-> (index, out_range)"""
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    f = lib().gs_list_sample_weighted_cpu
    f.restype = C.c_int64
    nseg = 1
    if range_ is not None:
        range_ = _i64(range_)
        nseg = range_.size - 1
    out_range = np.empty(nseg + 1, dtype=np.int64)
    args = [_p(probs), C.c_int64(probs.size), C.c_int64(num_picks), C.c_int(int(replace)),
            _p(range_), C.c_int64(nseg), C.c_uint64(seed), C.c_uint64(call_id)]
    total = f(*args, None, _p(out_range))
    out = np.empty(total, dtype=np.int64)
    f(*args, _p(out), _p(out_range))
    return out, out_range


# --------------------------------------------------------------------- walks
def random_walk(indptr, indices, seeds, walk_length, seed=7777, call_id=0):
    indptr, indices, seeds = _i64(indptr), _i64(indices), _i64(seeds)
    out = np.empty((walk_length + 1, seeds.size), dtype=np.int64)
    lib().gs_random_walk_cpu(_p(indptr), _p(indices), C.c_int64(indptr.size - 1), _p(seeds),
                             C.c_int64(seeds.size), C.c_int64(walk_length), C.c_uint64(seed),
                             C.c_uint64(call_id), _p(out))
    return out


def node2vec(indptr, indices, seeds, walk_length, p, q, seed=7777, call_id=0):
    indptr, indices, seeds = _i64(indptr), _i64(indices), _i64(seeds)
    out = np.empty((walk_length + 1, seeds.size), dtype=np.int64)
    lib().gs_node2vec_cpu(_p(indptr), _p(indices), C.c_int64(indptr.size - 1), _p(seeds),
                          C.c_int64(seeds.size), C.c_int64(walk_length), C.c_double(p),
                          C.c_double(q), C.c_uint64(seed), C.c_uint64(call_id), _p(out))
    return out


def segment_sort(indptr, keys):
    indptr, keys = _i64(indptr), _i64(keys)
    out = np.empty_like(keys)
    lib().gs_segment_sort_i64_cpu(_p(indptr), C.c_int64(indptr.size - 1), _p(keys), _p(out))
    return out


def gather_rows(table, ids):
    """out[i] = table[ids[i]] along the first axis (any dtype, any row shape);
    returns (out, number of ids outside the table, whose rows are zero)."""
    table = np.ascontiguousarray(table)
    ids = _i64(ids)
    out = np.empty((ids.size,) + table.shape[1:], dtype=table.dtype)
    row_bytes = int(table.dtype.itemsize * np.prod(table.shape[1:], dtype=np.int64))
    bad = C.c_int64(0)
    lib().gs_gather_rows_cpu(table.ctypes.data_as(C.c_void_p), C.c_int64(table.shape[0]),
                             C.c_int64(row_bytes), _p(ids), C.c_int64(ids.size),
                             out.ctypes.data_as(C.c_void_p), C.byref(bad))
    return out, bad.value


def coo_sort(major):
    major = _i64(major)
    out, perm = np.empty_like(major), np.empty_like(major)
    lib().gs_coo_sort_cpu(_p(major), C.c_int64(major.size), _p(out), _p(perm))
    return out, perm


def coo_to_csc(row, col, num_cols):
    """(indptr, row ids in column order, edge positions in column order)."""
    sorted_col, perm = coo_sort(col)
    return sorted_to_indptr(sorted_col, num_cols), _i64(row)[perm], perm
