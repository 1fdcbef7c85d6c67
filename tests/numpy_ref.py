"""Independent NumPy closed forms for the deterministic operators.  They share
no code with the oracle: a disagreement between the two is a bug in one."""
import numpy as np


def col_slice(indptr, indices, cols):
    indptr, indices, cols = map(np.asarray, (indptr, indices, cols))
    deg = indptr[cols + 1] - indptr[cols]
    sub_indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    sel = np.concatenate([np.arange(indptr[c], indptr[c + 1]) for c in cols]
                         + [np.empty(0, dtype=np.int64)]).astype(np.int64)
    coo_col = np.repeat(np.arange(len(cols)), deg).astype(np.int64)
    return sub_indptr, coo_col, indices[sel], sel


def first_occurrence_unique(x):
    x = np.asarray(x)
    _, first = np.unique(x, return_index=True)
    return x[np.sort(first)]


def relabel(unique, x):
    lut = {int(v): i for i, v in enumerate(unique)}
    return np.array([lut[int(v)] for v in x], dtype=np.int64)
