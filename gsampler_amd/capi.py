"""ctypes binding of the C ABI declared in include/gsampler_hip.h.

Two layers:

* ``lib()`` returns the loaded ``libgsampler_hip.so`` with argument types set,
  one attribute per exported symbol.  Loading fails loudly when the library has
  not been built -- there is no fallback path.
* thin helpers (``col_count``, ``col_slice``, ``sample_uniform``,
  ``unique_relabel`` ...) that take CUDA ``torch.Tensor`` arguments, allocate
  outputs and workspaces with torch (plumbing only) and launch on torch's
  current HIP stream.  They are what the tests and the benchmark call; the
  C++ operator library (``libgs.so``) binds the same symbols directly.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgsampler_hip.so")

GS_OK = 0
ALGO_AUTO, ALGO_RESERVOIR, ALGO_FLOYD = 0, 1, 2

_i64 = C.c_int64
_u64 = C.c_uint64
_p = C.c_void_p
_sz = C.c_size_t
_int = C.c_int

# name -> (restype, argtypes); the single source of truth for the loader and
# for the "every declared symbol is exported" test.
SIGNATURES = {
    "gs_last_error": (C.c_char_p, []),
    "gs_abi_version": (_int, []),
    "gs_profile_enable": (None, [_int]),
    "gs_profile_reset": (None, []),
    "gs_profile_count": (_int, []),
    "gs_profile_get": (_int, [_int, C.c_char_p, _sz, C.POINTER(C.c_longlong),
                              C.POINTER(C.c_double)]),
    "gs_copy_i64": (_int, [_p, _i64, _p, _p]),
    "gs_scan_workspace_bytes": (_sz, [_i64]),
    "gs_exclusive_scan_i64": (_int, [_p, _p, _i64, _p, _sz, _p]),
    "gs_csc_col_count": (_int, [_p, _i64, _p, _i64, _i64, _int, _p, _p, _p, _p, _sz, _p]),
    "gs_csc_col_count_static": (_int, [_p, _i64, _p, _i64, _i64, _int, _p, _p]),
    "gs_csc_col_slice_fill": (_int, [_p, _i64, _p, _p, _i64, _p, _i64, _p, _i64,
                                     _i64, _p, _p, _p, _p]),
    "gs_csc_col_sample_uniform_fill": (_int, [_p, _i64, _p, _p, _i64, _i64, _int,
                                              _int, _u64, _u64, _p, _p, _p, _p, _p,
                                              _p, _i64, _p]),
    "gs_csc_col_sample_uniform_fill_i32": (_int, [_p, _i64, _p, _p, _i64, _i64, _int,
                                                  _int, _u64, _u64, _p, _p, _p, _p, _p,
                                                  _p, _i64, _p]),
    "gs_unique_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "gs_unique_count": (_int, [_p, _p, _i64, _p, _p, _i64, _i64, _p, _p, _p, _sz, _p]),
    "gs_unique_fill": (_int, [_p, _p, _i64, _p, _p, _i64, _i64, _p, _p, _p, _sz, _p]),
    "gs_unique_relabel": (_int, [_p, _p, _i64, _p, _p, _i64, _i64, _p, _p, _p, _p, _int, _p,
                                 _sz, _p]),
    "gs_unique_fill_relabel": (_int, [_p, _p, _i64, _p, _p, _i64, _i64, _p, _p, _p, _p, _p, _p,
                                      _int, _p, _sz, _p]),
    "gs_csc2coo": (_int, [_p, _i64, _i64, _p, _p]),
    "gs_sorted_to_indptr": (_int, [_p, _i64, _i64, _p, _p]),
    "gs_decode_batch_ids": (_int, [_p, _i64, _i64, _p, _p, _p]),
    "gs_split_indptr": (_int, [_p, _p, _i64, _i64, _p, _p]),
    "gs_batch_seeds_distinct": (_int, [_p, _p, _p, _p, _i64, _p, _p]),
    "gs_first_position": (_int, [_p, _i64, _i64, _p, _p]),
    "gs_csc_col_slice_values": (_int, [_p, _p, _i64, _p, _i64, _p, _i64, _p, _p]),
    "gs_list_labels": (_int, [_p, _i64, _p, _p, _i64, _p, _p, _p, _p, _p, _p]),
    "gs_gather_rows": (_int, [_p, _i64, _i64, _p, _i64, _p, _p, _p]),
    "gs_coo_sort_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_coo_sort_flag_offset": (_i64, [_i64, _i64]),
    "gs_coo_sort": (_int, [_p, _i64, _i64, _p, _p, _p, _sz, _p]),
    "gs_sddmm": (_int, [_int, _p, _p, _i64, _i64, _p, _int, _int, _p, _p, _p, _int, _int,
                        _i64, _i64, _i64, _i64, _p, _p, _p]),
    "gs_fused_u_op_v": (_int, [_int, _p, _p, _i64, _i64, _p, _int, _int, _p, _p, _p, _p, _p,
                               _p, _i64, _i64, _i64, _i64, _p, _p, _p]),
    "gs_spmm_workspace_bytes": (_sz, [_int, _i64, _i64]),
    "gs_spmm": (_int, [_int, _p, _p, _i64, _i64, _p, _int, _int, _p, _p, _p, _p, _p, _int,
                       _i64, _i64, _i64, _p, _p, _i64, _p, _sz, _p]),
    "gs_e_square_sum": (_int, [_int, _p, _p, _i64, _i64, _p, _p, _p, _int, _i64, _i64, _p,
                               _sz, _p]),
    "gs_e_div_u_sum": (_int, [_int, _p, _p, _i64, _i64, _p, _p, _p, _p, _int, _i64, _i64,
                              _p, _sz, _p]),
    "gs_minor_slice_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_minor_slice_count": (_int, [_p, _i64, _p, _i64, _p, _i64, _p, _p, _p, _sz, _p]),
    "gs_minor_slice_fill": (_int, [_p, _i64, _i64, _p, _i64, _p, _p, _p, _p, _p, _sz, _p]),
    "gs_col_row_slice_count": (_int, [_p, _p, _p, _p, _p, _i64, _p, _i64, _p, _i64, _p, _p, _p,
                                      _sz, _p]),
    "gs_col_row_slice_fill": (_int, [_p, _p, _p, _i64, _p, _i64, _i64, _p, _p, _p, _p, _sz, _p]),
    "gs_probe_stream_copy": (_int, [_p, _p, _i64, _p]),
    "gs_probe_line_gather": (_int, [_p, _i64, _i64, _u64, _int, _p, _p]),
    "gs_probe_sample_uniform": (_int, [_p, _i64, _p, _p, _i64, _i64, _int, _i64, _u64, _u64, _p,
                                       _p, _p, _p, _p, _p]),
    "gs_sliced_e_square_sum_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_sliced_e_square_sum": (_int, [_p, _p, _p, _p, _i64, _p, _i64, _p, _p, _p, _i64, _p, _sz,
                                      _p]),
    "gs_weight_cdf_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_weight_cdf_build": (_int, [_p, _i64, _p, _i64, _p, _i64, _p, _p, _sz, _p]),
    "gs_csc_col_sample_weighted_fill": (_int, [_p, _i64, _p, _p, _p, _p, _i64, _i64, _int, _u64,
                                               _u64, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _p]),
    "gs_weighted_key_probe": (_int, [_u64, _u64, _u64, _u64, C.c_float, _u64, _p, _p]),
    "gs_list_sample_uniform": (_int, [_i64, _i64, _int, _int, _u64, _u64, _p, _p]),
    "gs_list_sample_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_list_sample_weighted_count": (_int, [_p, _i64, _i64, _i64, _int, _p, _p, _sz, _p]),
    "gs_list_sample_weighted_fill": (_int, [_p, _p, _i64, _i64, _i64, _int, _u64, _u64, _p,
                                            _i64, _p, _p, _sz, _p]),
    "gs_random_walk": (_int, [_p, _p, _i64, _p, _i64, _i64, _u64, _u64, _p, _p]),
    "gs_node2vec": (_int, [_p, _p, _i64, _p, _i64, _i64, C.c_double, C.c_double, _u64, _u64,
                           _p, _p]),
    "gs_segment_sort_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "gs_segment_sort_i64": (_int, [_p, _i64, _p, _p, _i64, _i64, _p, _sz, _p]),
}

_lib = None


class GsError(RuntimeError):
    pass


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GsError(
                f"{LIB_PATH} is missing: build it with "
                "`make -C gsampler_amd/csrc` (or __graft_entry__.build())")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> None:
    if rc != GS_OK:
        raise GsError(f"gsampler_hip error {rc}: {lib().gs_last_error().decode()}")


# --------------------------------------------------------------- plumbing
def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    return t.data_ptr() if t.numel() > 0 else None


def _stream() -> int:
    """Raw handle of torch's current stream on the current device (the direct
    binding: torch.cuda.current_stream() spends microseconds in Python per call,
    which a step of a few dozen launches notices)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _i64t(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int64 or not t.is_cuda:
        raise GsError(f"{name} must be a CUDA int64 tensor, got {t.dtype} on {t.device}")
    return t.contiguous()


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


class _Count:
    """A count on its way from the device to the host.  The kernel that produces
    it stores it into a word of pinned host memory as well (the `mirror` argument
    of the count entry points), so the host only waits for an event recorded
    behind that kernel, and only when it needs the value.  Kernels launched in
    between (into buffers sized by an upper bound) keep the GPU busy meanwhile.

        c = _Count(); entry_point(..., c.mirror(), ...); c.arm(); ...; c.get()

    A mirror of `words` entries (a whole offsets array) delivers its last one."""
    _slots = None
    _next = 0
    _RING = 64
    _WIDTH = 4096          # words per slot: offset arrays up to this many entries

    def __init__(self, words: int = 1):
        cls = _Count
        if words > cls._WIDTH:
            raise GsError(f"a mirrored offsets array holds at most {cls._WIDTH} entries")
        if cls._slots is None:
            cls._slots = torch.empty((cls._RING, cls._WIDTH), dtype=torch.int64).pin_memory()
        self._slot = cls._slots[cls._next % cls._RING]
        self._words = words
        cls._next += 1
        self._ticket = cls._next
        self._event = None
        self._value = None

    def mirror(self) -> int:
        return self._slot.data_ptr()

    def arm(self) -> "_Count":
        self._event = torch.cuda.Event()
        self._event.record()
        return self

    def get(self) -> int:
        if self._value is None:
            # helpers read their counts before they return; the ring is 64 deep
            if _Count._next - self._ticket >= _Count._RING:
                raise GsError("a pending count was overwritten by later requests")
            self._event.synchronize()
            self._value = int(self._slot[self._words - 1])
        return self._value


class _Fetched:
    """The last entry of a device array, read with a blocking copy on first use."""

    def __init__(self, prefix: torch.Tensor):
        self._prefix, self._value = prefix, None

    def get(self) -> int:
        if self._value is None:
            self._value = int(self._prefix[-1].item())
        return self._value


# Outputs are sized by an upper bound (and trimmed afterwards) only up to this
# many elements; beyond it the count is awaited first.
_BOUND_LIMIT = 1 << 26


# -------------------------------------------------------------- profiling
def profile_enable(on: bool) -> None:
    lib().gs_profile_enable(int(on))


def profile_reset() -> None:
    lib().gs_profile_reset()


def profile_totals() -> dict:
    """{kernel name: (launches, total milliseconds)} since the last reset."""
    l = lib()
    out = {}
    for i in range(l.gs_profile_count()):
        name = C.create_string_buffer(128)
        calls, ms = C.c_longlong(0), C.c_double(0.0)
        check(l.gs_profile_get(i, name, 128, C.byref(calls), C.byref(ms)))
        out[name.value.decode()] = (calls.value, ms.value)
    return out


# ---------------------------------------------------------------- helpers
def exclusive_scan(x: torch.Tensor) -> torch.Tensor:
    x = _i64t(x, "x")
    out = torch.empty_like(x)
    n = x.numel()
    ws = _workspace(lib().gs_scan_workspace_bytes(n), x.device)
    check(lib().gs_exclusive_scan_i64(_ptr(x), _ptr(out), n, ws.data_ptr(),
                                      ws.numel(), _stream()))
    return out


def col_count(indptr: torch.Tensor, column_ids: Optional[torch.Tensor],
              fanout: int, replace: bool,
              num_items: Optional[int] = None, count: Optional[_Count] = None,
              col_span: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sub_indptr[num_items + 1] for slicing (fanout < 0) or sampling.  With
    `count` the edge total is also on its way to the host when this returns;
    `col_span` (int64[num_items]) receives every column's start and degree in one
    word, which the sampler fills take in place of the column pointer."""
    indptr = _i64t(indptr, "indptr")
    num_cols = indptr.numel() - 1
    if column_ids is not None:
        column_ids = _i64t(column_ids, "column_ids")
        num_items = column_ids.numel()
    elif num_items is None:
        num_items = num_cols
    sub_indptr = torch.empty(num_items + 1, dtype=torch.int64, device=indptr.device)
    ws = _workspace(lib().gs_scan_workspace_bytes(num_items + 1), indptr.device)
    check(lib().gs_csc_col_count(_ptr(indptr), num_cols, _ptr(column_ids),
                                 num_items, fanout, int(replace),
                                 sub_indptr.data_ptr(), count.mirror() if count else None,
                                 _ptr(col_span), ws.data_ptr(), ws.numel(), _stream()))
    if count:
        count.arm()
    return sub_indptr


def col_slice(indptr, indices, column_ids, with_coo=True, batch_ptr=None,
              encode_stride=0):
    """A[:, column_ids] -> (sub_indptr, coo_col | None, sub_indices, select_index)."""
    indptr, indices = _i64t(indptr, "indptr"), _i64t(indices, "indices")
    column_ids = _i64t(column_ids, "column_ids")
    num_cols = indptr.numel() - 1
    n = column_ids.numel()
    sub_indptr = col_count(indptr, column_ids, -1, False)
    nnz = int(sub_indptr[-1].item())
    dev = indptr.device
    out_idx = torch.empty(nnz, dtype=torch.int64, device=dev)
    out_sel = torch.empty(nnz, dtype=torch.int64, device=dev)
    out_col = torch.empty(nnz, dtype=torch.int64, device=dev) if with_coo else None
    nb = 0
    if batch_ptr is not None:
        batch_ptr = _i64t(batch_ptr, "batch_ptr")
        nb = batch_ptr.numel() - 1
    check(lib().gs_csc_col_slice_fill(_ptr(indptr), num_cols, _ptr(indices),
                                      _ptr(column_ids), n, sub_indptr.data_ptr(),
                                      nnz, _ptr(batch_ptr), nb, encode_stride,
                                      _ptr(out_col), _ptr(out_idx), _ptr(out_sel),
                                      _stream()))
    return sub_indptr, out_col, out_idx, out_sel


def col_slice_values(indptr, column_ids, sub_indptr, values):
    """Per-edge values (4- or 8-byte elements) of A[:, column_ids], from the parent's
    `values` and the slice's `sub_indptr`."""
    indptr, sub_indptr = _i64t(indptr, "indptr"), _i64t(sub_indptr, "sub_indptr")
    if column_ids is not None:
        column_ids = _i64t(column_ids, "column_ids")
    values = values.contiguous()
    n = sub_indptr.numel() - 1
    nnz = int(sub_indptr[-1].item())
    out = torch.empty(nnz, dtype=values.dtype, device=values.device)
    check(lib().gs_csc_col_slice_values(_ptr(indptr), _ptr(column_ids), n, _ptr(sub_indptr), nnz,
                                        values.data_ptr(), values.element_size(),
                                        out.data_ptr(), _stream()))
    return out


def sample_uniform(indptr, indices, column_ids, fanout, replace=False,
                   algo=ALGO_AUTO, seed=7777, call_id=0, with_coo=True, col_batch_ptr=None,
                   spans=True):
    """Uniform per-column sampling, fused with the slice when column_ids is given.

    `indices` may be the matrix's int32 copy of the row ids (same outputs).
    `col_batch_ptr` (offsets that cut the columns into batches): coo_col then holds
    every column's place inside its batch instead of its place in the call.
    `spans`: the count pass leaves every column's start and degree for the fill
    pass, which then does not look the column pointer up again (same outputs).

    -> (sub_indptr, coo_col | None, sub_indices, select_index)
    """
    indptr = _i64t(indptr, "indptr")
    fill = lib().gs_csc_col_sample_uniform_fill
    if indices.dtype == torch.int32 and indices.is_cuda:
        indices, fill = indices.contiguous(), lib().gs_csc_col_sample_uniform_fill_i32
    else:
        indices = _i64t(indices, "indices")
    num_cols = indptr.numel() - 1
    if column_ids is not None:
        column_ids = _i64t(column_ids, "column_ids")
        n = column_ids.numel()
    else:
        n = num_cols
    if col_batch_ptr is not None:
        col_batch_ptr = _i64t(col_batch_ptr, "col_batch_ptr")
    count = _Count()
    dev = indptr.device
    col_span = torch.empty(n, dtype=torch.int64, device=dev) if spans else None
    sub_indptr = col_count(indptr, column_ids, fanout, replace, n, count, col_span)
    bound = n * fanout                       # no column yields more than fanout edges
    size = bound if bound <= _BOUND_LIMIT else count.get()
    out_idx = torch.empty(size, dtype=torch.int64, device=dev)
    out_sel = torch.empty(size, dtype=torch.int64, device=dev)
    out_col = torch.empty(size, dtype=torch.int64, device=dev) if with_coo else None
    if size > 0:
        check(fill(
            _ptr(indptr), num_cols, _ptr(indices), _ptr(column_ids), n, fanout,
            int(replace), algo, seed, call_id, sub_indptr.data_ptr(), _ptr(col_span),
            _ptr(out_col), out_idx.data_ptr(), out_sel.data_ptr(), _ptr(col_batch_ptr),
            col_batch_ptr.numel() - 1 if col_batch_ptr is not None else 0, _stream()))
    nnz = count.get()
    return (sub_indptr, out_col[:nnz] if with_coo else None, out_idx[:nnz], out_sel[:nnz])


def unique_relabel(seeds, rows, seeds_ptr=None, rows_ptr=None, edge_col=None,
                   want_row=True, want_col=True, col_indptr=None, fused=True, out_col=None):
    """First-occurrence unique of seeds_b ++ rows_b per batch, plus relabel.

    The column of an edge comes from `edge_col` (a position into `seeds` per
    edge) or, for edges grouped by column, from `col_indptr` (len(seeds) + 1).
    `fused`: frontier and labels from one launch (gs_unique_fill_relabel) instead
    of gs_unique_fill followed by gs_unique_relabel; same outputs.
    `out_col` (with col_indptr): the column labels as a sampler wrote them when it was
    given the batch offsets of its columns (every column's place inside its batch);
    batches with distinct seeds keep them, the others are rewritten in place.

    -> (unique, unique_ptr, out_row | None, out_col | None)
    """
    seeds, rows = _i64t(seeds, "seeds"), _i64t(rows, "rows")
    dev = seeds.device
    S, E = seeds.numel(), rows.numel()
    if seeds_ptr is not None:
        seeds_ptr, rows_ptr = _i64t(seeds_ptr, "seeds_ptr"), _i64t(rows_ptr, "rows_ptr")
        B = seeds_ptr.numel() - 1
    else:
        B = 1
    l = lib()
    ws = _workspace(l.gs_unique_workspace_bytes(S, E, B), dev)
    unique_ptr = torch.empty(B + 1, dtype=torch.int64, device=dev)
    sp = seeds_ptr.data_ptr() if seeds_ptr is not None else None
    rp = rows_ptr.data_ptr() if rows_ptr is not None else None
    count = _Count(B + 1) if B + 1 <= _Count._WIDTH else None
    check(l.gs_unique_count(_ptr(seeds), sp, S, _ptr(rows), rp, E, B,
                            unique_ptr.data_ptr(), count.mirror() if count else None,
                            ws.data_ptr(), ws.numel(), _stream()))
    count = count.arm() if count else _Fetched(unique_ptr)
    size = S + E if S + E <= _BOUND_LIMIT else count.get()   # U <= S + E
    unique = torch.empty(size, dtype=torch.int64, device=dev)
    want_col = want_col and (edge_col is not None or col_indptr is not None)
    out_row = torch.empty(E, dtype=torch.int64, device=dev) if want_row else None
    prefilled = 0
    if out_col is not None:
        if col_indptr is None or not want_col:
            raise ValueError("unique_relabel: out_col goes with col_indptr")
        out_col = _i64t(out_col, "out_col")
        if out_col.numel() != E:
            raise ValueError(f"unique_relabel: out_col has {out_col.numel()} entries for {E} edges")
        prefilled = 1
    else:
        out_col = torch.empty(E, dtype=torch.int64, device=dev) if want_col else None
    if edge_col is not None:
        edge_col = _i64t(edge_col, "edge_col")
    if col_indptr is not None:
        if edge_col is not None:
            raise ValueError("unique_relabel: give edge_col or col_indptr, not both")
        col_indptr = _i64t(col_indptr, "col_indptr")
        if col_indptr.numel() != S + 1:
            raise ValueError(f"unique_relabel: col_indptr has {col_indptr.numel()} entries "
                             f"for {S} seeds")
    if (want_row or want_col) and fused:
        check(l.gs_unique_fill_relabel(_ptr(seeds), sp, S, _ptr(rows), rp, E, B,
                                       unique_ptr.data_ptr(), _ptr(unique), _ptr(edge_col),
                                       _ptr(col_indptr), _ptr(out_row), _ptr(out_col), prefilled,
                                       ws.data_ptr(), ws.numel(), _stream()))
    else:
        check(l.gs_unique_fill(_ptr(seeds), sp, S, _ptr(rows), rp, E, B,
                               unique_ptr.data_ptr(), _ptr(unique), ws.data_ptr(),
                               ws.numel(), _stream()))
        if want_row or want_col:
            check(l.gs_unique_relabel(_ptr(seeds), sp, S, _ptr(rows), rp, E, B,
                                      _ptr(edge_col), _ptr(col_indptr), _ptr(out_row),
                                      _ptr(out_col), prefilled, ws.data_ptr(), ws.numel(),
                                      _stream()))
    total = count.get()
    return unique[:total], unique_ptr, out_row, out_col


def csc2coo(indptr: torch.Tensor, nnz: Optional[int] = None) -> torch.Tensor:
    """Column id of every edge of a CSC matrix."""
    indptr = _i64t(indptr, "indptr")
    if nnz is None:
        nnz = int(indptr[-1].item())
    out = torch.empty(nnz, dtype=torch.int64, device=indptr.device)
    check(lib().gs_csc2coo(_ptr(indptr), indptr.numel() - 1, nnz, _ptr(out), _stream()))
    return out


def sorted_to_indptr(sorted_ids: torch.Tensor, num_cols: int) -> torch.Tensor:
    sorted_ids = _i64t(sorted_ids, "sorted_ids")
    out = torch.empty(num_cols + 1, dtype=torch.int64, device=sorted_ids.device)
    check(lib().gs_sorted_to_indptr(_ptr(sorted_ids), sorted_ids.numel(), num_cols,
                                    out.data_ptr(), _stream()))
    return out


def first_position(ids: torch.Tensor, num_ids: int) -> torch.Tensor:
    """first[r] = smallest e with ids[e] == r, INT64_MAX when r does not occur."""
    ids = _i64t(ids, "ids")
    out = torch.empty(num_ids, dtype=torch.int64, device=ids.device)
    check(lib().gs_first_position(_ptr(ids), ids.numel(), num_ids, _ptr(out), _stream()))
    return out


LIST_LABELS_MAX_KEYS = 2048


def list_labels(seeds, list_ids, first_pos):
    """Frontier and labels of a matrix whose rows are positions in `list_ids`:
    the unique of seeds ++ list_ids[row[e]] in first-occurrence order, given the
    first edge of every listed id (first_position).

    -> (frontier, list_label, seed_label)
    """
    seeds, list_ids = _i64t(seeds, "seeds"), _i64t(list_ids, "list_ids")
    first_pos = _i64t(first_pos, "first_pos")
    S, R = seeds.numel(), list_ids.numel()
    if first_pos.numel() != R:
        raise ValueError(f"list_labels: {first_pos.numel()} first positions for {R} ids")
    dev = list_ids.device
    frontier = torch.empty(S + R, dtype=torch.int64, device=dev)
    list_label = torch.empty(R, dtype=torch.int64, device=dev)
    seed_label = torch.empty(S, dtype=torch.int64, device=dev)
    count = _Count()
    check(lib().gs_list_labels(_ptr(seeds), S, _ptr(list_ids), _ptr(first_pos), R,
                               _ptr(frontier), None, count.mirror(), _ptr(list_label),
                               _ptr(seed_label), _stream()))
    count.arm()
    return frontier[:count.get()], list_label, seed_label


def coo_sort(major: torch.Tensor, num_major: int, verify: bool = True):
    """Stable sort of edge positions by their id on the axis to compress:
    (sorted ids, positions).  `verify` waits for the call and raises when the
    sort's gave-up flag is set (a pass stopped waiting for another tile's counts:
    the result is then not fully sorted)."""
    major = _i64t(major, "major")
    n = major.numel()
    out, perm = torch.empty_like(major), torch.empty_like(major)
    ws = _workspace(lib().gs_coo_sort_workspace_bytes(n, num_major), major.device)
    check(lib().gs_coo_sort(_ptr(major), n, num_major, _ptr(out), _ptr(perm), ws.data_ptr(),
                            ws.numel(), _stream()))
    at = lib().gs_coo_sort_flag_offset(n, num_major)
    if verify and n > 0 and at >= 0 and int(ws[at:at + 4].view(torch.int32).item()) != 0:
        raise GsError("coo_sort: a pass gave up waiting for the counts of an earlier tile")
    return out, perm


def coo_to_csc(row: torch.Tensor, col: torch.Tensor, num_cols: int):
    """(indptr, row ids in column order, edge positions in column order)."""
    sorted_col, perm = coo_sort(col, num_cols)
    return sorted_to_indptr(sorted_col, num_cols), gather_rows(_i64t(row, "row"), perm), perm


def gather_rows(table: torch.Tensor, ids: torch.Tensor, count_bad: bool = False):
    """out[i] = table[ids[i]] along the first axis, for any dtype and row shape.
    `table` is a CUDA tensor or a pinned CPU tensor (read in place over the host
    link); the result lives on the device of `ids`.  Ids outside the table give
    zero rows; with `count_bad` the pair (out, number of such ids) is returned."""
    ids = _i64t(ids, "ids")
    if not (table.is_cuda or table.is_pinned()):
        raise GsError("gather_rows: table must be a CUDA tensor or a pinned CPU tensor")
    if table.dim() < 1:
        raise GsError("gather_rows: table needs at least one axis")
    table = table.contiguous()
    out = torch.empty((ids.numel(),) + tuple(table.shape[1:]), dtype=table.dtype,
                      device=ids.device)
    rows, row_bytes = table.shape[0], table.element_size()
    for extent in table.shape[1:]:
        row_bytes *= extent
    bad = torch.empty(1, dtype=torch.int64, device=ids.device) if count_bad else None
    check(lib().gs_gather_rows(table.data_ptr() if table.numel() else None, rows, row_bytes,
                               _ptr(ids), ids.numel(), _ptr(out), _ptr(bad), _stream()))
    return (out, int(bad.item())) if count_bad else out


def decode_batch_ids(encoded: torch.Tensor, stride: int):
    """-> (orig, batch) for ids encoded as id + batch * stride."""
    encoded = _i64t(encoded, "encoded")
    orig, batch = torch.empty_like(encoded), torch.empty_like(encoded)
    check(lib().gs_decode_batch_ids(_ptr(encoded), encoded.numel(), stride,
                                    _ptr(orig), _ptr(batch), _stream()))
    return orig, batch


def split_indptr(indptr: torch.Tensor, offset: torch.Tensor) -> torch.Tensor:
    """Per-batch indptr arrays rebased to 0, concatenated."""
    indptr, offset = _i64t(indptr, "indptr"), _i64t(offset, "offset")
    nb = offset.numel() - 1
    total = int((offset[-1] - offset[0]).item()) + nb
    out = torch.empty(total, dtype=torch.int64, device=indptr.device)
    check(lib().gs_split_indptr(_ptr(indptr), _ptr(offset), nb, total, _ptr(out),
                                _stream()))
    return out


# ------------------------------------------------------ edge-wise operators
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy_lhs": 4, "copy_rhs": 5, "dot": 6}
REDUCERS = {"sum": 0, "max": 1, "min": 2}
FMT_COO, FMT_COMPRESSED = 1, 2


def _view(view):
    """("coo", row, col) or ("csc", indptr, indices) -> ABI structure arguments."""
    kind, a, b = view
    a, b = _i64t(a, "a"), _i64t(b, "b")
    if kind == "coo":
        return FMT_COO, a, b, 0, a.numel()
    return FMT_COMPRESSED, a, b, a.numel() - 1, b.numel()


def _feat(t):
    if t is None:
        return None, 0
    t = t.contiguous()
    return t, (1 if t.dim() == 1 else int(t[0].numel()) if t.shape[0] > 0 else 1)


def _fptr(t):
    return None if t is None or t.numel() == 0 else t.data_ptr()


def sddmm(view, op, lhs, rhs, lhs_target, rhs_target, edge_map=None):
    """Same-shape (or scalar) features, no broadcasting; dot reduces the last dim."""
    fmt, a, b, nmaj, nnz = _view(view)
    lhs, llen = _feat(lhs)
    rhs, rlen = _feat(rhs)
    ref = lhs if lhs is not None else rhs
    flen = llen if lhs is not None else rlen
    red = flen if op == "dot" else 1
    out_len = flen // red
    shape = (nnz,) if ref.dim() == 1 else (nnz, out_len)
    out = torch.zeros(shape, dtype=ref.dtype, device=ref.device)
    dtype = 0 if ref.dtype == torch.float32 else 1
    check(lib().gs_sddmm(fmt, _ptr(a), _ptr(b), nmaj, nnz, _ptr(edge_map), OPS[op], dtype,
                         _fptr(lhs), _fptr(rhs), _fptr(out), lhs_target, rhs_target,
                         llen, rlen, out_len, red, None, None, _stream()))
    return out


def fused_u_op_v(view, op, lhs1, rhs1, lhs2, rhs2, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    lhs1, llen = _feat(lhs1)
    rhs1, rlen = _feat(rhs1)
    lhs2, _ = _feat(lhs2)
    rhs2, _ = _feat(rhs2)
    shape = (nnz,) if lhs1.dim() == 1 else (nnz, llen)
    out1 = torch.zeros(shape, dtype=lhs1.dtype, device=lhs1.device)
    out2 = torch.zeros_like(out1)
    dtype = 0 if lhs1.dtype == torch.float32 else 1
    check(lib().gs_fused_u_op_v(fmt, _ptr(a), _ptr(b), nmaj, nnz, _ptr(edge_map), OPS[op], dtype,
                                _fptr(lhs1), _fptr(rhs1), _fptr(out1), _fptr(lhs2),
                                _fptr(rhs2), _fptr(out2), llen, rlen, llen, 1, None, None,
                                _stream()))
    return out1, out2


def _spmm_workspace(fmt, nnz, n_out, device):
    return _workspace(lib().gs_spmm_workspace_bytes(fmt, nnz, n_out), device)


def spmm(view, op, reduce, ufeat, efeat, u_target, n_out, edge_map=None, want_arg=False):
    fmt, a, b, nmaj, nnz = _view(view)
    ufeat, ulen = _feat(ufeat)
    efeat, elen = _feat(efeat)
    ref = ufeat if (ufeat is not None and op != "copy_rhs") else efeat
    flen = ulen if ref is ufeat else elen
    shape = (n_out,) if ref.dim() == 1 else (n_out, flen)
    out = torch.zeros(shape, dtype=torch.float32, device=ref.device)
    arg_u = arg_e = None
    if want_arg:
        arg_u = torch.zeros(shape, dtype=torch.int64, device=ref.device)
        arg_e = torch.zeros(shape, dtype=torch.int64, device=ref.device)
    ws = _spmm_workspace(fmt, nnz, n_out, out.device)
    check(lib().gs_spmm(fmt, _ptr(a), _ptr(b), nmaj, nnz, _ptr(edge_map), OPS[op],
                        REDUCERS[reduce], _fptr(ufeat), _fptr(efeat), _fptr(out),
                        _ptr(arg_u), _ptr(arg_e), u_target, ulen, elen, flen, None, None,
                        n_out, ws.data_ptr(), ws.numel(), _stream()))
    return (out, arg_u, arg_e) if want_arg else out


def e_square_sum(view, efeat, u_target, n_out, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    efeat, elen = _feat(efeat)
    shape = (n_out,) if efeat.dim() == 1 else (n_out, elen)
    out = torch.zeros(shape, dtype=torch.float32, device=efeat.device)
    ws = _spmm_workspace(fmt, nnz, n_out, out.device)
    check(lib().gs_e_square_sum(fmt, _ptr(a), _ptr(b), nmaj, nnz, _ptr(edge_map),
                                _fptr(efeat), _fptr(out), u_target, elen, n_out,
                                ws.data_ptr(), ws.numel(), _stream()))
    return out


def e_div_u_sum(view, ufeat, efeat, u_target, n_out, edge_map=None):
    fmt, a, b, nmaj, nnz = _view(view)
    ufeat, ulen = _feat(ufeat)
    efeat, elen = _feat(efeat)
    shape = (n_out,) if efeat.dim() == 1 else (n_out, elen)
    out = torch.zeros(shape, dtype=torch.float32, device=efeat.device)
    ws = _spmm_workspace(fmt, nnz, n_out, out.device)
    check(lib().gs_e_div_u_sum(fmt, _ptr(a), _ptr(b), nmaj, nnz, _ptr(edge_map),
                               _fptr(ufeat), _fptr(efeat), _fptr(out), u_target, elen,
                               n_out, ws.data_ptr(), ws.numel(), _stream()))
    return out


def minor_slice(ids, picked, indptr=None, edge_major=None, with_major=True):
    """Keep edges whose id is in `picked`.
    -> (out_indptr | None, out_major | None, out_minor, out_select)"""
    ids, picked = _i64t(ids, "ids"), _i64t(picked, "picked")
    dev = ids.device
    nnz, npick = ids.numel(), picked.numel()
    nmaj = 0
    out_indptr = None
    if indptr is not None:
        indptr = _i64t(indptr, "indptr")
        nmaj = indptr.numel() - 1
        out_indptr = torch.empty(nmaj + 1, dtype=torch.int64, device=dev)
    if edge_major is not None:
        edge_major = _i64t(edge_major, "edge_major")
    l = lib()
    ws = _workspace(l.gs_minor_slice_workspace_bytes(nnz, npick), dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    check(l.gs_minor_slice_count(_ptr(ids), nnz, _ptr(picked), npick, _ptr(indptr), nmaj,
                                 _ptr(out_indptr), total.data_ptr(), ws.data_ptr(),
                                 ws.numel(), _stream()))
    kept = int(total.item())
    out_minor = torch.empty(kept, dtype=torch.int64, device=dev)
    out_select = torch.empty(kept, dtype=torch.int64, device=dev)
    want_major = with_major and (indptr is not None or edge_major is not None)
    out_major = torch.empty(kept, dtype=torch.int64, device=dev) if want_major else None
    check(l.gs_minor_slice_fill(_ptr(ids), nnz, npick, _ptr(indptr), nmaj, _ptr(edge_major),
                                _ptr(out_major), _ptr(out_minor), _ptr(out_select),
                                ws.data_ptr(), ws.numel(), _stream()))
    return out_indptr, out_major, out_minor, out_select


def col_row_slice(indptr, indices, cols, rows, key_offset=None, with_major=True,
                  indices32=None):
    """A[rows, cols] read from the parent matrix, the column slice never written.
    -> (out_indptr[len(cols) + 1], out_major | None = position of the edge's column in
    `cols`, out_minor = position of its row in `rows`, out_select = its position in the
    parent's `indices`).  `key_offset[len(cols)]` is added to the row ids of a column's
    edges before they are looked up among `rows`."""
    indptr, indices = _i64t(indptr, "indptr"), _i64t(indices, "indices")
    cols, rows = _i64t(cols, "cols"), _i64t(rows, "rows")
    if key_offset is not None:
        key_offset = _i64t(key_offset, "key_offset")
    dev = indptr.device
    ncol, nrow = cols.numel(), rows.numel()
    sub_indptr = col_count(indptr, cols, -1, False)
    nnz = int(sub_indptr[-1].item())
    l = lib()
    ws = _workspace(l.gs_minor_slice_workspace_bytes(nnz, nrow), dev)
    out_indptr = torch.empty(ncol + 1, dtype=torch.int64, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    check(l.gs_col_row_slice_count(_ptr(indptr), _ptr(indices),
                                   indices32.data_ptr() if indices32 is not None else None,
                                   _ptr(cols), _ptr(key_offset),
                                   ncol, sub_indptr.data_ptr(), nnz, _ptr(rows), nrow,
                                   out_indptr.data_ptr(), total.data_ptr(), ws.data_ptr(),
                                   ws.numel(), _stream()))
    kept = int(total.item())
    out_minor = torch.empty(kept, dtype=torch.int64, device=dev)
    out_select = torch.empty(kept, dtype=torch.int64, device=dev)
    out_major = torch.empty(kept, dtype=torch.int64, device=dev) if with_major else None
    check(l.gs_col_row_slice_fill(_ptr(indptr), _ptr(indices), _ptr(cols), ncol,
                                  sub_indptr.data_ptr(), nnz, nrow, _ptr(out_major),
                                  _ptr(out_minor), _ptr(out_select), ws.data_ptr(), ws.numel(),
                                  _stream()))
    return out_indptr, out_major, out_minor, out_select


def sliced_e_square_sum(indptr, indices, cols, efeat, num_out, use_workspace=True,
                        edge_map=None, indices32=None):
    """out[row] = sum of efeat^2 over the edges of A[:, cols], read from the parent
    (edge p's value is efeat[edge_map[p]] when an edge map is given)."""
    indptr, indices = _i64t(indptr, "indptr"), _i64t(indices, "indices")
    cols = _i64t(cols, "cols")
    efeat = efeat.contiguous()
    if efeat.dtype != torch.float32:
        raise GsError("efeat must be float32")
    dev = indptr.device
    sub_indptr = col_count(indptr, cols, -1, False)
    nnz = int(sub_indptr[-1].item())
    out = torch.zeros(num_out, dtype=torch.float32, device=dev)
    l = lib()
    ws = _workspace(l.gs_sliced_e_square_sum_workspace_bytes(nnz, num_out) if use_workspace
                    else 0, dev)
    check(l.gs_sliced_e_square_sum(_ptr(indptr), _ptr(indices),
                                   indices32.data_ptr() if indices32 is not None else None,
                                   _ptr(cols), cols.numel(),
                                   sub_indptr.data_ptr(), nnz, _ptr(edge_map), efeat.data_ptr(),
                                   out.data_ptr(), num_out, ws.data_ptr() if ws.numel() else None,
                                   ws.numel(), _stream()))
    return out


# ------------------------------------------------------------------ yardsticks
def probe_stream_copy(src, dst):
    """dst = src by the library's own copy kernel (a streaming yardstick)."""
    nbytes = src.numel() * src.element_size()
    check(lib().gs_probe_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, _stream()))


def probe_line_gather(table, num_picks, salt=0, ordered=False, out=None):
    """Every lane reads 4 bytes of a 128-byte line of its own of `table`."""
    if out is None:
        out = torch.empty(num_picks // 4 + 1, dtype=torch.int32, device=table.device)
    check(lib().gs_probe_line_gather(table.data_ptr(), table.numel() * table.element_size(),
                                     num_picks, salt, int(ordered), out.data_ptr(), _stream()))
    return out


def probe_sample_uniform(indptr, indices32, column_ids, fanout, variant, sub_indptr, outs,
                         probe_degree=0, seed=7777, call_id=0, col_span=None):
    """One launch of the packed uniform sampler with parts switched off (see
    gs_probe_sample_uniform); outs = (coo_col | None, rows, select) preallocated."""
    check(lib().gs_probe_sample_uniform(
        _ptr(indptr), indptr.numel() - 1, indices32.data_ptr(), _ptr(column_ids),
        column_ids.numel(), fanout, variant, probe_degree, seed, call_id, _ptr(sub_indptr),
        _ptr(col_span), _ptr(outs[0]), outs[1].data_ptr(), outs[2].data_ptr(), _stream()))


# --------------------------------------------------------- weighted sampling
def weighted_key_probe(seed, call_id, pos, draw, w, r64):
    """(-log2 of the unit draw r64, key of weight w) evaluated on the device."""
    out = torch.zeros(2, dtype=torch.float64, device="cuda")
    check(lib().gs_weighted_key_probe(seed, call_id, pos, draw, w, r64, out.data_ptr(),
                                      _stream()))
    return out.cpu().tolist()


def weight_cdf(indptr, probs, indices=None, num_rows=None):
    """Persistent packed CDF of the edge weights of a matrix (int64[nnz + 1]).
    With `indices` the row id of every edge is packed beside its share of the
    column's mass (ids below `num_rows`, default max id + 1), and the sampler
    never reads `indices`."""
    indptr = _i64t(indptr, "indptr")
    if indices is not None:
        indices = _i64t(indices, "indices")
        if num_rows is None:
            num_rows = int(indices.max().item()) + 1 if indices.numel() else 0
    probs = probs.contiguous()
    if probs.dtype != torch.float32:
        raise GsError("probs must be float32")
    nnz, num_cols = probs.numel(), indptr.numel() - 1
    cdf = torch.empty(nnz + 1, dtype=torch.int64, device=indptr.device)
    ws = _workspace(lib().gs_weight_cdf_workspace_bytes(num_cols, nnz), indptr.device)
    check(lib().gs_weight_cdf_build(_ptr(indptr), num_cols, _ptr(indices), num_rows or 0,
                                    probs.data_ptr(), nnz, cdf.data_ptr(), ws.data_ptr(),
                                    ws.numel(), _stream()))
    return cdf


def sample_weighted(indptr, indices, probs, column_ids, fanout, replace=False, seed=7777,
                    call_id=0, with_coo=True, cdf=None, col_batch_ptr=None):
    """Weighted per-column sampling -> (sub_indptr, coo_col | None, sub_indices, select).
    With `cdf` (from weight_cdf) draws are searches in the CDF instead of passes
    over the weights.  `col_batch_ptr`: as for sample_uniform."""
    indptr, indices = _i64t(indptr, "indptr"), _i64t(indices, "indices")
    if col_batch_ptr is not None:
        col_batch_ptr = _i64t(col_batch_ptr, "col_batch_ptr")
    if cdf is not None:
        return _sample_weighted_cdf(indptr, indices, _i64t(cdf, "cdf"), column_ids, fanout,
                                    replace, seed, call_id, with_coo, col_batch_ptr)
    probs = probs.contiguous()
    if probs.dtype != torch.float32:
        raise GsError("probs must be float32")
    num_cols = indptr.numel() - 1
    dev = indptr.device
    if column_ids is not None:
        column_ids = _i64t(column_ids, "column_ids")
        n = column_ids.numel()
    else:
        n = num_cols
    sub_indptr = col_count(indptr, column_ids, fanout, replace, n)
    nnz = int(sub_indptr[-1].item())
    out_idx = torch.empty(nnz, dtype=torch.int64, device=dev)
    out_sel = torch.empty(nnz, dtype=torch.int64, device=dev)
    out_col = torch.empty(nnz, dtype=torch.int64, device=dev) if with_coo else None
    cdf_off = scratch = None
    if replace:
        if column_ids is not None:
            cdf_off = col_count(indptr, column_ids, -1, False)
            scratch = torch.empty(int(cdf_off[-1].item()) + 1, dtype=torch.int64, device=dev)
        else:
            scratch = torch.empty(indices.numel() + 1, dtype=torch.int64, device=dev)
    if nnz > 0:
        check(lib().gs_csc_col_sample_weighted_fill(
            _ptr(indptr), num_cols, _ptr(indices), probs.data_ptr(), None, _ptr(column_ids),
            n, fanout, int(replace), seed, call_id, sub_indptr.data_ptr(), None, _ptr(cdf_off),
            _ptr(scratch), _ptr(out_col), out_idx.data_ptr(), out_sel.data_ptr(),
            _ptr(col_batch_ptr), col_batch_ptr.numel() - 1 if col_batch_ptr is not None else 0,
            _stream()))
    return sub_indptr, out_col, out_idx, out_sel


def _sample_weighted_cdf(indptr, indices, cdf, column_ids, fanout, replace, seed, call_id,
                         with_coo, col_batch_ptr=None, spans=True):
    num_cols = indptr.numel() - 1
    dev = indptr.device
    if column_ids is not None:
        column_ids = _i64t(column_ids, "column_ids")
        n = column_ids.numel()
    else:
        n = num_cols
    count = _Count()
    col_span = torch.empty(n, dtype=torch.int64, device=dev) if spans else None
    sub_indptr = col_count(indptr, column_ids, fanout, replace, n, count, col_span)
    bound = n * fanout
    size = bound if bound <= _BOUND_LIMIT else count.get()
    out_idx = torch.empty(size, dtype=torch.int64, device=dev)
    out_sel = torch.empty(size, dtype=torch.int64, device=dev)
    out_col = torch.empty(size, dtype=torch.int64, device=dev) if with_coo else None
    if size > 0:
        check(lib().gs_csc_col_sample_weighted_fill(
            _ptr(indptr), num_cols, _ptr(indices), None, cdf.data_ptr(), _ptr(column_ids), n,
            fanout, int(replace), seed, call_id, sub_indptr.data_ptr(), _ptr(col_span), None,
            None, _ptr(out_col), out_idx.data_ptr(), out_sel.data_ptr(), _ptr(col_batch_ptr),
            col_batch_ptr.numel() - 1 if col_batch_ptr is not None else 0, _stream()))
    nnz = count.get()
    return (sub_indptr, out_col[:nnz] if with_coo else None, out_idx[:nnz], out_sel[:nnz])


def list_sample_uniform(n, num_picks, replace=False, algo=ALGO_AUTO, seed=7777, call_id=0,
                        device="cuda"):
    count = (num_picks if n > 0 else 0) if replace else min(n, num_picks)
    out = torch.empty(count, dtype=torch.int64, device=device)
    check(lib().gs_list_sample_uniform(n, num_picks, int(replace), algo, seed, call_id,
                                       _ptr(out), _stream()))
    return out


def list_sample_weighted(probs, num_picks, replace=False, range_=None, seed=7777, call_id=0):
    """-> (index, out_range)"""
    probs = probs.contiguous()
    if probs.dtype != torch.float32 or not probs.is_cuda:
        raise GsError("probs must be a CUDA float32 tensor")
    dev = probs.device
    n = probs.numel()
    nseg = 1
    if range_ is not None:
        range_ = _i64t(range_, "range")
        nseg = range_.numel() - 1
    l = lib()
    ws = _workspace(l.gs_list_sample_workspace_bytes(n, nseg), dev)
    out_range = torch.empty(nseg + 1, dtype=torch.int64, device=dev)
    check(l.gs_list_sample_weighted_count(_ptr(range_), n, nseg, num_picks, int(replace),
                                          out_range.data_ptr(), ws.data_ptr(), ws.numel(),
                                          _stream()))
    total = int(out_range[-1].item())
    out = torch.empty(total, dtype=torch.int64, device=dev)
    check(l.gs_list_sample_weighted_fill(_fptr(probs), _ptr(range_), n, nseg, num_picks,
                                         int(replace), seed, call_id, out_range.data_ptr(),
                                         total, _ptr(out), ws.data_ptr(), ws.numel(),
                                         _stream()))
    return out, out_range


# --------------------------------------------------------------------- walks
def random_walk(indptr, indices, seeds, walk_length, seed=7777, call_id=0):
    """-> int64 [walk_length + 1, num_seeds] (step-major)."""
    indptr, indices, seeds = _i64t(indptr, "indptr"), _i64t(indices, "indices"), _i64t(seeds, "seeds")
    n = seeds.numel()
    out = torch.empty((walk_length + 1, n), dtype=torch.int64, device=indptr.device)
    check(lib().gs_random_walk(_ptr(indptr), _ptr(indices), indptr.numel() - 1, _ptr(seeds), n,
                               walk_length, seed, call_id, _ptr(out), _stream()))
    return out


def node2vec(indptr, indices, seeds, walk_length, p, q, seed=7777, call_id=0):
    indptr, indices, seeds = _i64t(indptr, "indptr"), _i64t(indices, "indices"), _i64t(seeds, "seeds")
    n = seeds.numel()
    out = torch.empty((walk_length + 1, n), dtype=torch.int64, device=indptr.device)
    check(lib().gs_node2vec(_ptr(indptr), _ptr(indices), indptr.numel() - 1, _ptr(seeds), n,
                            walk_length, p, q, seed, call_id, _ptr(out), _stream()))
    return out


def segment_sort(indptr, keys, key_bound=0):
    """Keys sorted inside every segment.  `key_bound` (every key in [0, key_bound),
    e.g. the number of rows) selects the much faster packed sort; 0 = not known."""
    indptr, keys = _i64t(indptr, "indptr"), _i64t(keys, "keys")
    out = torch.empty_like(keys)
    nseg = indptr.numel() - 1
    ws = _workspace(lib().gs_segment_sort_workspace_bytes(keys.numel(), nseg, key_bound),
                    keys.device)
    check(lib().gs_segment_sort_i64(_ptr(indptr), nseg, _ptr(keys), _ptr(out), keys.numel(),
                                    key_bound, ws.data_ptr(), ws.numel(), _stream()))
    return out
