// fused_slices.cc -- operators that read a column slice A[:, cols] straight
// from the matrix it is a slice of, without writing it first: the row sums of
// squared edge values over the slice, and the row slice of the slice
// (A[rows, cols]).  gs.jit.compile rewrites  A[:, cols] -> sum(e^2, axis=1) /
// -> [rows, :]  into these when nothing else reads the slice, which is the
// shape of a layer-wise sampler (examples/ladies/ladies.py:7-21 of the
// reference); the reference fuses the second pair only, and only for
// super-batches (src/cuda/fusion/column_row_slicing.cu).
#include "abi_call.h"
#include "graph.h"

namespace gs {

// Offsets and size of A[:, cols]: shared by the operators of this file when
// they are handed the same tensor of columns (one wait for the size, not two).
const Graph::SliceOffsets& Graph::slice_offsets_for(const torch::Tensor& cols) {
  const Compressed& m = compressed(kCSC);
  if (slice_offsets_ && slice_offsets_->cols.is_same(cols) &&
      slice_offsets_->version == (int64_t)cols._version() &&
      slice_offsets_->indptr_version == (int64_t)m.indptr._version() &&
      slice_offsets_->epoch == cache_epoch())
    return *slice_offsets_;
  auto so = std::make_unique<SliceOffsets>();
  const int64_t num_major = m.indptr.numel() - 1, n = cols.numel();
  so->cols = cols;
  so->version = cols._version();
  so->indptr_version = m.indptr._version();
  so->epoch = cache_epoch();
  so->sub_indptr = new_ids(n + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_scan_workspace_bytes(n + 1), m.indptr);
  AsyncCount count = AsyncCount::mirrored();
  GS_CALL(gs_csc_col_count(cptr(m.indptr), num_major, cptr(cols), n, -1, 0,
                           mptr(so->sub_indptr), count.mirror(), nullptr, ws.data_ptr(), ws.numel(),
                           cur_stream()));
  count.arm();
  so->nnz = count.get();
  slice_offsets_ = std::move(so);
  return *slice_offsets_;
}

// Reading a slice in place pays when its columns are long: the kernels look a
// run of a few thousand consecutive edges up in the column pointer once, and
// only runs inside one column (or across one border) are free of per-edge
// look-ups.  A slice of short columns is small: it is written once (and kept
// for the next operator on the same columns) and the plain operators run on it.
bool Graph::read_in_place(int64_t slice_nnz, int64_t num_cols_picked) {
  return slice_nnz >= (int64_t(1) << 20) && slice_nnz >= 4096 * num_cols_picked;
}

const MajorResult& Graph::written_slice(const torch::Tensor& cols) {
  slice_offsets_for(cols);
  SliceOffsets& so = *slice_offsets_;
  if (!so.written.indptr.defined()) so.written = major_slice(compressed(kCSC), cols, true, {}, 0);
  return so.written;
}

// out[row] += sum of efeat^2 over the edges of A[:, cols]; efeat is aligned with
// this matrix's edges (as edge data of the Python layer is).
void Graph::SlicedESquareSum(torch::Tensor cols, torch::Tensor efeat, torch::Tensor out) {
  cols = ids(cols, "cols");
  const Compressed& m = compressed(kCSC);
  TORCH_CHECK(efeat.defined() && out.defined(), "SlicedESquareSum: undefined operand");
  TORCH_CHECK(efeat.is_cuda() && out.is_cuda() && efeat.scalar_type() == torch::kFloat32 &&
                  out.scalar_type() == torch::kFloat32,
              "SlicedESquareSum needs float32 tensors on the GPU");
  efeat = efeat.contiguous();
  TORCH_CHECK(out.is_contiguous(), "SlicedESquareSum: out must be contiguous");
  TORCH_CHECK(efeat.numel() == m.indices.numel(), "SlicedESquareSum: ", efeat.numel(),
              " edge values for ", m.indices.numel(), " edges (scalar edge values only)");
  TORCH_CHECK(out.numel() == num_rows_, "SlicedESquareSum: out has ", out.numel(),
              " entries for ", num_rows_, " rows");
  const SliceOffsets& so = slice_offsets_for(cols);
  if (so.nnz == 0) return;
  if (!read_in_place(so.nnz, cols.numel())) {
    const MajorResult& r = written_slice(cols);
    torch::Tensor w = efeat.index_select(0, edge_index(m.e_ids, r.select));
    torch::Tensor ws =
        new_workspace(gs_spmm_workspace_bytes(GS_FMT_COO, so.nnz, num_rows_), m.indptr);
    GS_CALL(gs_e_square_sum(GS_FMT_COO, cptr(r.minor_ids), cptr(r.major_ids), 0, so.nnz, nullptr,
                            w.data_ptr<float>(), out.data_ptr<float>(), 2, 1, num_rows_,
                            ws.data_ptr(), (size_t)ws.numel(), cur_stream()));
    return;
  }
  torch::Tensor ws = new_workspace(gs_sliced_e_square_sum_workspace_bytes(so.nnz, num_rows_),
                                   m.indptr);
  const torch::Tensor e_ids = m.e_ids.has_value() ? m.e_ids.value() : torch::Tensor();
  const torch::Tensor& narrow = m.narrow_indices();  // half the bytes behind every id
  GS_CALL(gs_sliced_e_square_sum(cptr(m.indptr), cptr(m.indices),
                                 narrow.defined() ? narrow.data_ptr<int32_t>() : nullptr,
                                 cptr(cols), cols.numel(),
                                 cptr(so.sub_indptr), so.nnz, cptr(e_ids),
                                 efeat.data_ptr<float>(), out.data_ptr<float>(), num_rows_,
                                 ws.data_ptr(), (size_t)ws.numel(), cur_stream()));
}

// Shared by the plain and the super-batched form.  key_offset (per picked
// column) and `picked` carry the batch in their values when there are batches.
static MajorResult col_row_slice(const Compressed& m, const torch::Tensor& cols,
                                 const torch::Tensor& sub_indptr, int64_t nnz,
                                 const torch::Tensor& key_offset, const torch::Tensor& picked,
                                 bool with_coo) {
  const int64_t n = cols.numel(), np = picked.numel();
  MajorResult r;
  torch::Tensor ws = new_workspace(gs_minor_slice_workspace_bytes(nnz, np), m.indptr);
  r.indptr = new_ids(n + 1, m.indptr);
  // the number of kept edges goes straight to pinned host memory; the fill pass
  // is queued into buffers sized by the bound (every edge kept) and runs while
  // the number travels
  AsyncCount kept = AsyncCount::mirrored();
  const torch::Tensor& narrow = m.narrow_indices();  // half the bytes behind every id
  GS_CALL(gs_col_row_slice_count(cptr(m.indptr), cptr(m.indices),
                                 narrow.defined() ? narrow.data_ptr<int32_t>() : nullptr,
                                 cptr(cols), cptr(key_offset),
                                 n, cptr(sub_indptr), nnz, cptr(picked), np, mptr(r.indptr),
                                 kept.mirror(), ws.data_ptr(), ws.numel(), cur_stream()));
  kept.arm();
  const int64_t size = nnz <= kBoundLimit ? nnz : kept.get();
  r.minor_ids = new_ids(size, m.indptr);
  r.select = new_ids(size, m.indptr);
  if (with_coo) r.major_ids = new_ids(size, m.indptr);
  GS_CALL(gs_col_row_slice_fill(cptr(m.indptr), cptr(m.indices), cptr(cols), n,
                                cptr(sub_indptr), nnz, np,
                                with_coo ? mptr(r.major_ids) : nullptr, mptr(r.minor_ids),
                                mptr(r.select), ws.data_ptr(), ws.numel(), cur_stream()));
  const int64_t k = kept.get();
  r.minor_ids = trim_to(r.minor_ids, k);
  r.select = trim_to(r.select, k);
  if (with_coo) r.major_ids = trim_to(r.major_ids, k);
  return r;
}

// A[rows, cols]: rows become positions in `rows`, columns positions in `cols`;
// the edge index addresses this matrix's edges.
GraphAndIndex Graph::ColRowSlicing(torch::Tensor cols, torch::Tensor rows, int64_t on_format,
                                   int64_t output_format) {
  TORCH_CHECK(on_format == kCSC, "ColRowSlicing runs on the CSC format, got ", on_format);
  TORCH_CHECK(output_format != 0 && (output_format & kCSR) == 0,
              "ColRowSlicing produces CSC and COO, got output_format ", output_format);
  cols = ids(cols, "cols");
  rows = ids(rows, "rows");
  const Compressed& m = compressed(kCSC);
  const SliceOffsets& so = slice_offsets_for(cols);
  MajorResult r;
  if (read_in_place(so.nnz, cols.numel())) {
    r = col_row_slice(m, cols, so.sub_indptr, so.nnz, torch::Tensor(), rows,
                      output_format & kCOO);
  } else {
    const MajorResult& sliced = written_slice(cols);
    Compressed tmp{sliced.indptr, sliced.minor_ids, c10::nullopt};
    r = minor_slice(tmp, rows, output_format & kCOO);
    r.select = sliced.select.index_select(0, r.select);
  }
  GraphPtr g = derive(kCSC, output_format, r, rows.numel(), cols.numel());
  return {g, edge_index(m.e_ids, r.select)};
}

// Per batch b: the columns col[col_bptr[b] : col_bptr[b+1]] restricted to the
// rows row[row_bptr[b] : row_bptr[b+1]]; row ids become positions in `row`.
// The returned edge index addresses the parent's edges.  One pass over the
// parent's columns (BatchCSCColRowSlicingCUDA,
// src/cuda/fusion/column_row_slicing.cu:356-362): a batch's rows and the row
// ids of its columns' edges are both moved by batch * num_rows, so one table of
// picked rows serves all batches.
GraphAndIndex Graph::BatchColRowSlcing(torch::Tensor col, torch::Tensor col_bptr,
                                       torch::Tensor row, torch::Tensor row_bptr) {
  col = ids(col, "col");
  row = ids(row, "row");
  col_bptr = ids(col_bptr, "col_bptr");
  row_bptr = ids(row_bptr, "row_bptr");
  TORCH_CHECK(col_bptr.numel() == row_bptr.numel() && col_bptr.numel() >= 2,
              "BatchColRowSlcing: column and row batch pointers must have the same length");
  BatchOffsets::check(col_bptr, col.numel(), "BatchColRowSlicing");
  BatchOffsets::check(row_bptr, row.numel(), "BatchColRowSlicing");
  const Compressed& m = compressed(kCSC);
  const int64_t stride = num_rows_;
  auto batch_of = [&](const torch::Tensor& bptr, int64_t n) {
    torch::Tensor b = new_ids(n, m.indptr);
    GS_CALL(gs_csc2coo(cptr(bptr), bptr.numel() - 1, n, mptr(b), cur_stream()));
    return b;
  };
  torch::Tensor key_offset = batch_of(col_bptr, col.numel()) * stride;
  torch::Tensor picked = row + batch_of(row_bptr, row.numel()) * stride;
  const SliceOffsets& so = slice_offsets_for(col);
  MajorResult kept;
  if (read_in_place(so.nnz, col.numel())) {
    kept = col_row_slice(m, col, so.sub_indptr, so.nnz, key_offset, picked, false);
  } else {
    // short columns: the batched column slice with rows moved by batch * num_rows
    // is written and row-sliced
    MajorResult sliced = major_slice(m, col, false, col_bptr, stride);
    Compressed tmp{sliced.indptr, sliced.minor_ids, c10::nullopt};
    kept = minor_slice(tmp, picked, false);
    kept.select = sliced.select.index_select(0, kept.select);
  }
  auto g = c10::make_intrusive<Graph>(row.numel(), col.numel());
  auto csc = std::make_shared<Compressed>();
  csc->indptr = kept.indptr;
  csc->indices = kept.minor_ids;
  g->csc_ = csc;
  g->num_edges_ = kept.select.numel();
  g->col_bptr_ = col_bptr;
  g->row_bptr_ = row_bptr;
  g->orig_col_ids_ = col;
  g->orig_row_ids_ = row;
  g->edge_bptr_ = kept.indptr.index_select(0, col_bptr);
  BatchOffsets::trust(g->edge_bptr_);
  return {g, edge_index(m.e_ids, kept.select)};
}

}  // namespace gs
