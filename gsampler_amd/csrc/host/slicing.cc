// slicing.cc -- slicing across the compressed axis (A[rows, :] on a CSC,
// A[:, cols] on a CSR) and coordinate-form slicing.
#include "abi_call.h"
#include "graph.h"

namespace gs {

// The first n entries of a buffer that was sized by an upper bound.  A view
// keeps the whole buffer alive for as long as the result lives: when the result
// is a small part of a large buffer (a row slice that keeps one edge in a hundred
// of a 60 M-edge matrix would pin three 480 MB buffers) it is copied out instead.
torch::Tensor trim_to(const torch::Tensor& buffer, int64_t n) {
  constexpr int64_t kLarge = int64_t(1) << 22;  // elements
  torch::Tensor head = buffer.narrow(0, 0, n);
  if (buffer.numel() > kLarge && n * 8 < buffer.numel()) return head.clone();
  return head;
}

namespace {
struct MinorKept {
  torch::Tensor indptr, major, minor, select;
};

// ids: the per-edge ids that are tested against `picked`.
MinorKept keep_members(const torch::Tensor& ids_per_edge, const torch::Tensor& picked,
                       const torch::Tensor& indptr, const torch::Tensor& edge_major,
                       bool want_major) {
  const int64_t nnz = ids_per_edge.numel(), np = picked.numel();
  const int64_t num_major = indptr.defined() ? indptr.numel() - 1 : 0;
  MinorKept r;
  torch::Tensor ws = new_workspace(gs_minor_slice_workspace_bytes(nnz, np), ids_per_edge);
  if (indptr.defined()) r.indptr = new_ids(num_major + 1, ids_per_edge);
  // the number of kept edges goes straight to pinned host memory; the fill pass
  // is queued into buffers sized by the bound (every edge kept) and runs while
  // the number travels
  AsyncCount kept = AsyncCount::mirrored();
  GS_CALL(gs_minor_slice_count(cptr(ids_per_edge), nnz, cptr(picked), np,
                               cptr(indptr), num_major,
                               indptr.defined() ? mptr(r.indptr) : nullptr,
                               kept.mirror(), ws.data_ptr(), ws.numel(),
                               cur_stream()));
  kept.arm();
  const int64_t size = nnz <= kBoundLimit ? nnz : kept.get();
  r.minor = new_ids(size, ids_per_edge);
  r.select = new_ids(size, ids_per_edge);
  if (want_major) r.major = new_ids(size, ids_per_edge);
  GS_CALL(gs_minor_slice_fill(cptr(ids_per_edge), nnz, np, cptr(indptr), num_major,
                              cptr(edge_major), want_major ? mptr(r.major) : nullptr,
                              mptr(r.minor), mptr(r.select), ws.data_ptr(),
                              ws.numel(), cur_stream()));
  const int64_t n = kept.get();
  r.minor = trim_to(r.minor, n);
  r.select = trim_to(r.select, n);
  if (want_major) r.major = trim_to(r.major, n);
  return r;
}
}  // namespace

MajorResult minor_slice(const Compressed& m, const torch::Tensor& picked,
                        bool with_coo) {
  MinorKept k = keep_members(m.indices, picked, m.indptr, {}, with_coo);
  return MajorResult{k.indptr, k.major, k.minor, k.select};
}

// axis 0 filters on rows, axis 1 on columns; the filtered axis is relabelled to
// positions in `seeds`, the other one is carried through.
GraphAndIndex Graph::slice_coo(const torch::Tensor& seeds, int64_t axis,
                               int64_t new_rows, int64_t new_cols) {
  CreateSparseFormat(kCOO);
  const torch::Tensor& tested = axis == 0 ? coo_->row : coo_->col;
  const torch::Tensor& other = axis == 0 ? coo_->col : coo_->row;
  MinorKept k = keep_members(tested, seeds, {}, other, true);
  auto g = c10::make_intrusive<Graph>(new_rows, new_cols);
  auto coo = std::make_shared<Coordinate>();
  coo->row = axis == 0 ? k.minor : k.major;
  coo->col = axis == 0 ? k.major : k.minor;
  // the carried-through axis keeps its order; the relabelled one does not
  coo->row_sorted = axis == 1 && coo_->row_sorted;
  coo->col_sorted = axis == 0 && coo_->col_sorted;
  g->coo_ = coo;
  g->num_edges_ = k.select.numel();
  return {g, edge_index(coo_->e_ids, k.select)};
}

}  // namespace gs
