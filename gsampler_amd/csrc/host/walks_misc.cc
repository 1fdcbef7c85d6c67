// walks_misc.cc -- walks, per-column index sort, compaction and the batched
// column+row slice of gs_classes.Graph.
#include "abi_call.h"
#include "graph.h"

namespace gs {

static uint64_t take_call_id() { return random_state().next_call++; }

// Traces are stored step-major ([walk_length + 1][num_seeds] in memory) and
// returned with shape [num_seeds, walk_length + 1] exactly as the reference
// does (src/cuda/fusion/random_walk.cu:34,67): callers obtain per-step rows
// with `.reshape(-1, num_seeds)`.
torch::Tensor Graph::RandomWalk(torch::Tensor seeds, int64_t walk_length) {
  TORCH_CHECK(csc_ != nullptr, "RandomWalk needs the CSC format");
  TORCH_CHECK(walk_length >= 0, "walk_length must be non-negative");
  seeds = ids(seeds, "seeds");
  const int64_t n = seeds.numel();
  torch::Tensor out = new_ids(n * (walk_length + 1), seeds);
  const RandomState& rs = random_state();
  GS_CALL(gs_random_walk(cptr(csc_->indptr), cptr(csc_->indices), num_cols_,
                         cptr(seeds), n, walk_length, rs.seed, take_call_id(),
                         mptr(out), cur_stream()));
  return out.reshape({n, -1});
}

torch::Tensor Graph::Node2Vec(torch::Tensor seeds, int64_t walk_length, double p,
                              double q) {
  TORCH_CHECK(csc_ != nullptr, "Node2Vec needs the CSC format");
  TORCH_CHECK(walk_length >= 0, "walk_length must be non-negative");
  TORCH_CHECK(p > 0 && q > 0, "Node2Vec: p and q must be positive");
  // The connectivity test bisects the previous node's column: row ids must be
  // sorted inside every column.  Looked at once per matrix (one pass over the
  // edges); the reference walks on unsorted columns without noticing.
  if (!csc_sorted_) {
    const torch::Tensor& idx = csc_->indices;
    const int64_t nnz = idx.numel();
    if (nnz > 1) {
      torch::Tensor drop = idx.slice(0, 1).lt(idx.slice(0, 0, nnz - 1));
      torch::Tensor ends = csc_->indptr.slice(0, 1, num_cols_) - 1;  // last edge of a column
      ends = ends.masked_select(ends.ge(0).logical_and(ends.lt(nnz - 1)));
      drop.index_fill_(0, ends.to(drop.device()), false);
      TORCH_CHECK(!drop.any().item<bool>(),
                  "Node2Vec needs row ids sorted inside every column: call SortCSCIndices first");
    }
    csc_sorted_ = true;
  }
  seeds = ids(seeds, "seeds");
  const int64_t n = seeds.numel();
  torch::Tensor out = new_ids(n * (walk_length + 1), seeds);
  const RandomState& rs = random_state();
  GS_CALL(gs_node2vec(cptr(csc_->indptr), cptr(csc_->indices), num_cols_,
                      cptr(seeds), n, walk_length, p, q, rs.seed, take_call_id(),
                      mptr(out), cur_stream()));
  return out.reshape({n, -1});
}

void Graph::SortCSCIndices() {
  TORCH_CHECK(csc_ != nullptr, "SortCSCIndices: the graph has no CSC format");
  TORCH_CHECK(!csc_->e_ids.has_value(), "SortCSCIndices: the CSC format carries e_ids");
  const int64_t nnz = csc_->indices.numel();
  torch::Tensor sorted = new_ids(nnz, csc_->indices);
  // row ids lie in [0, num_rows): the loaders check that
  torch::Tensor ws = new_workspace(gs_segment_sort_workspace_bytes(nnz, num_cols_, num_rows_),
                                   csc_->indices);
  GS_CALL(gs_segment_sort_i64(cptr(csc_->indptr), num_cols_, cptr(csc_->indices),
                              mptr(sorted), nnz, num_rows_, ws.data_ptr(), ws.numel(),
                              cur_stream()));
  csc_->indices = sorted;
  csc_->forget_derived();
  csc_sorted_ = true;
  coo_ = nullptr;  // derived formats followed the old edge order
  csr_ = nullptr;
}

// (sorted distinct ids, rank of every element among them): TensorCompact,
// src/cuda/compact.cu:11-34, which is torch's sorted unique with inverse.
static std::tuple<torch::Tensor, torch::Tensor> compact_ids(const torch::Tensor& x) {
  auto r = torch::_unique2(x, /*sorted=*/true, /*return_inverse=*/true,
                           /*return_counts=*/false);
  return {std::get<0>(r), std::get<1>(r)};
}

// Drops ids that no edge uses on `axis` (0 rows, 1 columns) and renumbers the
// rest densely; returns the kept original ids.  Formats whose compressed axis
// is the compacted one are dropped (they can be rebuilt from the COO).
GraphAndIndex Graph::Compact(int64_t axis) {
  TORCH_CHECK(axis == 0 || axis == 1, "Compact: axis must be 0 or 1");
  torch::Tensor kept, local;
  std::shared_ptr<Coordinate> coo;
  std::shared_ptr<Compressed> csc, csr;
  if (coo_) {
    const torch::Tensor& src = axis == 0 ? coo_->row : coo_->col;
    std::tie(kept, local) = compact_ids(src);
    coo = std::make_shared<Coordinate>(*coo_);
    (axis == 0 ? coo->row : coo->col) = local;
  }
  const std::shared_ptr<Compressed>& other = axis == 0 ? csc_ : csr_;
  if (other) {
    const torch::Tensor& coo_src = coo_ ? (axis == 0 ? coo_->row : coo_->col) : other->indices;
    torch::Tensor ids_local;
    if (coo_ && other->indices.is_same(coo_src)) {
      ids_local = local;
    } else {
      torch::Tensor k2;
      std::tie(k2, ids_local) = compact_ids(other->indices);
      if (!kept.defined()) kept = k2;
    }
    auto m = std::make_shared<Compressed>(*other);
    m->indices = ids_local;
    m->forget_derived();
    (axis == 0 ? csc : csr) = m;
  }
  TORCH_CHECK(kept.defined(), "Compact: the graph has no format with explicit ids on axis ",
              axis);
  auto g = c10::make_intrusive<Graph>(axis == 0 ? kept.numel() : num_rows_,
                                      axis == 0 ? num_cols_ : kept.numel());
  g->coo_ = coo;
  g->csc_ = csc;
  g->csr_ = csr;
  g->num_edges_ = num_edges_;
  return {g, kept};
}

}  // namespace gs
