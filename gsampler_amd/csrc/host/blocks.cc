// blocks.cc -- the hand-off of a super-batched sampler: all mini-batch blocks
// of one layer from a single operator call.
//
// The reference relabels the super-batch, splits the relabelled edge list and
// the frontier per mini-batch and builds one DGL block per mini-batch in a
// Python loop (python/gs/matrix_api/batch_matrix.py:13-36,232-248), from the
// edge list only, so that DGL derives the compressed formats later
// (python/gs/utils/to_dgl_block.py:19-23).  Here one call does the relabel and
// the per-block offsets arrays on the device and returns a BlockBatch: every
// block's edge list (row -> col, batch-local ids), its compressed form by
// destination (indptr over the block's destination nodes, indices = row) and
// its source ids are views into the layer's concatenated arrays.
#include "abi_call.h"
#include "graph.h"

namespace gs {

int64_t BlockBatch::NumSrcOf(int64_t b) {
  fetch();
  return f_off_[(size_t)b + 1] - f_off_[(size_t)b];
}

void BlockBatch::fetch() {
  if (have_host_) return;
  // Offsets by destination of every block: the columns of the sampled matrix
  // are the destinations, so its indptr, cut at the batch boundaries and
  // rebased, is the blocks' indptr (the relabelled edges keep their order).
  // Two small launches, made when the first block is asked for rather than in
  // the sampler's launch sequence.
  const int64_t total = sampled_indptr.numel() - 1 + num_batches;
  indptr = new_ids(total, sampled_indptr);
  GS_CALL(gs_split_indptr(cptr(sampled_indptr), cptr(col_bptr), num_batches, total, mptr(indptr),
                          cur_stream()));
  distinct = new_ids(num_batches, sampled_indptr);
  GS_CALL(gs_batch_seeds_distinct(cptr(frontier), cptr(frontier_ptr), cptr(col_seeds),
                                  cptr(col_bptr), num_batches, mptr(distinct), cur_stream()));
  f_off_ = OffsetMirror::values(frontier_ptr);
  e_off_ = OffsetMirror::values(coo_ptr);
  c_off_ = OffsetMirror::values(col_bptr);
  // Destination ids are labels in the frontier's numbering.  While the seeds of
  // a mini-batch are distinct the label of a seed is its position, and the
  // block's edges are grouped by destination in the order of the offsets; a
  // repeated seed shares the label of its first occurrence, and the offsets by
  // position no longer describe the block.
  grouped_.assign((size_t)num_batches, 1);
  if (distinct.defined()) {
    const std::vector<int64_t>& d = OffsetMirror::values(distinct);
    for (int64_t b = 0; b < num_batches; ++b) grouped_[(size_t)b] = d[(size_t)b] != 0;
  }
  have_host_ = true;
}

std::vector<int64_t> BlockBatch::Totals() {
  return {frontier.numel(), num_dst_total, row.numel()};
}

std::tuple<std::vector<int64_t>, std::vector<int64_t>, std::vector<int64_t>>
BlockBatch::Offsets() {
  fetch();
  return {f_off_, c_off_, e_off_};
}

BlockViews BlockBatch::Block(int64_t b) {
  TORCH_CHECK(b >= 0 && b < num_batches, "BlockBatch: no mini-batch ", b, " (there are ",
              num_batches, ")");
  fetch();
  const size_t i = (size_t)b;
  const int64_t e0 = e_off_[i], ne = e_off_[i + 1] - e0;
  const int64_t c0 = c_off_[i], nc = c_off_[i + 1] - c0;
  const int64_t f0 = f_off_[i], nf = f_off_[i + 1] - f0;
  c10::optional<torch::Tensor> eids, offsets;
  if (e_ids.has_value()) eids = e_ids.value().narrow(0, e0, ne);
  // block b's offsets sit at [c0 + b, c0 + b + nc] of the split array
  if (grouped_[i]) offsets = indptr.narrow(0, c0 + b, nc + 1);
  return {row.narrow(0, e0, ne), col.narrow(0, e0, ne), offsets, frontier.narrow(0, f0, nf), eids,
          nf, nc};
}

// All blocks at once, one list per field (the per-batch splits are made by
// torch's split, which is far cheaper than a view at a time).
BlockParts BlockBatch::Blocks() {
  fetch();
  auto sizes = [](const std::vector<int64_t>& off) {
    std::vector<int64_t> s(off.size() - 1);
    for (size_t i = 0; i + 1 < off.size(); ++i) s[i] = off[i + 1] - off[i];
    return s;
  };
  const std::vector<int64_t> ne = sizes(e_off_), nf = sizes(f_off_), nc = sizes(c_off_);
  std::vector<torch::Tensor> rows = torch::split_with_sizes(row, ne);
  std::vector<torch::Tensor> cols = torch::split_with_sizes(col, ne);
  std::vector<torch::Tensor> fronts = torch::split_with_sizes(frontier, nf);
  std::vector<c10::optional<torch::Tensor>> eids((size_t)num_batches), offs((size_t)num_batches);
  if (e_ids.has_value()) {
    std::vector<torch::Tensor> parts = torch::split_with_sizes(e_ids.value(), ne);
    for (size_t i = 0; i < parts.size(); ++i) eids[i] = parts[i];
  }
  std::vector<int64_t> with_end(nc);
  for (int64_t& n : with_end) n += 1;  // a block's offsets have one entry more than it has columns
  std::vector<torch::Tensor> pieces = torch::split_with_sizes(indptr, with_end);
  for (size_t i = 0; i < pieces.size(); ++i)
    if (grouped_[i]) offs[i] = pieces[i];
  return {rows, cols, offs, fronts, eids, nf, nc};
}

// Everything is queued before the host waits for the size of the frontier (the
// last statement): the device works through the relabel while that number
// travels, and the caller's next launches follow at once.
c10::intrusive_ptr<BlockBatch> Graph::BatchBlocks(torch::Tensor col_seeds,
                                                  torch::Tensor row_ids) {
  TORCH_CHECK(col_bptr_.defined() && col_bptr_.numel() >= 2,
              "BatchBlocks: the graph has no column batch pointer");
  auto out = c10::make_intrusive<BlockBatch>();
  out->num_batches = col_bptr_.numel() - 1;
  if (csc_) {
    out->sampled_indptr = csc_->indptr;
  } else {
    CreateSparseFormat(kCOO);
    TORCH_CHECK(coo_->col_sorted, "BatchBlocks: the COO format must be column-sorted");
    out->sampled_indptr = new_ids(num_cols_ + 1, coo_->col);
    GS_CALL(gs_sorted_to_indptr(cptr(coo_->col), coo_->col.numel(), num_cols_,
                                mptr(out->sampled_indptr), cur_stream()));
  }
  Frontier& f = batch_relabel_launch(col_seeds, row_ids, &out->row, &out->col, &out->e_ids);
  out->col_seeds = col_seeds;
  out->num_dst_total = col_seeds.numel();
  out->frontier_ptr = f.unique_ptr;
  out->coo_ptr = edge_bptr_;
  out->col_bptr = col_bptr_;
  // (the pointer arrays are on their way to the host or there already: the
  // sampler sent the edge pointer, the unique pass the frontier pointer, and the
  // column pointer is the caller's or the previous layer's frontier pointer)
  out->frontier = f.frontier();  // waits for the number of unique ids
  return out;
}

}  // namespace gs
