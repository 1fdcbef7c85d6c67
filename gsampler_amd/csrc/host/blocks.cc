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
  f_off_ = OffsetMirror::values(frontier_ptr);
  e_off_ = OffsetMirror::values(coo_ptr);
  c_off_ = OffsetMirror::values(col_bptr);
  // Destination ids are labels in the frontier's numbering.  While the seeds of
  // a mini-batch are distinct the label of a seed is its position, and the
  // block's edges are grouped by destination in the order of the offsets; a
  // repeated seed shares the label of its first occurrence, and the offsets by
  // position no longer describe the block.  A batch's seeds are distinct exactly
  // when its last seed sits at the place ns - 1 of the batch's frontier: one
  // small gather per layer, on first use.
  grouped_.assign((size_t)num_batches, 1);
  if (num_batches > 0 && col_seeds.numel() > 0) {
    torch::Tensor ns = col_bptr.narrow(0, 1, num_batches) - col_bptr.narrow(0, 0, num_batches);
    torch::Tensor nu =
        frontier_ptr.narrow(0, 1, num_batches) - frontier_ptr.narrow(0, 0, num_batches);
    torch::Tensor has = (ns > 0) & (nu >= ns);
    torch::Tensor at_f = (frontier_ptr.narrow(0, 0, num_batches) + ns - 1)
                             .clamp(0, std::max<int64_t>(frontier.numel() - 1, 0));
    torch::Tensor at_s =
        (col_bptr.narrow(0, 1, num_batches) - 1).clamp(0, col_seeds.numel() - 1);
    torch::Tensor ok = (ns == 0);
    if (frontier.numel() > 0)
      ok = ok | (has & (frontier.index_select(0, at_f) == col_seeds.index_select(0, at_s)));
    torch::Tensor host = ok.to(torch::kCPU).to(torch::kUInt8).contiguous();
    for (int64_t b = 0; b < num_batches; ++b)
      grouped_[(size_t)b] = host.data_ptr<uint8_t>()[b];
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

std::vector<BlockViews> BlockBatch::Blocks() {
  std::vector<BlockViews> out;
  out.reserve((size_t)num_batches);
  for (int64_t b = 0; b < num_batches; ++b) out.push_back(Block(b));
  return out;
}

c10::intrusive_ptr<BlockBatch> Graph::BatchBlocks(torch::Tensor col_seeds,
                                                  torch::Tensor row_ids) {
  auto rel = BatchGraphRelabel(col_seeds, row_ids);  // queues count, fill and relabel
  auto out = c10::make_intrusive<BlockBatch>();
  out->frontier = std::get<0>(rel);
  out->frontier_ptr = std::get<1>(rel);
  out->row = std::get<2>(rel);
  out->col = std::get<3>(rel);
  out->e_ids = std::get<4>(rel);
  out->coo_ptr = std::get<5>(rel);
  out->col_bptr = col_bptr_;
  out->col_seeds = ids(col_seeds, "col_seeds");
  out->num_batches = col_bptr_.numel() - 1;
  out->num_dst_total = col_seeds.numel();
  // Offsets by destination of every block: the columns of the sampled matrix
  // are the destinations, so its indptr, cut at the batch boundaries and
  // rebased, is the blocks' indptr (the relabelled edges keep their order).
  torch::Tensor indptr;
  if (csc_) {
    indptr = csc_->indptr;
  } else {
    indptr = new_ids(num_cols_ + 1, coo_->col);  // the edge list is column-sorted
    GS_CALL(gs_sorted_to_indptr(cptr(coo_->col), coo_->col.numel(), num_cols_, mptr(indptr),
                                cur_stream()));
  }
  const int64_t total = num_cols_ + out->num_batches;
  out->indptr = new_ids(total, indptr);
  GS_CALL(gs_split_indptr(cptr(indptr), cptr(col_bptr_), out->num_batches, total,
                          mptr(out->indptr), cur_stream()));
  OffsetMirror::prefetch(col_bptr_);
  OffsetMirror::prefetch(out->coo_ptr);
  return out;
}

}  // namespace gs
