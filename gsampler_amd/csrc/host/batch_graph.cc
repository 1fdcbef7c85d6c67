// batch_graph.cc -- super-batch operators: B independent mini-batches share one
// launch; per-batch boundaries travel as int64[B + 1] pointer arrays
// (col_bptr over the seed columns, edge_bptr over the edges, row_bptr over
// compacted rows).  Mirrors the interface of src/batch_graph.cc of gSampler.
#include "abi_call.h"
#include "graph.h"

namespace gs {

void Graph::copy_batch_state_to(Graph& g, bool with_rows) {
  g.col_bptr_ = col_bptr_;
  g.orig_col_ids_ = orig_col_ids_;
  if (with_rows) {
    g.row_bptr_ = row_bptr_;
    g.orig_row_ids_ = orig_row_ids_;
  }
  g.row_encoding_size_ = row_encoding_size_;
  if (g.csc_ && col_bptr_.defined()) {
    g.edge_bptr_ = g.csc_->indptr.index_select(0, col_bptr_);
    BatchOffsets::trust(g.edge_bptr_);
  }
}

std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCSCIndptr() {
  CreateSparseFormat(kCSC);
  return {csc_->indptr, col_bptr_};
}
std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCSCIndices() {
  CreateSparseFormat(kCSC);
  return {csc_->indices, edge_bptr_};
}
std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCSCEids() {
  CreateSparseFormat(kCSC);
  if (csc_->e_ids.has_value()) return {csc_->e_ids.value(), edge_bptr_};
  return {torch::Tensor(), torch::Tensor()};
}
std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCOORows() {
  CreateSparseFormat(kCOO);
  return {coo_->row, edge_bptr_};
}
std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCOOCols() {
  CreateSparseFormat(kCOO);
  return {coo_->col, edge_bptr_};
}
std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetCOOEids() {
  CreateSparseFormat(kCOO);
  if (coo_->e_ids.has_value()) return {coo_->e_ids.value(), edge_bptr_};
  return {torch::Tensor(), torch::Tensor()};
}

static const std::vector<int64_t>& host_offsets(const torch::Tensor& offset) {
  if (offset.scalar_type() != torch::kInt64)
    return OffsetMirror::values(offset.to(torch::kInt64));
  return OffsetMirror::values(offset);
}

std::vector<int64_t> Graph::BatchGetColCounts() {
  TORCH_CHECK(col_bptr_.defined() && col_bptr_.numel() > 0,
              "BatchGetColCounts: no column batch pointer set");
  const std::vector<int64_t>& p = host_offsets(col_bptr_);
  std::vector<int64_t> counts(p.size() - 1);
  for (size_t i = 0; i < counts.size(); ++i) counts[i] = p[i + 1] - p[i];
  return counts;
}

// Decodes ids of the form id + batch * stride (row encoding of batched
// slicing): returns (per-batch offsets into the sorted encoded array, original
// ids).  Counterpart of GetBatchOffsets, src/cuda/batch/encoding_decoding.cu:99.
static std::tuple<torch::Tensor, torch::Tensor> batch_offsets(
    const torch::Tensor& encoded, int64_t num_batches, int64_t stride) {
  const int64_t n = encoded.numel();
  torch::Tensor batch = new_ids(n, encoded), orig = new_ids(n, encoded);
  GS_CALL(gs_decode_batch_ids(cptr(encoded), n, stride, mptr(orig), mptr(batch),
                              cur_stream()));
  torch::Tensor ptr = new_ids(num_batches + 1, encoded);
  GS_CALL(gs_sorted_to_indptr(cptr(batch), n, num_batches, mptr(ptr),
                              cur_stream()));
  return {ptr, orig};
}

GraphAndIndex Graph::BatchColSlicing(torch::Tensor seeds, torch::Tensor col_bptr,
                                     bool encoding) {
  seeds = ids(seeds, "seeds");
  col_bptr = ids(col_bptr, "col_bptr");
  const int64_t B = col_bptr.numel() - 1;
  TORCH_CHECK(B >= 1, "BatchColSlicing: col_bptr needs at least two entries");
  BatchOffsets::check(col_bptr, seeds.numel(), "BatchColSlicing");
  const Compressed& m = compressed(kCSC);
  const int64_t stride = num_rows_;
  MajorResult r = major_slice(m, seeds, true, col_bptr, encoding ? stride : 0);
  torch::Tensor row_bptr, orig_rows;
  if (encoding) {
    // compact the encoded row ids: sorted unique + rank of every edge's row
    auto uniq = torch::_unique2(r.minor_ids, /*sorted=*/true,
                                /*return_inverse=*/true, /*return_counts=*/false);
    r.minor_ids = std::get<1>(uniq);
    std::tie(row_bptr, orig_rows) = batch_offsets(std::get<0>(uniq), B, stride);
    BatchOffsets::trust(row_bptr);
  }
  const int64_t new_rows = encoding ? orig_rows.numel() : num_rows_ * B;
  GraphPtr g = derive(kCSC, kCSC | kCOO, r, new_rows, seeds.numel());
  g->col_bptr_ = col_bptr;
  g->orig_col_ids_ = seeds;
  g->edge_bptr_ = r.indptr.index_select(0, col_bptr);
  BatchOffsets::trust(g->edge_bptr_);
  if (encoding) {
    g->row_bptr_ = row_bptr;
    g->orig_row_ids_ = orig_rows;
    g->row_encoding_size_ = stride;
  }
  return {g, edge_index(m.e_ids, r.select)};
}

GraphAndIndex Graph::BatchRowSlicing(torch::Tensor row_ids,
                                     torch::Tensor row_bptr) {
  BatchOffsets::check(ids(row_bptr, "row_bptr"), row_ids.numel(), "BatchRowSlicing");
  auto ret = Slicing(row_ids, 0, kCSC, kCSC | kCOO);
  Graph& g = *std::get<0>(ret);
  copy_batch_state_to(g, false);
  g.row_bptr_ = row_bptr;
  g.orig_row_ids_ = row_ids;
  return ret;
}

GraphAndIndex Graph::BatchRowSampling(int64_t fanout, bool replace) {
  auto ret = Sampling(1, fanout, replace, kCSC, kCSC | kCOO);
  copy_batch_state_to(*std::get<0>(ret), true);
  return ret;
}

GraphAndIndex Graph::BatchRowSamplingProbs(int64_t fanout, bool replace,
                                           torch::Tensor edge_probs) {
  auto ret = SamplingProbs(1, edge_probs, fanout, replace, kCSC, kCSC | kCOO);
  copy_batch_state_to(*std::get<0>(ret), true);
  return ret;
}

// One launch samples the columns of every batch: a column's picks depend on
// its position in the concatenated seed array, never on the batch split.
GraphAndIndex Graph::BatchFusedSlicingSampling(torch::Tensor seeds,
                                               torch::Tensor col_bptr,
                                               int64_t fanout, bool replace) {
  col_bptr = ids(col_bptr, "col_bptr");
  BatchOffsets::check(col_bptr, seeds.numel(), "BatchFusedSlicingSampling");
  EdgeCount::HintScope batch(col_bptr);  // the sampler leaves the edge pointer here
  // compressed by column only: the relabel pass reads the column pointer, and
  // the coordinate form is expanded from it if somebody asks
  auto ret = FusedSlicingSampling(1, seeds, fanout, replace, kCSC, kCSC);
  Graph& g = *std::get<0>(ret);
  g.col_labels_ = EdgeCount::hint().col_labels;
  g.col_bptr_ = col_bptr;
  g.orig_col_ids_ = ids(seeds, "seeds");
  g.edge_bptr_ = EdgeCount::hint().edge_bptr;
  if (!g.edge_bptr_.defined()) g.edge_bptr_ = g.csc_->indptr.index_select(0, col_bptr);
  BatchOffsets::trust(g.edge_bptr_, g.num_edges_);
  return ret;
}

// A compressed-by-column matrix whose coordinate form nobody has asked for
// hands over its column pointer; the coordinate form is then not built at all.
Graph::ColumnOrderedEdges Graph::column_ordered_edges(const char* who) {
  if (csc_ && !coo_) return {csc_->indices, {}, csc_->indptr, csc_->e_ids};
  CreateSparseFormat(kCOO);
  TORCH_CHECK(coo_->col_sorted, who, ": the COO format must be column-sorted");
  return {coo_->row, coo_->col, {}, coo_->e_ids};
}

// Global row ids of every edge as the relabel pass needs them: rows of an
// encoded (compacted) batch graph are decoded back through row_ids.
torch::Tensor Graph::batch_rows_for_relabel(const torch::Tensor& edge_rows,
                                            const torch::Tensor& row_ids) {
  if (row_ids.numel() == 0) return edge_rows;
  if (!(mapped_out_.defined() && mapped_from_.is_same(edge_rows) &&
        mapped_by_.is_same(row_ids))) {
    torch::Tensor enc = ids(row_ids, "row_ids").index_select(0, edge_rows);
    const int64_t B = edge_bptr_.numel() - 1;
    torch::Tensor orig = enc;
    if (row_encoding_size_ > 0)
      orig = std::get<1>(batch_offsets(enc, B, row_encoding_size_));
    mapped_out_ = orig;
    mapped_from_ = edge_rows;
    mapped_by_ = row_ids;
  }
  return mapped_out_;
}

// Queues unique (count + fill) and relabel for the super-batch; nothing here
// waits for the device.  The frontier's size is still on its way when this
// returns: f.frontier() waits for it.
Graph::Frontier& Graph::batch_relabel_launch(torch::Tensor& col_seeds,
                                             const torch::Tensor& row_ids,
                                             torch::Tensor* out_row, torch::Tensor* out_col,
                                             c10::optional<torch::Tensor>* e_ids) {
  TORCH_CHECK(edge_bptr_.defined() && edge_bptr_.numel() > 0,
              "BatchGraphRelabel: the graph has no edge batch pointer");
  ColumnOrderedEdges edges = column_ordered_edges("BatchGraphRelabel");
  col_seeds = ids(col_seeds, "col_seeds");
  // the kernels read seeds[col_bptr[b] ...]: the seeds must be the ones the
  // batch pointer was recorded for
  BatchOffsets::check(col_bptr_, col_seeds.numel(), "BatchGraphRelabel");
  if (edges.col_indptr.defined())
    TORCH_CHECK(edges.col_indptr.numel() == col_seeds.numel() + 1,
                "BatchGraphRelabel: ", col_seeds.numel(), " seeds for a matrix of ",
                edges.col_indptr.numel() - 1, " columns");
  torch::Tensor rows = batch_rows_for_relabel(edges.row, row_ids);
  const int64_t E = rows.numel();
  *out_row = new_ids(E, rows);
  // the column labels that the sampler left go out as they are wherever a batch
  // has distinct seeds (the relabel pass rewrites the other batches in place)
  const bool prefilled = edges.col_indptr.defined() && col_labels_.defined() &&
                         col_labels_.numel() == E && E > 0;
  *out_col = prefilled ? col_labels_ : new_ids(E, rows);
  LabelRequest labels{edges.col.defined() ? cptr(edges.col) : nullptr,
                      edges.col_indptr.defined() ? cptr(edges.col_indptr) : nullptr,
                      mptr(*out_row), mptr(*out_col), prefilled};
  Frontier& f = frontier_for(col_seeds, rows, col_bptr_, edge_bptr_, &labels);
  if (!labels.done)
    GS_CALL(gs_unique_relabel(cptr(col_seeds), cptr(col_bptr_), col_seeds.numel(),
                              cptr(rows), cptr(edge_bptr_), E, f.num_batches,
                              labels.edge_col, labels.col_indptr, labels.out_row,
                              labels.out_col, prefilled ? 1 : 0, f.workspace.data_ptr(),
                              f.workspace.numel(),
                              cur_stream()));
  if (e_ids) *e_ids = edges.e_ids;
  return f;
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
           c10::optional<torch::Tensor>, torch::Tensor>
Graph::BatchGraphRelabel(torch::Tensor col_seeds, torch::Tensor row_ids) {
  torch::Tensor out_row, out_col;
  c10::optional<torch::Tensor> e_ids;
  Frontier& f = batch_relabel_launch(col_seeds, row_ids, &out_row, &out_col, &e_ids);
  return {f.frontier(), f.unique_ptr, out_row, out_col, e_ids, edge_bptr_};
}

std::tuple<torch::Tensor, torch::Tensor> Graph::BatchGetValidNodes(
    torch::Tensor col_seeds, torch::Tensor row_ids) {
  TORCH_CHECK(edge_bptr_.defined() && edge_bptr_.numel() > 0,
              "BatchGetValidNodes: the graph has no edge batch pointer");
  ColumnOrderedEdges edges = column_ordered_edges("BatchGetValidNodes");
  col_seeds = ids(col_seeds, "col_seeds");
  BatchOffsets::check(col_bptr_, col_seeds.numel(), "BatchGetValidNodes");
  torch::Tensor rows = batch_rows_for_relabel(edges.row, row_ids);
  Frontier& f = frontier_for(col_seeds, rows, col_bptr_, edge_bptr_);
  return {f.frontier(), f.unique_ptr};
}

// ------------------------------------------------------------ free operators
std::vector<torch::Tensor> SplitByOffset(torch::Tensor data,
                                         torch::Tensor offset) {
  const std::vector<int64_t>& p = host_offsets(offset);
  std::vector<int64_t> sizes;
  for (size_t i = 0; i + 1 < p.size(); ++i) sizes.push_back(p[i + 1] - p[i]);
  return torch::split_with_sizes(data, sizes);
}

// Per-batch indptr arrays rebased to start at 0; batch i covers columns
// [offset[i], offset[i+1]] of the shared indptr
// (src/cuda/batch/batch_split.cu:53-94).
std::vector<torch::Tensor> SplitIndptrByOffset(torch::Tensor indptr,
                                               torch::Tensor offset) {
  indptr = ids(indptr, "indptr");
  offset = ids(offset, "offset");
  const int64_t B = offset.numel() - 1;
  const std::vector<int64_t>& p = host_offsets(offset);
  std::vector<int64_t> sizes;
  int64_t total = 0;
  for (int64_t i = 0; i < B; ++i) {
    sizes.push_back(p[i + 1] - p[i] + 1);
    total += sizes.back();
  }
  torch::Tensor out = new_ids(total, indptr);
  GS_CALL(gs_split_indptr(cptr(indptr), cptr(offset), B, total, mptr(out),
                          cur_stream()));
  return torch::split_with_sizes(out, sizes);
}

}  // namespace gs
