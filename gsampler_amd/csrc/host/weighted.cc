// weighted.cc -- weighted per-column sampling and the collective (list)
// sampling operators.
#include "abi_call.h"
#include "graph.h"

namespace gs {

static uint64_t take_call_id() { return random_state().next_call++; }

static torch::Tensor f32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined() && t.is_cuda(), name, " must live on the GPU");
  TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be float32 (got ",
              t.scalar_type(), ")");
  return t.contiguous();
}

GraphAndIndex Graph::SamplingProbs(int64_t axis, torch::Tensor edge_probs,
                                   int64_t fanout, bool replace,
                                   int64_t on_format, int64_t output_format) {
  TORCH_CHECK((axis == 1 && on_format == kCSC) || (axis == 0 && on_format == kCSR),
              "SamplingProbs: not implemented for axis ", axis, " on format ",
              on_format);
  const int64_t other = on_format == kCSC ? kCSR : kCSC;
  TORCH_CHECK(output_format != other, "SamplingProbs: on_format ", on_format,
              " cannot produce output_format ", output_format);
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative, got ", fanout);
  const Compressed& m = compressed(on_format);
  torch::Tensor probs = f32(edge_probs, "edge_probs");
  TORCH_CHECK(probs.numel() == m.indices.numel(), "SamplingProbs: ", probs.numel(),
              " probabilities for ", m.indices.numel(), " edges");
  // probabilities follow the original edge order; bring them into this
  // format's order (src/graph_ops.cc:138-142 of the reference)
  if (m.e_ids.has_value()) probs = probs.index_select(0, m.e_ids.value());
  const bool with_coo = output_format & kCOO;
  const int64_t n = m.indptr.numel() - 1;
  MajorResult r;
  r.indptr = new_ids(n + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_scan_workspace_bytes(n + 1), m.indptr);
  GS_CALL(gs_csc_col_count(cptr(m.indptr), n, nullptr, n, fanout, replace ? 1 : 0,
                           mptr(r.indptr), nullptr, nullptr, ws.data_ptr(), ws.numel(),
                           cur_stream()));
  const int64_t nnz = read_last(r.indptr);
  r.minor_ids = new_ids(nnz, m.indptr);
  r.select = new_ids(nnz, m.indptr);
  if (with_coo) r.major_ids = new_ids(nnz, m.indptr);
  torch::Tensor scratch;
  if (replace) scratch = new_ids(m.indices.numel() + 1, m.indptr);
  const RandomState& rs = random_state();
  GS_CALL(gs_csc_col_sample_weighted_fill(
      cptr(m.indptr), n, cptr(m.indices), probs.data_ptr<float>(), nullptr,
      nullptr, n, fanout, replace ? 1 : 0, rs.seed, take_call_id(), cptr(r.indptr),
      nullptr, nullptr,
      replace ? scratch.data_ptr() : nullptr,
      with_coo ? mptr(r.major_ids) : nullptr, mptr(r.minor_ids), mptr(r.select),
      nullptr, 0, cur_stream()));
  GraphPtr g = derive(on_format, output_format, r, num_rows_, num_cols_);
  return {g, edge_index(m.e_ids, r.select)};
}

// ----------------------------------------- fused slice + weighted sampling
torch::Tensor Graph::weight_cdf_for(const torch::Tensor& edge_probs, int64_t format) {
  if (cdf_.defined() && cdf_format_ == format && cdf_probs_.is_same(edge_probs) &&
      cdf_version_ == (int64_t)edge_probs._version() && cdf_epoch_ == cache_epoch())
    return cdf_;
  const Compressed& m = compressed(format);
  torch::Tensor probs = f32(edge_probs, "edge_probs");
  TORCH_CHECK(probs.numel() == m.indices.numel(), "weighted sampling: ", probs.numel(),
              " probabilities for ", m.indices.numel(), " edges");
  if (m.e_ids.has_value()) probs = probs.index_select(0, m.e_ids.value());
  const int64_t n = m.indptr.numel() - 1, nnz = m.indices.numel();
  torch::Tensor cdf = new_ids(nnz + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_weight_cdf_workspace_bytes(n, nnz), m.indptr);
  // the ids on the other axis ride in the CDF's entries
  const int64_t num_minor = format == kCSC ? num_rows_ : num_cols_;
  GS_CALL(gs_weight_cdf_build(cptr(m.indptr), n, cptr(m.indices), num_minor,
                              probs.data_ptr<float>(), nnz, mptr(cdf), ws.data_ptr(),
                              ws.numel(), cur_stream()));
  cdf_ = cdf;
  cdf_probs_ = edge_probs;
  cdf_version_ = edge_probs._version();
  cdf_epoch_ = cache_epoch();
  cdf_format_ = format;
  return cdf_;
}

GraphAndIndex Graph::FusedSlicingSamplingProbs(int64_t axis, torch::Tensor seeds,
                                               torch::Tensor edge_probs,
                                               int64_t fanout, bool replace,
                                               int64_t on_format,
                                               int64_t output_format) {
  TORCH_CHECK((axis == 1 && on_format == kCSC) || (axis == 0 && on_format == kCSR),
              "FusedSlicingSamplingProbs: not implemented for axis ", axis,
              " on format ", on_format);
  const int64_t other = on_format == kCSC ? kCSR : kCSC;
  TORCH_CHECK(output_format != other, "FusedSlicingSamplingProbs: on_format ", on_format,
              " cannot produce output_format ", output_format);
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative, got ", fanout);
  TORCH_CHECK(replace || fanout <= 64,
              "FusedSlicingSamplingProbs: fanout above 64 needs replace=True");
  seeds = ids(seeds, "seeds");
  const Compressed& m = compressed(on_format);
  torch::Tensor cdf = weight_cdf_for(edge_probs, on_format);
  const bool with_coo = output_format & kCOO;
  const int64_t num_major = m.indptr.numel() - 1, n = seeds.numel();
  MajorResult r;
  r.indptr = new_ids(n + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_scan_workspace_bytes(n + 1), m.indptr);
  EdgeCount count;
  torch::Tensor col_span = new_ids(n, m.indptr);  // the columns' starts and degrees, for the fill pass
  GS_CALL(gs_csc_col_count(cptr(m.indptr), num_major, cptr(seeds), n, fanout,
                           replace ? 1 : 0, mptr(r.indptr), count.mirror(), mptr(col_span),
                           ws.data_ptr(), ws.numel(), cur_stream()));
  count.arm(r.indptr);
  const int64_t bound = n * fanout;
  const int64_t size = bound <= kBoundLimit ? bound : count.get();
  r.minor_ids = new_ids(size, m.indptr);
  r.select = new_ids(size, m.indptr);
  if (with_coo) r.major_ids = new_ids(size, m.indptr);
  // (as in the uniform sampler: a super-batched caller without a coordinate form
  // gets the columns' places inside their batches)
  EdgeCount::Hint& hint = EdgeCount::hint();
  const bool label_cols = !with_coo && hint.col_bptr.defined();
  torch::Tensor col_labels = label_cols ? new_ids(size, m.indptr) : torch::Tensor();
  const RandomState& rs = random_state();
  GS_CALL(gs_csc_col_sample_weighted_fill(
      cptr(m.indptr), num_major, cptr(m.indices), nullptr, cptr(cdf), cptr(seeds), n,
      fanout, replace ? 1 : 0, rs.seed, take_call_id(), cptr(r.indptr), cptr(col_span),
      nullptr, nullptr,
      with_coo ? mptr(r.major_ids) : label_cols ? mptr(col_labels) : nullptr,
      mptr(r.minor_ids), mptr(r.select), label_cols ? cptr(hint.col_bptr) : nullptr,
      label_cols ? hint.col_bptr.numel() - 1 : 0, cur_stream()));
  const int64_t nnz = count.get();
  if (label_cols) hint.col_labels = col_labels.narrow(0, 0, nnz);
  r.minor_ids = r.minor_ids.narrow(0, 0, nnz);
  r.select = r.select.narrow(0, 0, nnz);
  if (with_coo) r.major_ids = r.major_ids.narrow(0, 0, nnz);
  const int64_t new_rows = axis == 0 ? n : num_rows_;
  const int64_t new_cols = axis == 0 ? num_cols_ : n;
  GraphPtr g = derive(on_format, output_format, r, new_rows, new_cols);
  return {g, edge_index(m.e_ids, r.select)};
}

GraphAndIndex Graph::BatchFusedSlicingSamplingProbs(torch::Tensor seeds,
                                                    torch::Tensor col_bptr,
                                                    torch::Tensor edge_probs,
                                                    int64_t fanout, bool replace) {
  col_bptr = ids(col_bptr, "col_bptr");
  BatchOffsets::check(col_bptr, seeds.numel(), "BatchFusedSlicingSamplingProbs");
  EdgeCount::HintScope batch(col_bptr);  // the sampler leaves the edge pointer here
  // compressed by column only, as the uniform twin: the relabel pass reads the
  // column pointer and the labels the sampler left
  auto ret = FusedSlicingSamplingProbs(1, seeds, edge_probs, fanout, replace, kCSC, kCSC);
  Graph& g = *std::get<0>(ret);
  g.col_labels_ = EdgeCount::hint().col_labels;
  g.col_bptr_ = col_bptr;
  g.orig_col_ids_ = ids(seeds, "seeds");
  g.edge_bptr_ = EdgeCount::hint().edge_bptr;
  if (!g.edge_bptr_.defined()) g.edge_bptr_ = g.csc_->indptr.index_select(0, col_bptr);
  BatchOffsets::trust(g.edge_bptr_, g.num_edges_);
  return ret;
}

// ------------------------------------------------------------ list sampling
torch::Tensor ListSampling(int64_t num_items, int64_t num_picks, bool replace) {
  TORCH_CHECK(num_items >= 0 && num_picks >= 0, "ListSampling: negative size");
  const int64_t count = replace ? (num_items > 0 ? num_picks : 0)
                                : std::min(num_items, num_picks);
  torch::Tensor out = torch::empty(
      {count}, torch::TensorOptions().dtype(torch::kInt64).device(torch::kCUDA));
  const RandomState& rs = random_state();
  GS_CALL(gs_list_sample_uniform(num_items, num_picks, replace ? 1 : 0,
                                 (int)rs.algo, rs.seed, take_call_id(), mptr(out),
                                 cur_stream()));
  return out;
}

static std::tuple<torch::Tensor, torch::Tensor> list_weighted(
    const torch::Tensor& probs_in, int64_t num_picks, bool replace,
    const torch::Tensor& range) {
  TORCH_CHECK(num_picks >= 0, "list sampling: negative number of picks");
  torch::Tensor probs = f32(probs_in, "probs");
  const int64_t n = probs.numel();
  const int64_t nseg = range.defined() ? range.numel() - 1 : 1;
  TORCH_CHECK(nseg >= 1, "list sampling: range needs at least two entries");
  if (range.defined()) BatchOffsets::check(range, n, "list sampling");
  torch::Tensor ws = new_workspace(gs_list_sample_workspace_bytes(n, nseg), probs);
  torch::Tensor out_range = new_ids(nseg + 1, probs);
  GS_CALL(gs_list_sample_weighted_count(cptr(range), n, nseg, num_picks,
                                        replace ? 1 : 0, mptr(out_range),
                                        ws.data_ptr(), ws.numel(), cur_stream()));
  BatchOffsets::trust(out_range);
  // The number of picks follows from the sizes alone, so it is worked out here
  // instead of being read back from the device (which would wait for all the
  // work queued so far): the segment sizes of a range are already on the host,
  // where its check left them.
  auto picks_of = [&](int64_t size) {
    return replace ? (size > 0 ? num_picks : 0) : std::min(size, num_picks);
  };
  int64_t total = 0;
  if (range.defined()) {
    const std::vector<int64_t>& p = OffsetMirror::values(range);
    for (size_t b = 0; b + 1 < p.size(); ++b) total += picks_of(p[b + 1] - p[b]);
  } else {
    total = picks_of(n);
  }
  torch::Tensor out = new_ids(total, probs);
  const RandomState& rs = random_state();
  GS_CALL(gs_list_sample_weighted_fill(
      probs.data_ptr<float>(), cptr(range), n, nseg, num_picks, replace ? 1 : 0,
      rs.seed, take_call_id(), cptr(out_range), total, mptr(out), ws.data_ptr(),
      ws.numel(), cur_stream()));
  return {out, out_range};
}

torch::Tensor ListSamplingProbs(torch::Tensor probs, int64_t num_picks,
                                bool replace) {
  return std::get<0>(list_weighted(probs, num_picks, replace, {}));
}

std::tuple<torch::Tensor, torch::Tensor> BatchListSamplingProbs(
    torch::Tensor probs, int64_t num_picks, bool replace, torch::Tensor range) {
  return list_weighted(probs, num_picks, replace, ids(range, "range"));
}

// Uniform batched selection = weighted selection with unit weights over the
// items the range covers (src/tensor_ops.cc:21-28 of the reference, which
// sizes the weights by the number of segments; the number of items is meant).
std::tuple<torch::Tensor, torch::Tensor> BatchListSampling(int64_t num_picks,
                                                           bool replace,
                                                           torch::Tensor range) {
  range = ids(range, "range");
  const int64_t n = read_last(range);
  torch::Tensor ones = torch::ones(
      {n}, torch::TensorOptions().dtype(torch::kFloat32).device(range.device()));
  return list_weighted(ones, num_picks, replace, range);
}

}  // namespace gs
