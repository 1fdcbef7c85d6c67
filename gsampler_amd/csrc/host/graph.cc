// graph.cc -- format management and the extract / select / finalize operators
// of gs_classes.Graph.  Each operator validates its tensors, sizes outputs and
// workspaces through torch, and calls the C ABI on the current HIP stream.
#include "graph.h"

#include <limits>

#include "abi_call.h"

#include <mutex>

namespace gs {

RandomState& random_state() {
  static RandomState state;
  return state;
}

static uint64_t next_call_id() { return random_state().next_call++; }

// ------------------------------------------------------------------ loading
// A loaded matrix is checked once (a few reductions and one read-back): every
// kernel afterwards trusts offsets and ids, and a malformed array would send
// its loads out of bounds.  The reference loads without looking
// (src/graph.h:19-37).
static void check_ids_below(const torch::Tensor& ids, int64_t bound, const char* who,
                            const char* name) {
  if (ids.numel() == 0) return;
  const int64_t lo = ids.min().item<int64_t>(), hi = ids.max().item<int64_t>();
  TORCH_CHECK(lo >= 0 && hi < bound, who, ": ", name, " must lie in [0, ", bound,
              "), found ", lo, " .. ", hi);
}

static void check_compressed(const torch::Tensor& indptr, const torch::Tensor& indices,
                             int64_t num_minor, const char* who) {
  const int64_t first = indptr[0].item<int64_t>();
  const int64_t last = indptr[indptr.numel() - 1].item<int64_t>();
  TORCH_CHECK(first == 0 && last == indices.numel(), who, ": indptr must run from 0 to ",
              indices.numel(), " (the number of indices), found ", first, " .. ", last);
  if (indptr.numel() > 1)
    TORCH_CHECK(indptr.slice(0, 1).ge(indptr.slice(0, 0, indptr.numel() - 1)).all().item<bool>(),
                who, ": indptr must not decrease");
  check_ids_below(indices, num_minor, who, "indices");
}

void Graph::LoadCSC(torch::Tensor indptr, torch::Tensor indices) {
  invalidate_caches();  // whatever was derived from an earlier matrix of this object
  auto m = std::make_shared<Compressed>();
  m->indptr = graph_ids(indptr, "indptr");
  m->indices = graph_ids(indices, "indices");
  TORCH_CHECK(m->indptr.numel() == num_cols_ + 1, "LoadCSC: indptr has ",
              indptr.numel(), " entries for ", num_cols_, " columns");
  check_compressed(m->indptr, m->indices, num_rows_, "LoadCSC");
  m->num_minor = num_rows_;
  csc_ = m;
  num_edges_ = indices.numel();
}

void Graph::LoadCSR(torch::Tensor indptr, torch::Tensor indices) {
  invalidate_caches();  // whatever was derived from an earlier matrix of this object
  auto m = std::make_shared<Compressed>();
  m->indptr = graph_ids(indptr, "indptr");
  m->indices = graph_ids(indices, "indices");
  TORCH_CHECK(m->indptr.numel() == num_rows_ + 1, "LoadCSR: indptr has ",
              indptr.numel(), " entries for ", num_rows_, " rows");
  check_compressed(m->indptr, m->indices, num_cols_, "LoadCSR");
  m->num_minor = num_cols_;
  csr_ = m;
  num_edges_ = indices.numel();
}

void Graph::LoadCOO(torch::Tensor row, torch::Tensor col, bool row_sorted,
                    bool col_sorted) {
  invalidate_caches();  // whatever was derived from an earlier matrix of this object
  auto m = std::make_shared<Coordinate>();
  m->row = graph_ids(row, "row");
  m->col = graph_ids(col, "col");
  TORCH_CHECK(row.numel() == col.numel(), "LoadCOO: row and col differ in length");
  check_ids_below(m->row, num_rows_, "LoadCOO", "row ids");
  check_ids_below(m->col, num_cols_, "LoadCOO", "column ids");
  m->row_sorted = row_sorted;
  m->col_sorted = col_sorted;
  coo_ = m;
  num_edges_ = row.numel();
}

// --------------------------------------------------------- format conversion
// CSC/CSR -> COO: the id on the compressed axis of every edge position.
static torch::Tensor expand_indptr(const torch::Tensor& indptr, int64_t nnz) {
  torch::Tensor out = new_ids(nnz, indptr);
  GS_CALL(gs_csc2coo(cptr(indptr), indptr.numel() - 1, nnz, mptr(out),
                     cur_stream()));
  return out;
}

// COO -> CSC/CSR along `major`: stable sort by the major id (the permutation is
// kept as e_ids, like the reference's COO2CSC, src/cuda/format_transform.cu:
// 121-142), then indptr by binary search.
static std::shared_ptr<Compressed> compress(const Coordinate& coo, bool by_col,
                                            int64_t num_major) {
  const torch::Tensor& major = by_col ? coo.col : coo.row;
  const torch::Tensor& minor = by_col ? coo.row : coo.col;
  const bool sorted = by_col ? coo.col_sorted : coo.row_sorted;
  auto out = std::make_shared<Compressed>();
  torch::Tensor sorted_major;
  if (sorted) {
    sorted_major = major;
    out->indices = minor;
    out->e_ids = coo.e_ids;
  } else {
    const int64_t nnz = major.numel();
    torch::Tensor perm = new_ids(nnz, major);
    sorted_major = new_ids(nnz, major);
    torch::Tensor ws = new_workspace(gs_coo_sort_workspace_bytes(nnz, num_major), major);
    GS_CALL(gs_coo_sort(cptr(major), nnz, num_major, mptr(sorted_major), mptr(perm),
                        ws.data_ptr(), (size_t)ws.numel(), cur_stream()));
    out->indices = GatherRows(minor, perm);
    out->e_ids = coo.e_ids.has_value() ? GatherRows(coo.e_ids.value(), perm) : perm;
    // A format conversion is no part of a sampling step: it can afford to wait for
    // the sort and look at its gave-up flag.
    const int64_t flag_at = gs_coo_sort_flag_offset(nnz, num_major);
    if (nnz > 0 && flag_at >= 0) {
      const torch::Tensor flag = ws.narrow(0, flag_at, 4).view(torch::kInt32).cpu();
      TORCH_CHECK(flag.item<int32_t>() == 0,
                  "coo_sort: a pass gave up waiting for the counts of an earlier tile");
    }
  }
  out->indptr = new_ids(num_major + 1, major);
  GS_CALL(gs_sorted_to_indptr(cptr(sorted_major), sorted_major.numel(),
                              num_major, mptr(out->indptr), cur_stream()));
  return out;
}

static std::shared_ptr<Coordinate> expand(const Compressed& m, bool is_csc) {
  auto coo = std::make_shared<Coordinate>();
  torch::Tensor major = expand_indptr(m.indptr, m.indices.numel());
  coo->row = is_csc ? m.indices : major;
  coo->col = is_csc ? major : m.indices;
  coo->e_ids = m.e_ids;
  coo->col_sorted = is_csc;
  coo->row_sorted = !is_csc;
  return coo;
}

void Graph::CreateSparseFormat(int64_t format) {
  TORCH_CHECK(csc_ || csr_ || coo_, "the graph holds no sparse format yet");
  const bool have = (format == kCOO && coo_) || (format == kCSC && csc_) ||
                    (format == kCSR && csr_);
  if (!have) {
    const torch::Tensor& any = csc_ ? csc_->indices : csr_ ? csr_->indices : coo_->row;
    TORCH_CHECK(any.is_cuda(), "a matrix in pinned host memory is not converted to "
                "another sparse format: load the format the operator runs on");
  }
  if (format == kCOO) {
    if (coo_) return;
    coo_ = csc_ ? expand(*csc_, true) : expand(*csr_, false);
  } else if (format == kCSC) {
    if (csc_) return;
    if (!coo_) coo_ = expand(*csr_, false);
    csc_ = compress(*coo_, true, num_cols_);
    csc_->num_minor = num_rows_;
  } else if (format == kCSR) {
    if (csr_) return;
    if (!coo_) coo_ = expand(*csc_, true);
    csr_ = compress(*coo_, false, num_rows_);
    csr_->num_minor = num_cols_;
  } else {
    TORCH_CHECK(false, "unsupported sparse format ", format);
  }
}

static torch::Tensor or_empty(const c10::optional<torch::Tensor>& t) {
  return t.has_value() ? t.value() : torch::Tensor();
}

torch::Tensor Graph::GetCSCIndptr() { CreateSparseFormat(kCSC); return csc_->indptr; }
torch::Tensor Graph::GetCSCIndices() { CreateSparseFormat(kCSC); return csc_->indices; }
torch::Tensor Graph::GetCSCEids() { CreateSparseFormat(kCSC); return or_empty(csc_->e_ids); }
torch::Tensor Graph::GetCOORows() { CreateSparseFormat(kCOO); return coo_->row; }
torch::Tensor Graph::GetCOOCols() { CreateSparseFormat(kCOO); return coo_->col; }
torch::Tensor Graph::GetCOOEids() { CreateSparseFormat(kCOO); return or_empty(coo_->e_ids); }
torch::Tensor Graph::GetCSRIndptr() { CreateSparseFormat(kCSR); return csr_->indptr; }
torch::Tensor Graph::GetCSRIndices() { CreateSparseFormat(kCSR); return csr_->indices; }
torch::Tensor Graph::GetCSREids() { CreateSparseFormat(kCSR); return or_empty(csr_->e_ids); }

const Compressed& Graph::compressed(int64_t format) {
  CreateSparseFormat(format);
  return format == kCSC ? *csc_ : *csr_;
}

// ---------------------------------------------------- operators, major axis
MajorResult major_slice(const Compressed& m, const torch::Tensor& picked,
                               bool with_coo, const torch::Tensor& batch_ptr,
                               int64_t encode_stride) {
  const int64_t num_major = m.indptr.numel() - 1;
  const int64_t n = picked.numel();
  MajorResult r;
  r.indptr = new_ids(n + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_scan_workspace_bytes(n + 1), m.indptr);
  GS_CALL(gs_csc_col_count(cptr(m.indptr), num_major, cptr(picked), n, -1, 0,
                           mptr(r.indptr), nullptr, nullptr, ws.data_ptr(), ws.numel(),
                           cur_stream()));
  const int64_t nnz = read_last(r.indptr);
  r.minor_ids = new_ids(nnz, m.indptr);
  r.select = new_ids(nnz, m.indptr);
  if (with_coo) r.major_ids = new_ids(nnz, m.indptr);
  const int64_t nb = batch_ptr.defined() ? batch_ptr.numel() - 1 : 0;
  GS_CALL(gs_csc_col_slice_fill(
      cptr(m.indptr), num_major, cptr(m.indices), cptr(picked), n,
      cptr(r.indptr), nnz, nb > 0 ? cptr(batch_ptr) : nullptr, nb,
      encode_stride, with_coo ? mptr(r.major_ids) : nullptr, mptr(r.minor_ids),
      mptr(r.select), cur_stream()));
  return r;
}

// The int32 copy pays from a few megabytes of ids on (below that the int64
// array stays in cache anyway); undefined when the matrix does not qualify.
const torch::Tensor& Compressed::narrow_indices() const {
  constexpr int64_t kMinEdges = int64_t(1) << 20;
  // one matrix is shared by every handle derived from it and by every sampler
  // thread: the copy is made (and dropped) under a lock
  static std::mutex guard;
  std::lock_guard<std::mutex> lock(guard);
  const int64_t version = (int64_t)indices._version();
  if (indices32.defined() &&
      (indices32_version != version || indices32_source != indices.data_ptr() ||
       indices32_epoch != cache_epoch() || !narrow_ids_allowed().load()))
    indices32 = torch::Tensor();  // edited, another array, or switched off
  if (!indices32.defined() && narrow_ids_allowed().load() && num_minor >= 0 &&
      num_minor < (int64_t(1) << 31) && indices.is_cuda() && indices.numel() >= kMinEdges) {
    indices32 = indices.to(torch::kInt32);
    indices32_version = version;
    indices32_epoch = cache_epoch();
    indices32_source = indices.data_ptr();
  }
  return indices32;
}

// picked undefined: sample every column of the matrix itself.
MajorResult major_sample_uniform(const Compressed& m,
                                        const torch::Tensor& picked,
                                        int64_t fanout, bool replace,
                                        bool with_coo) {
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative, got ", fanout);
  const int64_t num_major = m.indptr.numel() - 1;
  const bool fused = picked.defined();
  const int64_t n = fused ? picked.numel() : num_major;
  MajorResult r;
  r.indptr = new_ids(n + 1, m.indptr);
  torch::Tensor ws = new_workspace(gs_scan_workspace_bytes(n + 1), m.indptr);
  // No column yields more than fanout edges: size the outputs by that bound,
  // launch, and trim when the count has arrived.
  EdgeCount count;
  // the count pass leaves every column's start and degree for the fill pass, which
  // then does not look the column pointer up a second time
  torch::Tensor col_span = new_ids(n, m.indptr);
  GS_CALL(gs_csc_col_count(cptr(m.indptr), num_major,
                           fused ? cptr(picked) : nullptr, n, fanout,
                           replace ? 1 : 0, mptr(r.indptr), count.mirror(), mptr(col_span),
                           ws.data_ptr(), ws.numel(), cur_stream()));
  count.arm(r.indptr);
  const int64_t bound = n * fanout;
  const int64_t size = bound <= kBoundLimit ? bound : count.get();
  r.minor_ids = new_ids(size, m.indptr);
  r.select = new_ids(size, m.indptr);
  if (with_coo) r.major_ids = new_ids(size, m.indptr);
  // a super-batched caller that asked for no coordinate form gets the columns'
  // places inside their batches instead (EdgeCount::Hint)
  EdgeCount::Hint& hint = EdgeCount::hint();
  const bool label_cols = !with_coo && fused && hint.col_bptr.defined();
  torch::Tensor col_labels = label_cols ? new_ids(size, m.indptr) : torch::Tensor();
  int64_t* out_col = with_coo ? mptr(r.major_ids) : label_cols ? mptr(col_labels) : nullptr;
  const int64_t* col_batch_ptr = label_cols ? cptr(hint.col_bptr) : nullptr;
  const int64_t col_batches = label_cols ? hint.col_bptr.numel() - 1 : 0;
  const RandomState& rs = random_state();
  const torch::Tensor& narrow = m.narrow_indices();
  if (narrow.defined()) {
    GS_CALL(gs_csc_col_sample_uniform_fill_i32(
        cptr(m.indptr), num_major, narrow.data_ptr<int32_t>(),
        fused ? cptr(picked) : nullptr, n, fanout, replace ? 1 : 0, (int)rs.algo,
        rs.seed, next_call_id(), cptr(r.indptr), cptr(col_span), out_col, mptr(r.minor_ids),
        mptr(r.select),
        col_batch_ptr, col_batches, cur_stream()));
  } else {
    GS_CALL(gs_csc_col_sample_uniform_fill(
        cptr(m.indptr), num_major, cptr(m.indices),
        fused ? cptr(picked) : nullptr, n, fanout, replace ? 1 : 0, (int)rs.algo,
        rs.seed, next_call_id(), cptr(r.indptr), cptr(col_span), out_col, mptr(r.minor_ids),
        mptr(r.select),
        col_batch_ptr, col_batches, cur_stream()));
  }
  const int64_t nnz = count.get();
  if (label_cols) hint.col_labels = col_labels.narrow(0, 0, nnz);
  r.minor_ids = r.minor_ids.narrow(0, 0, nnz);
  r.select = r.select.narrow(0, 0, nnz);
  if (with_coo) r.major_ids = r.major_ids.narrow(0, 0, nnz);
  return r;
}

// Wraps a MajorResult into a new Graph in the requested output formats
// (bit-OR of kCOO and the format the operator ran on).
GraphPtr Graph::derive(int64_t on_format, int64_t output_format,
                       const MajorResult& r, int64_t new_rows,
                       int64_t new_cols) {
  auto g = c10::make_intrusive<Graph>(new_rows, new_cols);
  const bool is_csc = on_format == kCSC;
  if (output_format & on_format) {
    auto c = std::make_shared<Compressed>();
    c->indptr = r.indptr;
    c->indices = r.minor_ids;
    (is_csc ? g->csc_ : g->csr_) = c;
  }
  if (output_format & kCOO) {
    auto coo = std::make_shared<Coordinate>();
    coo->row = is_csc ? r.minor_ids : r.major_ids;
    coo->col = is_csc ? r.major_ids : r.minor_ids;
    coo->col_sorted = is_csc;
    coo->row_sorted = !is_csc;
    g->coo_ = coo;
  }
  g->num_edges_ = r.select.numel();
  return g;
}

// out[i] = table[ids[i]] along the first axis.  The table may be a pinned host
// tensor, which the kernel reads in place (IndexSelectCPUFromGPU,
// src/cuda/index_select_uvm.cu:22-50, and dgl's gather_pinned_tensor_rows that
// python/gs/matrix_api/matrix.py:19-23 calls for pinned edge data).
// The edge index that the latest slice along a compressed axis returned, with
// where its edges come from.  A slice copies runs of the parent's edges, so
// scalar edge data of the slice (data[edge_index], which the Python layer asks
// for right after slicing) can be copied by column ranges of the parent's
// array without reading the 8-byte positions back.  Recognised by the identity
// and version of the index tensor; one entry per thread, replaced by the next
// slice.  The index itself (8 bytes per edge) is held weakly, so the entry does
// not keep it alive after its users are gone; the three small arrays the copy
// kernel reads are held.
struct SliceRuns {
  c10::optional<c10::weak_intrusive_ptr<c10::TensorImpl>> select;
  torch::Tensor parent_indptr, picked, sub_indptr;
  int64_t version = -1, parent_edges = 0, epoch = -1;
  int64_t source_versions[3] = {-1, -1, -1};  // of parent_indptr, picked, sub_indptr
  static SliceRuns& last() {
    static thread_local SliceRuns s;
    return s;
  }
  static void remember(const torch::Tensor& select, const torch::Tensor& parent_indptr,
                       const torch::Tensor& picked, const torch::Tensor& sub_indptr,
                       int64_t parent_edges) {
    SliceRuns& s = last();
    s.parent_edges = parent_edges;
    s.select = c10::weak_intrusive_ptr<c10::TensorImpl>(select.getIntrusivePtr());
    s.parent_indptr = parent_indptr;
    s.picked = picked;
    s.sub_indptr = sub_indptr;
    s.version = (int64_t)select._version();
    s.epoch = cache_epoch();
    s.source_versions[0] = (int64_t)parent_indptr._version();
    s.source_versions[1] = (int64_t)picked._version();
    s.source_versions[2] = (int64_t)sub_indptr._version();
  }
  // the index is the one remembered and nothing was written to since
  bool covers(const torch::Tensor& ids) const {
    if (!select.has_value() || !ids.defined()) return false;
    // a live target cannot have been replaced by another tensor at the same address
    const c10::intrusive_ptr<c10::TensorImpl> held = select->lock();
    return held && held.get() == ids.unsafeGetTensorImpl() && epoch == cache_epoch() &&
           (int64_t)ids._version() == version &&
           (int64_t)parent_indptr._version() == source_versions[0] &&
           (int64_t)picked._version() == source_versions[1] &&
           (int64_t)sub_indptr._version() == source_versions[2];
  }
};

torch::Tensor GatherRows(torch::Tensor table, torch::Tensor ids) {
  TORCH_CHECK(table.dim() >= 1, "GatherRows: the table needs at least one axis");
  {
    const SliceRuns& runs = SliceRuns::last();
    if (runs.covers(ids) && table.is_cuda() && table.dim() == 1 && table.is_contiguous() &&
        (table.element_size() == 4 || table.element_size() == 8) &&
        table.numel() >= runs.parent_edges) {
      torch::Tensor out = torch::empty({ids.numel()}, table.options());
      GS_CALL(gs_csc_col_slice_values(cptr(runs.parent_indptr), cptr(runs.picked),
                                      runs.picked.numel(), cptr(runs.sub_indptr), ids.numel(),
                                      table.data_ptr(), (int64_t)table.element_size(),
                                      out.data_ptr(), cur_stream()));
      return out;
    }
  }
  TORCH_CHECK(table.is_cuda() || table.is_pinned(),
              "GatherRows: the table must be on the GPU or in pinned host memory");
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == torch::kInt64 && ids.dim() == 1,
              "GatherRows: ids must be a 1-D int64 GPU tensor");
  table = table.contiguous();
  ids = ids.contiguous();
  std::vector<int64_t> shape = table.sizes().vec();
  shape[0] = ids.numel();
  torch::Tensor out = torch::empty(shape, table.options().device(ids.device()).pinned_memory(false));
  int64_t row_bytes = (int64_t)table.element_size();
  for (size_t d = 1; d < shape.size(); ++d) row_bytes *= shape[d];
  GS_CALL(gs_gather_rows(table.numel() ? table.data_ptr() : nullptr, table.size(0),
                         row_bytes, cptr(ids), ids.numel(),
                         out.numel() ? out.data_ptr() : nullptr, nullptr, cur_stream()));
  return out;
}

torch::Tensor Graph::edge_index(const c10::optional<torch::Tensor>& parent_eids,
                                const torch::Tensor& select) {
  if (!parent_eids.has_value()) return select;
  if (parent_eids.value().is_pinned()) return GatherRows(parent_eids.value(), select);
  return parent_eids.value().index_select(0, select);
}

static void check_out_format(int64_t on_format, int64_t output_format,
                             const char* op) {
  TORCH_CHECK(on_format == kCSC || on_format == kCSR || on_format == kCOO, op,
              ": unknown on_format ", on_format);
  const int64_t other = on_format == kCSC ? kCSR : kCSC;
  TORCH_CHECK(on_format == kCOO || output_format != other, op,
              ": on_format ", on_format, " cannot produce output_format ",
              output_format);
}

// axis 0 = rows, axis 1 = columns (src/graph.cc:88-89 of the reference).
GraphAndIndex Graph::Slicing(torch::Tensor seeds, int64_t axis,
                             int64_t on_format, int64_t output_format) {
  check_out_format(on_format, output_format, "Slicing");
  TORCH_CHECK(axis == 0 || axis == 1, "Slicing: axis must be 0 or 1");
  seeds = ids(seeds, "seeds");
  const int64_t new_rows = axis == 0 ? seeds.numel() : num_rows_;
  const int64_t new_cols = axis == 0 ? num_cols_ : seeds.numel();
  if (on_format == kCOO) return slice_coo(seeds, axis, new_rows, new_cols);
  const Compressed& m = compressed(on_format);
  const bool with_coo = output_format & kCOO;
  const bool along_major = (on_format == kCSC) == (axis == 1);
  MajorResult r = along_major ? major_slice(m, seeds, with_coo, {}, 0)
                              : minor_slice(m, seeds, with_coo);
  GraphPtr g = derive(on_format, output_format, r, new_rows, new_cols);
  if (along_major && !m.e_ids.has_value()) SliceRuns::remember(r.select, m.indptr, seeds, r.indptr, m.indices.numel());
  return {g, edge_index(m.e_ids, r.select)};
}

GraphAndIndex Graph::Sampling(int64_t axis, int64_t fanout, bool replace,
                              int64_t on_format, int64_t output_format) {
  check_out_format(on_format, output_format, "Sampling");
  TORCH_CHECK((axis == 1 && on_format == kCSC) || (axis == 0 && on_format == kCSR),
              "Sampling: not implemented for axis ", axis, " on format ",
              on_format);
  const Compressed& m = compressed(on_format);
  MajorResult r = major_sample_uniform(m, {}, fanout, replace, output_format & kCOO);
  GraphPtr g = derive(on_format, output_format, r, num_rows_, num_cols_);
  return {g, edge_index(m.e_ids, r.select)};
}

GraphAndIndex Graph::FusedSlicingSampling(int64_t axis, torch::Tensor seeds,
                                          int64_t fanout, bool replace,
                                          int64_t on_format,
                                          int64_t output_format) {
  check_out_format(on_format, output_format, "FusedSlicingSampling");
  TORCH_CHECK((axis == 1 && on_format == kCSC) || (axis == 0 && on_format == kCSR),
              "FusedSlicingSampling: not implemented for axis ", axis,
              " on format ", on_format);
  seeds = ids(seeds, "seeds");
  const Compressed& m = compressed(on_format);
  MajorResult r = major_sample_uniform(m, seeds, fanout, replace, output_format & kCOO);
  const int64_t new_rows = axis == 0 ? seeds.numel() : num_rows_;
  const int64_t new_cols = axis == 0 ? num_cols_ : seeds.numel();
  GraphPtr g = derive(on_format, output_format, r, new_rows, new_cols);
  return {g, edge_index(m.e_ids, r.select)};
}

// ------------------------------------------------------- unique and relabel
bool Graph::Frontier::matches(const torch::Tensor& s, const torch::Tensor& r,
                              const torch::Tensor& sp,
                              const torch::Tensor& rp) const {
  auto same = [](const torch::Tensor& a, const torch::Tensor& b) {
    if (!a.defined() || !b.defined()) return a.defined() == b.defined();
    return a.is_same(b) ||
           (a.data_ptr() == b.data_ptr() && a.numel() == b.numel());
  };
  return same(seeds, s) && same(rows, r) && same(seeds_ptr, sp) &&
         same(rows_ptr, rp) && seeds_version == (int64_t)s._version() &&
         rows_version == (int64_t)r._version() && epoch == cache_epoch();
}

// Unique (first-occurrence order) of seeds_b ++ rows_b per batch; the hash
// tables stay in the workspace for the relabel pass.
Graph::Frontier& Graph::frontier_for(const torch::Tensor& seeds,
                                     const torch::Tensor& rows,
                                     const torch::Tensor& seeds_ptr,
                                     const torch::Tensor& rows_ptr,
                                     LabelRequest* labels) {
  if (frontier_ && frontier_->matches(seeds, rows, seeds_ptr, rows_ptr))
    return *frontier_;
  auto f = std::make_unique<Frontier>();
  f->seeds = seeds;
  f->rows = rows;
  f->seeds_ptr = seeds_ptr;
  f->rows_ptr = rows_ptr;
  f->seeds_version = seeds._version();
  f->rows_version = rows._version();
  f->epoch = cache_epoch();
  const int64_t B = seeds_ptr.defined() ? seeds_ptr.numel() - 1 : 1;
  TORCH_CHECK(B >= 1, "unique: at least one batch is required");
  f->num_batches = B;
  const int64_t S = seeds.numel(), E = rows.numel();
  f->workspace = new_workspace(gs_unique_workspace_bytes(S, E, B), rows);
  f->unique_ptr = new_ids(B + 1, rows);
  // The whole pointer array goes to the host as well, written there by the kernel
  // that computes it: its last entry is the size of the frontier, the rest is
  // what per-batch splits ask for later.
  int64_t* mirror = OffsetMirror::reserve(f->unique_ptr);
  GS_CALL(gs_unique_count(cptr(seeds), cptr(seeds_ptr), S, cptr(rows),
                          cptr(rows_ptr), E, B, mptr(f->unique_ptr), mirror,
                          f->workspace.data_ptr(), f->workspace.numel(),
                          cur_stream()));
  OffsetMirror::arm(f->unique_ptr);
  BatchOffsets::trust(f->unique_ptr);
  // at most S + E unique keys
  f->unique_buffer =
      new_ids(S + E <= kBoundLimit ? S + E : f->total(), rows);
  if (labels) {
    GS_CALL(gs_unique_fill_relabel(cptr(seeds), cptr(seeds_ptr), S, cptr(rows),
                                   cptr(rows_ptr), E, B, cptr(f->unique_ptr),
                                   mptr(f->unique_buffer), labels->edge_col,
                                   labels->col_indptr, labels->out_row, labels->out_col,
                                   labels->col_prefilled ? 1 : 0, f->workspace.data_ptr(),
                                   f->workspace.numel(), cur_stream()));
    labels->done = true;
  } else {
    GS_CALL(gs_unique_fill(cptr(seeds), cptr(seeds_ptr), S, cptr(rows),
                           cptr(rows_ptr), E, B, cptr(f->unique_ptr),
                           mptr(f->unique_buffer), f->workspace.data_ptr(),
                           f->workspace.numel(), cur_stream()));
  }
  frontier_ = std::move(f);
  return *frontier_;
}

// row_ids[base] when row_ids is non-empty (rows of a compacted or row-sliced
// matrix are local ids), else base.  The gathered tensor is kept so that
// all_nodes() and to_dgl_block() on the same matrix share one frontier.
torch::Tensor Graph::mapped_rows(const torch::Tensor& base,
                                 const torch::Tensor& row_ids) {
  if (row_ids.numel() == 0) return base;
  torch::Tensor table = ids(row_ids, "row_ids");
  if (!(mapped_out_.defined() && mapped_from_.is_same(base) &&
        mapped_by_.is_same(row_ids))) {
    mapped_out_ = table.index_select(0, base);
    mapped_from_ = base;
    mapped_by_ = row_ids;
  }
  return mapped_out_;
}

// Worth it when the edges outnumber the listed ids by far (a layer-wise
// sampler keeps a few hundred rows and millions of edges between them).
bool Graph::use_list_labels(const torch::Tensor& col_seeds,
                            const torch::Tensor& row_ids) const {
  const int64_t R = row_ids.numel(), S = col_seeds.numel();
  return R > 0 && coo_ && coo_->row.numel() >= 8 * (R + S);
}

// The frontier is the unique of seeds ++ row_ids[coo.row] in first-occurrence
// order.  Every edge of local row l carries the same key row_ids[l], so the
// listed ids, ordered by the first edge that uses them, give the same frontier
// as the edges themselves; ids that no edge uses are replaced by a key that is
// already there.  One pass over the edges (first position per local row)
// replaces hashing every edge.
Graph::ListLabels& Graph::list_labels_for(const torch::Tensor& col_seeds,
                                          const torch::Tensor& row_ids) {
  const torch::Tensor& base = coo_->row;
  if (list_labels_ && list_labels_->base.is_same(base) &&
      list_labels_->row_ids.is_same(row_ids) && list_labels_->seeds.is_same(col_seeds) &&
      list_labels_->row_ids_version == (int64_t)row_ids._version() &&
      list_labels_->seeds_version == (int64_t)col_seeds._version() &&
      list_labels_->epoch == cache_epoch())
    return *list_labels_;
  auto out = std::make_unique<ListLabels>();
  out->base = base;
  out->row_ids = row_ids;
  out->seeds = col_seeds;
  out->row_ids_version = row_ids._version();
  out->seeds_version = col_seeds._version();
  out->epoch = cache_epoch();
  torch::Tensor table = ids(row_ids, "row_ids");
  const int64_t R = table.numel(), S = col_seeds.numel(), E = base.numel();
  torch::Tensor first = new_ids(R, base);
  GS_CALL(gs_first_position(cptr(base), E, R, mptr(first), cur_stream()));
  if (R + S <= GS_LIST_LABELS_MAX_KEYS) {
    // few enough keys for one work-group: frontier and labels in one launch
    torch::Tensor frontier = new_ids(R + S, base);
    out->label_by_local = new_ids(R, base);
    out->seed_label = new_ids(S, base);
    AsyncCount count = AsyncCount::mirrored();
    GS_CALL(gs_list_labels(cptr(col_seeds), S, cptr(table), cptr(first), R, mptr(frontier),
                           nullptr, count.mirror(), mptr(out->label_by_local),
                           mptr(out->seed_label), cur_stream()));
    count.arm();
    out->frontier_bound = frontier;
    out->frontier_count = count;
    list_labels_ = std::move(out);
    return *list_labels_;
  }
  auto sorted = torch::sort(first);  // R values: which listed id is met first
  const torch::Tensor& when = std::get<0>(sorted);
  const torch::Tensor& order = std::get<1>(sorted);
  torch::Tensor keys = table.index_select(0, order);
  // E > 0, so the earliest listed id is used by some edge
  keys = torch::where(when != std::numeric_limits<int64_t>::max(), keys, keys.select(0, 0));
  torch::Tensor rows = torch::cat({keys, col_seeds});  // the seeds again: their labels
  Frontier& f = frontier_for(col_seeds, rows, {}, {});
  torch::Tensor labels = new_ids(R + S, base);
  GS_CALL(gs_unique_relabel(cptr(col_seeds), nullptr, S, cptr(rows), nullptr, R + S, 1,
                            nullptr, nullptr, mptr(labels), nullptr, 0, f.workspace.data_ptr(),
                            f.workspace.numel(), cur_stream()));
  out->label_by_local = new_ids(R, base);
  out->label_by_local.index_copy_(0, order, labels.narrow(0, 0, R));
  out->seed_label = labels.narrow(0, R, S);
  out->frontier_bound = f.frontier();
  list_labels_ = std::move(out);
  return *list_labels_;
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor,
           c10::optional<torch::Tensor>>
Graph::GraphRelabel(torch::Tensor col_seeds, torch::Tensor row_ids) {
  CreateSparseFormat(kCOO);
  col_seeds = ids(col_seeds, "col_seeds");
  TORCH_CHECK(col_seeds.numel() > 0 || coo_->col.numel() == 0,
              "GraphRelabel: the matrix has edges but col_seeds is empty");
  if (use_list_labels(col_seeds, row_ids)) {
    ListLabels& l = list_labels_for(col_seeds, row_ids);
    // the gathers are queued before the host waits for the size of the frontier
    torch::Tensor out_row = l.label_by_local.index_select(0, coo_->row);
    torch::Tensor out_col = l.seed_label.index_select(0, coo_->col);
    return {l.frontier(), out_row, out_col, coo_->e_ids};
  }
  torch::Tensor rows = mapped_rows(coo_->row, row_ids);
  const int64_t E = rows.numel();
  torch::Tensor out_row = new_ids(E, rows), out_col = new_ids(E, rows);
  LabelRequest labels{cptr(coo_->col), nullptr, mptr(out_row), mptr(out_col)};
  Frontier& f = frontier_for(col_seeds, rows, {}, {}, &labels);
  if (!labels.done)
    GS_CALL(gs_unique_relabel(cptr(col_seeds), nullptr, col_seeds.numel(),
                              cptr(rows), nullptr, E, 1, cptr(coo_->col), nullptr,
                              mptr(out_row), mptr(out_col), 0,
                              f.workspace.data_ptr(), f.workspace.numel(),
                              cur_stream()));
  return {f.frontier(), out_row, out_col, coo_->e_ids};
}

torch::Tensor Graph::GetValidNodes(torch::Tensor col_seeds,
                                   torch::Tensor row_ids) {
  col_seeds = ids(col_seeds, "col_seeds");
  // The frontier order must be the one GraphRelabel produces, because the next
  // layer's seeds (all_nodes) have to line up with this layer's block sources
  // (to_dgl_block): both walk the COO rows.  (The reference reads csc.indices
  // here when a CSC exists, src/graph.cc:593-608, which is another edge order
  // whenever that CSC was built by sorting a row-sorted COO.)
  CreateSparseFormat(kCOO);
  if (use_list_labels(col_seeds, row_ids)) return list_labels_for(col_seeds, row_ids).frontier();
  const torch::Tensor& base = coo_->row;
  torch::Tensor rows = mapped_rows(base, row_ids);
  return frontier_for(col_seeds, rows, {}, {}).frontier();
}

}  // namespace gs
