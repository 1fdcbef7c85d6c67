// graph.h -- the `gs_classes.Graph` operator object: one sparse matrix held in
// up to three formats, plus the super-batch bookkeeping.  Method names,
// argument order and return shapes follow the reference's class
// (src/graph.h:11-232 of gSampler) because its Python layer and JIT address
// them by name and position; the bodies call the C ABI of gsampler_hip.h.
#ifndef GS_HOST_GRAPH_H_
#define GS_HOST_GRAPH_H_

#include <torch/custom_class.h>
#include <torch/script.h>

#include "abi_call.h"

#include <memory>
#include <string>
#include <tuple>
#include <vector>

namespace gs {

// Format bit flags (src/graph_storage.h:31-33).
constexpr int64_t kCOO = 1, kCSC = 2, kCSR = 4;

// CSC or CSR: `indptr` over the compressed ("major") axis, `indices` holds the
// ids on the other ("minor") axis.
struct Compressed {
  torch::Tensor indptr, indices;
  c10::optional<torch::Tensor> e_ids;
  // Exclusive bound of the ids in `indices` when it is known (a loaded or
  // converted matrix), else -1.
  int64_t num_minor = -1;
  // int32 copy of `indices` for the uniform sampler (half the bytes behind
  // every random pick); made on the first sampling call of a matrix in device
  // memory whose ids fit.
  mutable torch::Tensor indices32;
  mutable int64_t indices32_version = -1;  // version of `indices` the copy was made from
  mutable int64_t indices32_epoch = -1;    // and the cache epoch (invalidate_caches)
  mutable const void* indices32_source = nullptr;  // and its address
  const torch::Tensor& narrow_indices() const;
  // Call after assigning another `indices` or `indptr` to a matrix that was used.
  void forget_derived() {
    indices32 = torch::Tensor();
  }
};

struct Coordinate {
  torch::Tensor row, col;
  c10::optional<torch::Tensor> e_ids;
  bool row_sorted = false, col_sorted = false;
};

// Output of an operator that works along the compressed axis.
struct MajorResult {
  torch::Tensor indptr;     // [items + 1]
  torch::Tensor major_ids;  // local id on the compressed axis per edge (COO), may be undefined
  torch::Tensor minor_ids;  // id on the other axis per edge
  torch::Tensor select;     // position of the edge in the parent's `indices`
};

// Process-wide sampler state: every sampling call consumes one call id, so
// successive layers / epochs draw from disjoint Philox streams while a fixed
// seed reproduces a whole run.
struct RandomState {
  uint64_t seed = 7777;  // the reference's literal, src/cuda/sampling.cu:143
  uint64_t next_call = 0;
  int64_t algo = 0;      // GS_ALGO_AUTO
};
RandomState& random_state();

// Views of one mini-batch block: (row, col, indptr by destination -- absent for
// a mini-batch whose seeds repeat --, source ids, edge ids if the matrix carries
// any, number of source nodes, number of destination nodes).
using BlockViews = std::tuple<torch::Tensor, torch::Tensor, c10::optional<torch::Tensor>,
                              torch::Tensor, c10::optional<torch::Tensor>, int64_t, int64_t>;

// The same for every block of a layer, one list per field.
using BlockParts =
    std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>,
               std::vector<c10::optional<torch::Tensor>>, std::vector<torch::Tensor>,
               std::vector<c10::optional<torch::Tensor>>, std::vector<int64_t>,
               std::vector<int64_t>>;

// All blocks of one layer of a super-batched sampler (see blocks.cc).  The
// tensors are the layer's concatenated arrays; a block is a set of views.  The
// per-batch offsets reach the host on first use (they are already on their way
// when the object is handed out).
class BlockBatch : public torch::CustomClassHolder {
 public:
  torch::Tensor frontier, frontier_ptr, row, col, coo_ptr, col_bptr, col_seeds;
  torch::Tensor sampled_indptr;    // offsets of the sampled matrix over all its columns
  torch::Tensor indptr, distinct;  // per-block offsets and per-batch flags, made on first use
  c10::optional<torch::Tensor> e_ids;
  int64_t num_batches = 0, num_dst_total = 0;

  int64_t Size() { return num_batches; }
  // (source nodes, destination nodes, edges) over all blocks; no device read
  std::vector<int64_t> Totals();
  // host copies of (frontier_ptr, col_bptr, coo_ptr)
  std::tuple<std::vector<int64_t>, std::vector<int64_t>, std::vector<int64_t>> Offsets();
  BlockViews Block(int64_t b);
  BlockParts Blocks();
  int64_t NumSrcOf(int64_t b);
  torch::Tensor Frontier() { return frontier; }
  torch::Tensor FrontierPtr() { return frontier_ptr; }
  torch::Tensor Row() { return row; }
  torch::Tensor Col() { return col; }
  torch::Tensor Indptr() {
    fetch();
    return indptr;
  }
  torch::Tensor EdgePtr() { return coo_ptr; }
  torch::Tensor ColPtr() { return col_bptr; }
  c10::optional<torch::Tensor> EdgeIds() { return e_ids; }

 private:
  void fetch();
  bool have_host_ = false;
  std::vector<int64_t> f_off_, e_off_, c_off_;
  std::vector<uint8_t> grouped_;  // per batch: edges grouped by destination in offset order
};

class Graph;
using GraphPtr = c10::intrusive_ptr<Graph>;
using GraphAndIndex = std::tuple<GraphPtr, torch::Tensor>;

class Graph : public torch::CustomClassHolder {
 public:
  Graph(int64_t num_rows, int64_t num_cols)
      : num_rows_(num_rows), num_cols_(num_cols) {}

  // ---- loading and inspection
  void LoadCSC(torch::Tensor indptr, torch::Tensor indices);
  void LoadCOO(torch::Tensor row, torch::Tensor col, bool row_sorted,
               bool col_sorted);
  void LoadCSR(torch::Tensor indptr, torch::Tensor indices);
  int64_t GetNumRows() { return num_rows_; }
  int64_t GetNumCols() { return num_cols_; }
  int64_t GetNumEdges() { return num_edges_; }
  torch::Tensor GetCSCIndptr();
  torch::Tensor GetCSCIndices();
  torch::Tensor GetCSCEids();
  torch::Tensor GetCOORows();
  torch::Tensor GetCOOCols();
  torch::Tensor GetCOOEids();
  torch::Tensor GetCSRIndptr();
  torch::Tensor GetCSRIndices();
  torch::Tensor GetCSREids();
  void CreateSparseFormat(int64_t format);

  // ---- extract / select operators
  GraphAndIndex Slicing(torch::Tensor seeds, int64_t axis, int64_t on_format,
                        int64_t output_format);
  GraphAndIndex Sampling(int64_t axis, int64_t fanout, bool replace,
                         int64_t on_format, int64_t output_format);
  GraphAndIndex SamplingProbs(int64_t axis, torch::Tensor edge_probs,
                              int64_t fanout, bool replace, int64_t on_format,
                              int64_t output_format);
  // Not in the reference: column slice + weighted sampling in one step, on the
  // weights of this (unsliced) matrix.  What gs.jit.compile turns
  // Slicing -> SamplingProbs into; draws go through a persistent CDF of the
  // weights that is built on first use and kept while the same tensor comes in.
  GraphAndIndex FusedSlicingSamplingProbs(int64_t axis, torch::Tensor seeds,
                                          torch::Tensor edge_probs, int64_t fanout,
                                          bool replace, int64_t on_format,
                                          int64_t output_format);
  GraphAndIndex FusedSlicingSampling(int64_t axis, torch::Tensor seeds,
                                     int64_t fanout, bool replace,
                                     int64_t on_format, int64_t output_format);
  // Not in the reference: operators that read the column slice A[:, cols]
  // straight from this matrix instead of from a written slice (fused_slices.cc).
  // out[row] += sum of efeat^2 over the edges of A[:, cols];
  void SlicedESquareSum(torch::Tensor cols, torch::Tensor efeat, torch::Tensor out);
  // A[rows, cols], the edge index addressing this matrix's edges.
  GraphAndIndex ColRowSlicing(torch::Tensor cols, torch::Tensor rows, int64_t on_format,
                              int64_t output_format);
  GraphAndIndex Compact(int64_t axis);
  torch::Tensor RandomWalk(torch::Tensor seeds, int64_t walk_length);
  torch::Tensor Node2Vec(torch::Tensor seeds, int64_t walk_length, double p,
                         double q);
  void SortCSCIndices();

  // ---- compute operators
  void SDDMM(const std::string& op, torch::Tensor lhs, torch::Tensor rhs,
             torch::Tensor out, int64_t lhs_target, int64_t rhs_target,
             int64_t on_format);
  void SpMM(const std::string& op, const std::string& reduce,
            torch::Tensor ufeat, torch::Tensor efeat, torch::Tensor out,
            torch::Tensor argu, torch::Tensor arge, int64_t u_target,
            int64_t on_format);
  void FusedUOPV(const std::string& op, torch::Tensor lhs1, torch::Tensor rhs1,
                 torch::Tensor out1, torch::Tensor lhs2, torch::Tensor rhs2,
                 torch::Tensor out2, int64_t on_format);
  void FusedESquareSum(const std::string& op, const std::string& reduce,
                       torch::Tensor ufeat, torch::Tensor efeat,
                       torch::Tensor out, torch::Tensor argu,
                       torch::Tensor arge, int64_t u_target, int64_t on_format);
  void FusedEDivUSum(const std::string& op, const std::string& reduce,
                     torch::Tensor ufeat, torch::Tensor efeat,
                     torch::Tensor out, torch::Tensor argu, torch::Tensor arge,
                     int64_t u_target, int64_t on_format);

  // ---- finalize operators
  std::tuple<torch::Tensor, torch::Tensor, torch::Tensor,
             c10::optional<torch::Tensor>>
  GraphRelabel(torch::Tensor col_seeds, torch::Tensor row_ids);
  torch::Tensor GetValidNodes(torch::Tensor col_seeds, torch::Tensor row_ids);

  // ---- super-batch interface
  void SetEdgeBptr(torch::Tensor p) { edge_bptr_ = p; }
  void SetColBptr(torch::Tensor p) { col_bptr_ = p; }
  void SetRowBptr(torch::Tensor p) { row_bptr_ = p; }
  void SetOrigRowIds(torch::Tensor t) { orig_row_ids_ = t; }
  void SetOrigColIds(torch::Tensor t) { orig_col_ids_ = t; }
  torch::Tensor GetEdgeBptr() { return edge_bptr_; }
  torch::Tensor GetColBptr() { return col_bptr_; }
  torch::Tensor GetRowBptr() { return row_bptr_; }
  std::tuple<torch::Tensor, torch::Tensor> BatchGetRows() {
    return {orig_row_ids_, row_bptr_};
  }
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCols() {
    return {orig_col_ids_, col_bptr_};
  }
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCSCIndptr();
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCSCIndices();
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCSCEids();
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCOORows();
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCOOCols();
  std::tuple<torch::Tensor, torch::Tensor> BatchGetCOOEids();
  std::vector<int64_t> BatchGetColCounts();
  GraphAndIndex BatchColSlicing(torch::Tensor seeds, torch::Tensor col_bptr,
                                bool encoding);
  GraphAndIndex BatchColRowSlcing(torch::Tensor col, torch::Tensor col_bptr,
                                  torch::Tensor row, torch::Tensor row_bptr);
  GraphAndIndex BatchRowSlicing(torch::Tensor row_ids, torch::Tensor row_bptr);
  GraphAndIndex BatchRowSampling(int64_t fanout, bool replace);
  GraphAndIndex BatchRowSamplingProbs(int64_t fanout, bool replace,
                                      torch::Tensor edge_probs);
  GraphAndIndex BatchFusedSlicingSamplingProbs(torch::Tensor seeds,
                                               torch::Tensor col_bptr,
                                               torch::Tensor edge_probs,
                                               int64_t fanout, bool replace);
  GraphAndIndex BatchFusedSlicingSampling(torch::Tensor seeds,
                                          torch::Tensor col_bptr,
                                          int64_t fanout, bool replace);
  std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
             c10::optional<torch::Tensor>, torch::Tensor>
  BatchGraphRelabel(torch::Tensor col_seeds, torch::Tensor row_ids);
  std::tuple<torch::Tensor, torch::Tensor> BatchGetValidNodes(
      torch::Tensor col_seeds, torch::Tensor row_ids);
  // Not in the reference: relabel + all mini-batch blocks of the layer (edge
  // list and compressed form) in one call; see blocks.cc.
  c10::intrusive_ptr<BlockBatch> BatchBlocks(torch::Tensor col_seeds, torch::Tensor row_ids);

 private:
  // Unique/relabel state shared by all_nodes() and to_dgl_block(): the
  // frontier is computed once, the relabel pass reuses the hash tables.
  struct Frontier {
    torch::Tensor seeds, rows, seeds_ptr, rows_ptr;  // the keys it was built from
    int64_t seeds_version = -1, rows_version = -1, epoch = -1;
    torch::Tensor workspace, unique_ptr;
    int64_t num_batches = 0;
    // The unique keys: filled into a buffer sized by the upper bound, trimmed
    // once the count has arrived (frontier() waits for it).
    torch::Tensor unique_buffer;
    int64_t total() { return OffsetMirror::values(unique_ptr).back(); }
    const torch::Tensor& frontier() {
      if (!unique_.defined()) unique_ = unique_buffer.narrow(0, 0, total());
      return unique_;
    }
    bool matches(const torch::Tensor& s, const torch::Tensor& r,
                 const torch::Tensor& sp, const torch::Tensor& rp) const;

   private:
    torch::Tensor unique_;
  };
  // Labels wanted together with a frontier: when the frontier has to be built,
  // both come from one launch and `done` is set; a frontier that is already there
  // leaves `done` false and the caller labels on its own.
  struct LabelRequest {
    const int64_t* edge_col = nullptr;
    const int64_t* col_indptr = nullptr;
    int64_t* out_row = nullptr;
    int64_t* out_col = nullptr;
    bool col_prefilled = false;  // out_col holds the samplers' column labels
    bool done = false;
  };
  Frontier& frontier_for(const torch::Tensor& seeds, const torch::Tensor& rows,
                         const torch::Tensor& seeds_ptr,
                         const torch::Tensor& rows_ptr, LabelRequest* labels = nullptr);
  Frontier& batch_relabel_launch(torch::Tensor& col_seeds, const torch::Tensor& row_ids,
                                 torch::Tensor* out_row, torch::Tensor* out_col,
                                 c10::optional<torch::Tensor>* e_ids);

  const Compressed& compressed(int64_t format);
  // Offsets and size of the column slice A[:, cols], kept for the next operator
  // that is handed the same tensor of columns.
  struct SliceOffsets {
    torch::Tensor cols, sub_indptr;
    int64_t version = -1, indptr_version = -1, epoch = -1, nnz = 0;
    MajorResult written;  // the slice itself, when an operator had to write it
  };
  std::unique_ptr<SliceOffsets> slice_offsets_;
  const SliceOffsets& slice_offsets_for(const torch::Tensor& cols);
  static bool read_in_place(int64_t slice_nnz, int64_t num_cols_picked);
  const MajorResult& written_slice(const torch::Tensor& cols);
  // CDF of edge_probs in the edge order of `format` (cached per weights tensor).
  torch::Tensor weight_cdf_for(const torch::Tensor& edge_probs, int64_t format);
  void check_reduce_operands(const std::string& op, const torch::Tensor& ufeat,
                             const torch::Tensor& efeat, const torch::Tensor& out,
                             int64_t u_target, const char* who) const;
  bool csc_sorted_ = false;  // row ids known to be sorted inside every column
  torch::Tensor cdf_, cdf_probs_;
  int64_t cdf_version_ = -1, cdf_format_ = 0, cdf_epoch_ = -1;
  torch::Tensor mapped_rows(const torch::Tensor& base, const torch::Tensor& row_ids);
  GraphAndIndex slice_coo(const torch::Tensor& seeds, int64_t axis,
                          int64_t new_rows, int64_t new_cols);
  GraphPtr derive(int64_t on_format, int64_t output_format,
                  const MajorResult& r, int64_t new_rows, int64_t new_cols);
  torch::Tensor edge_index(const c10::optional<torch::Tensor>& parent_eids,
                           const torch::Tensor& select);
  void copy_batch_state_to(Graph& g, bool with_rows);
  // The edges in column order, for the relabel pass: their row ids and either
  // the column of every edge or the column pointer that implies it.
  struct ColumnOrderedEdges {
    torch::Tensor row;
    torch::Tensor col;         // undefined when col_indptr is given
    torch::Tensor col_indptr;  // undefined when col is given
    c10::optional<torch::Tensor> e_ids;
  };
  ColumnOrderedEdges column_ordered_edges(const char* who);
  torch::Tensor batch_rows_for_relabel(const torch::Tensor& edge_rows,
                                       const torch::Tensor& row_ids);

  int64_t num_rows_ = 0, num_cols_ = 0, num_edges_ = 0;
  std::shared_ptr<Compressed> csc_, csr_;
  std::shared_ptr<Coordinate> coo_;
  torch::Tensor col_bptr_, row_bptr_, edge_bptr_;
  // per edge, the place of its column inside its batch, as the super-batched
  // samplers write it (see EdgeCount::Hint); undefined for any other matrix
  torch::Tensor col_labels_;
  torch::Tensor orig_row_ids_, orig_col_ids_;
  int64_t row_encoding_size_ = 0;
  std::unique_ptr<Frontier> frontier_;
  torch::Tensor mapped_out_, mapped_from_, mapped_by_;
  // Relabel of a matrix whose rows are positions in a short list of ids
  // (row slicing leaves it that way): label of every list entry and of every
  // seed, computed from the list instead of from every edge.
  struct ListLabels {
    torch::Tensor base, row_ids, seeds;
    int64_t row_ids_version = -1, seeds_version = -1, epoch = -1;
    torch::Tensor label_by_local, seed_label;
    // The unique keys sit at the front of a buffer sized by the bound; how many
    // there are may still be on its way from the device.
    torch::Tensor frontier_bound;
    AsyncCount frontier_count;
    bool counted = false;
    const torch::Tensor& frontier() {
      if (!counted) {
        if (frontier_count.requested())
          frontier_bound = frontier_bound.narrow(0, 0, frontier_count.get());
        counted = true;
      }
      return frontier_bound;
    }
  };
  std::unique_ptr<ListLabels> list_labels_;
  bool use_list_labels(const torch::Tensor& col_seeds, const torch::Tensor& row_ids) const;
  ListLabels& list_labels_for(const torch::Tensor& col_seeds, const torch::Tensor& row_ids);
};

// Operators along the compressed axis (graph.cc) and across it (slicing.cc).
MajorResult major_slice(const Compressed& m, const torch::Tensor& picked,
                        bool with_coo, const torch::Tensor& batch_ptr,
                        int64_t encode_stride);
MajorResult major_sample_uniform(const Compressed& m, const torch::Tensor& picked,
                                 int64_t fanout, bool replace, bool with_coo);
MajorResult minor_slice(const Compressed& m, const torch::Tensor& picked,
                        bool with_coo);
// First n entries of a buffer sized by an upper bound: a view, or a copy when
// the view would pin a large buffer for a small result.
torch::Tensor trim_to(const torch::Tensor& buffer, int64_t n);

// ---- free operators (gs_ops)
torch::Tensor GatherRows(torch::Tensor table, torch::Tensor ids);
torch::Tensor ListSampling(int64_t num_items, int64_t num_picks, bool replace);
torch::Tensor ListSamplingProbs(torch::Tensor probs, int64_t num_picks,
                                bool replace);
std::tuple<torch::Tensor, torch::Tensor> BatchListSamplingProbs(
    torch::Tensor probs, int64_t num_picks, bool replace, torch::Tensor range);
std::tuple<torch::Tensor, torch::Tensor> BatchListSampling(
    int64_t num_picks, bool replace, torch::Tensor range);
std::vector<torch::Tensor> SplitByOffset(torch::Tensor data,
                                         torch::Tensor offset);
std::vector<torch::Tensor> SplitIndptrByOffset(torch::Tensor indptr,
                                               torch::Tensor offset);

}  // namespace gs

#endif  // GS_HOST_GRAPH_H_
