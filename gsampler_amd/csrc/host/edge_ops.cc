// edge_ops.cc -- compute-step operators of gs_classes.Graph: SDDMM, SpMM and
// the fusions used by layer-wise samplers.  The host side resolves operator
// names, broadcast shapes and the sparse format, then calls the C ABI.
#include <algorithm>

#include "abi_call.h"
#include "graph.h"

namespace gs {
namespace {

int op_code(const std::string& op) {
  static const char* names[] = {"add", "sub", "mul", "div", "copy_lhs", "copy_rhs", "dot"};
  for (int i = 0; i < 7; ++i)
    if (op == names[i]) return i;
  TORCH_CHECK(false, "unsupported binary operator '", op, "'");
}

int reduce_code(const std::string& r) {
  if (r == "sum") return GS_REDUCE_SUM;
  if (r == "max") return GS_REDUCE_MAX;
  if (r == "min") return GS_REDUCE_MIN;
  TORCH_CHECK(false, "unsupported reducer '", r, "'");
}

// Broadcast bookkeeping between two feature tensors [n, d1, d2, ...]:
// flattened feature lengths, output length, the reduce length of `dot`, and --
// only when the trailing shapes differ -- for every output feature position
// the position to read in each operand (NumPy broadcasting from the last axis).
// Same contract as CalcBcastOff, src/bcast.cc:24-76 of the reference.
struct Broadcast {
  int64_t lhs_len = 1, rhs_len = 1, out_len = 1, reduce_size = 1;
  torch::Tensor lhs_off, rhs_off;  // device int64[out_len] or undefined
};

Broadcast make_broadcast(const std::string& op, const torch::Tensor& lhs,
                         const torch::Tensor& rhs, const torch::Tensor& device_like) {
  Broadcast bc;
  const bool use_l = op != "copy_rhs" && lhs.defined();
  const bool use_r = op != "copy_lhs" && rhs.defined();
  if (use_l)
    for (int64_t i = 1; i < lhs.dim(); ++i) bc.lhs_len *= lhs.size(i);
  if (use_r)
    for (int64_t i = 1; i < rhs.dim(); ++i) bc.rhs_len *= rhs.size(i);
  bool differ = false;
  if (use_l && use_r) {
    differ = lhs.dim() != rhs.dim();
    for (int64_t i = 1; !differ && i < lhs.dim(); ++i)
      differ = lhs.size(i) != rhs.size(i);
  }
  if (op == "dot") {
    TORCH_CHECK(use_l && use_r && lhs.dim() >= 2 && rhs.dim() >= 2 &&
                    lhs.size(-1) == rhs.size(-1),
                "dot needs operands with equal last dimensions");
    bc.reduce_size = lhs.size(-1);
  }
  if (!differ) {
    bc.out_len = (use_l ? bc.lhs_len : bc.rhs_len) / bc.reduce_size;
    return bc;
  }
  // Feature axes from the last one (skipping the reduce axis of dot) forward.
  std::vector<int64_t> loff{0}, roff{0};
  const int64_t ndim = std::max(lhs.dim(), rhs.dim()) - 1;
  int64_t out_len = 1, stride_l = 1, stride_r = 1;
  for (int64_t j = (op == "dot" ? 1 : 0); j < ndim; ++j) {
    const int64_t dl = lhs.dim() - 1 - j < 1 ? 1 : lhs.size(lhs.dim() - 1 - j);
    const int64_t dr = rhs.dim() - 1 - j < 1 ? 1 : rhs.size(rhs.dim() - 1 - j);
    TORCH_CHECK(dl == dr || dl == 1 || dr == 1, "feature shapes do not broadcast");
    const int64_t d = std::max(dl, dr);
    for (int64_t i = 1; i < d; ++i)
      for (int64_t k = 0; k < out_len; ++k) {
        loff.push_back(loff[k] + (i < dl ? i * stride_l : 0));
        roff.push_back(roff[k] + (i < dr ? i * stride_r : 0));
      }
    out_len *= d;
    stride_l *= dl;
    stride_r *= dr;
  }
  bc.out_len = out_len;
  auto opts = torch::TensorOptions().dtype(torch::kInt64);
  bc.lhs_off = torch::from_blob(loff.data(), {(int64_t)loff.size()}, opts)
                   .to(device_like.device());
  bc.rhs_off = torch::from_blob(roff.data(), {(int64_t)roff.size()}, opts)
                   .to(device_like.device());
  return bc;
}

const void* fptr(const torch::Tensor& t) {
  return (t.defined() && t.numel() > 0) ? t.data_ptr() : nullptr;
}

torch::Tensor feat(const torch::Tensor& t, const char* name) {
  if (!t.defined()) return t;
  TORCH_CHECK(t.is_cuda(), name, " must live on the GPU");
  return t.contiguous();
}

// An operand indexed by row ids, edge ids or column ids must have a row for
// every one of them: a shorter tensor would be read out of bounds on the GPU
// (the reference does not check, src/graph.cc:320-379).
void need_rows(const torch::Tensor& t, int64_t rows, const char* who, const char* name) {
  if (!t.defined()) return;
  TORCH_CHECK(t.dim() >= 1 && t.size(0) >= rows, who, ": ", name, " has ",
              t.dim() >= 1 ? t.size(0) : 0, " rows, the matrix needs ", rows);
}

void same_dtype(const torch::Tensor& t, const torch::Tensor& out, const char* who,
                const char* name) {
  if (!t.defined()) return;
  TORCH_CHECK(t.scalar_type() == out.scalar_type(), who, ": ", name, " is ",
              t.scalar_type(), " but out is ", out.scalar_type());
}

int dtype_code(const torch::Tensor& t) {
  if (t.scalar_type() == torch::kFloat32) return GS_F32;
  if (t.scalar_type() == torch::kFloat64) return GS_F64;
  TORCH_CHECK(false, "edge operators need float32 or float64 features, got ",
              t.scalar_type());
}

}  // namespace

// The structure arrays of `format` in the ABI's (format, a, b, num_major, nnz,
// edge_map) form.
struct StructureArgs {
  int format;
  const int64_t *a, *b, *edge_map;
  int64_t num_major, nnz;
};

static StructureArgs structure_of(const Compressed& m) {
  return {GS_FMT_COMPRESSED, cptr(m.indptr), cptr(m.indices),
          m.e_ids.has_value() ? cptr(m.e_ids.value()) : nullptr,
          m.indptr.numel() - 1, m.indices.numel()};
}

static StructureArgs structure_of(const Coordinate& c) {
  return {GS_FMT_COO, cptr(c.row), cptr(c.col),
          c.e_ids.has_value() ? cptr(c.e_ids.value()) : nullptr, 0,
          c.row.numel()};
}

void Graph::SDDMM(const std::string& op, torch::Tensor lhs, torch::Tensor rhs,
                  torch::Tensor out, int64_t lhs_target, int64_t rhs_target,
                  int64_t on_format) {
  if (num_edges_ <= 0) return;
  TORCH_CHECK(on_format == kCOO || on_format == kCSC || on_format == kCSR,
              "SDDMM only supports CSC, CSR and COO formats");
  CreateSparseFormat(on_format);
  lhs = feat(lhs, "lhs");
  rhs = feat(rhs, "rhs");
  TORCH_CHECK(out.defined() && out.is_cuda() && out.is_contiguous(),
              "SDDMM: out must be a contiguous GPU tensor");
  const int64_t per_target[3] = {num_rows_, num_edges_, num_cols_};
  TORCH_CHECK(lhs_target >= 0 && lhs_target <= 2 && rhs_target >= 0 && rhs_target <= 2,
              "SDDMM: targets must be 0 (u), 1 (e) or 2 (v)");
  if (op != "copy_rhs") need_rows(lhs, per_target[lhs_target], "SDDMM", "lhs");
  if (op != "copy_lhs") need_rows(rhs, per_target[rhs_target], "SDDMM", "rhs");
  need_rows(out, num_edges_, "SDDMM", "out");
  same_dtype(lhs, out, "SDDMM", "lhs");
  same_dtype(rhs, out, "SDDMM", "rhs");
  const Broadcast bc = make_broadcast(op, lhs, rhs, out);
  TORCH_CHECK(out.numel() >= num_edges_ * bc.out_len, "SDDMM: out holds ", out.numel(),
              " values, ", num_edges_ * bc.out_len, " are written");
  if (on_format == kCSR) {  // rows are the compressed axis: swap u and v
    lhs_target = lhs_target == 1 ? 1 : 2 - lhs_target;
    rhs_target = rhs_target == 1 ? 1 : 2 - rhs_target;
  }
  const StructureArgs s = on_format == kCOO ? structure_of(*coo_)
                                            : structure_of(compressed(on_format));
  GS_CALL(gs_sddmm(s.format, s.a, s.b, s.num_major, s.nnz, s.edge_map,
                   op_code(op), dtype_code(out), fptr(lhs), fptr(rhs),
                   out.data_ptr(), (int)lhs_target, (int)rhs_target, bc.lhs_len,
                   bc.rhs_len, bc.out_len, bc.reduce_size, cptr(bc.lhs_off),
                   cptr(bc.rhs_off), cur_stream()));
}

void Graph::FusedUOPV(const std::string& op, torch::Tensor lhs1,
                      torch::Tensor rhs1, torch::Tensor out1, torch::Tensor lhs2,
                      torch::Tensor rhs2, torch::Tensor out2, int64_t on_format) {
  TORCH_CHECK(on_format == kCOO || on_format == kCSC,
              "fused SDDMM only supports CSC and COO formats");
  CreateSparseFormat(on_format);
  lhs1 = feat(lhs1, "lhs1"), rhs1 = feat(rhs1, "rhs1");
  lhs2 = feat(lhs2, "lhs2"), rhs2 = feat(rhs2, "rhs2");
  TORCH_CHECK(lhs1.sizes() == lhs2.sizes() && rhs1.sizes() == rhs2.sizes(),
              "FusedUOPV: the two operand pairs must have equal shapes");
  TORCH_CHECK(out1.defined() && out2.defined() && out1.is_cuda() && out2.is_cuda() &&
                  out1.is_contiguous() && out2.is_contiguous() &&
                  out1.scalar_type() == out2.scalar_type(),
              "FusedUOPV: outputs must be contiguous GPU tensors of one type");
  need_rows(lhs1, num_rows_, "FusedUOPV", "lhs");
  need_rows(rhs1, num_cols_, "FusedUOPV", "rhs");
  same_dtype(lhs1, out1, "FusedUOPV", "lhs1");
  same_dtype(rhs1, out1, "FusedUOPV", "rhs1");
  same_dtype(lhs2, out1, "FusedUOPV", "lhs2");
  same_dtype(rhs2, out1, "FusedUOPV", "rhs2");
  const Broadcast bc = make_broadcast(op, lhs1, rhs1, out1);
  TORCH_CHECK(out1.numel() >= num_edges_ * bc.out_len && out2.numel() >= num_edges_ * bc.out_len,
              "FusedUOPV: outputs are too small for ", num_edges_, " edges");
  const StructureArgs s = on_format == kCOO ? structure_of(*coo_)
                                            : structure_of(compressed(kCSC));
  GS_CALL(gs_fused_u_op_v(s.format, s.a, s.b, s.num_major, s.nnz, s.edge_map, op_code(op),
                          dtype_code(out1), fptr(lhs1), fptr(rhs1),
                          out1.data_ptr(), fptr(lhs2), fptr(rhs2),
                          out2.data_ptr(), bc.lhs_len, bc.rhs_len, bc.out_len,
                          bc.reduce_size, cptr(bc.lhs_off), cptr(bc.rhs_off),
                          cur_stream()));
}

// Which structure an SpMM-like reduction runs on: COO with an explicit
// direction, or the compressed format whose segments are the reduce targets.
static StructureArgs reduce_structure(Graph& g, const Coordinate* coo,
                                      const Compressed* csx, int64_t on_format,
                                      int64_t u_target, const char* who) {
  TORCH_CHECK(u_target == 0 || u_target == 2, who, ": invalid u_target ", u_target);
  if (on_format == kCOO) return structure_of(*coo);
  TORCH_CHECK((on_format == kCSR && u_target == 2) ||
                  (on_format == kCSC && u_target == 0),
              who, ": format ", on_format, " does not match u_target ", u_target);
  (void)g;
  return structure_of(*csx);
}

// Scratch for the per-die accumulators of a coordinate-form sum (1 byte when
// the reduction does not use them).
static torch::Tensor reduce_workspace(const StructureArgs& s,
                                      const torch::Tensor& out) {
  return new_workspace(gs_spmm_workspace_bytes(s.format, s.nnz, out.size(0)), out);
}

// Shapes and types of a reduction's operands: u features per source node,
// e features per edge, one output row per target node, all float32.
void Graph::check_reduce_operands(const std::string& op, const torch::Tensor& ufeat,
                                  const torch::Tensor& efeat, const torch::Tensor& out,
                                  int64_t u_target, const char* who) const {
  TORCH_CHECK(u_target == 0 || u_target == 2, who, ": invalid u_target ", u_target);
  TORCH_CHECK(out.defined() && out.is_cuda() && out.is_contiguous() && out.dim() >= 1 &&
                  out.scalar_type() == torch::kFloat32,
              who, ": out must be a contiguous float32 GPU tensor");
  if (op != "copy_rhs") need_rows(ufeat, u_target == 0 ? num_rows_ : num_cols_, who, "ufeat");
  if (op != "copy_lhs") need_rows(efeat, num_edges_, who, "efeat");
  need_rows(out, u_target == 0 ? num_cols_ : num_rows_, who, "out");
  same_dtype(ufeat, out, who, "ufeat");
  same_dtype(efeat, out, who, "efeat");
}

void Graph::SpMM(const std::string& op, const std::string& reduce,
                 torch::Tensor ufeat, torch::Tensor efeat, torch::Tensor out,
                 torch::Tensor argu, torch::Tensor arge, int64_t u_target,
                 int64_t on_format) {
  if (num_edges_ <= 0) return;
  TORCH_CHECK(on_format == kCOO || on_format == kCSC || on_format == kCSR,
              "SpMM only supports CSC, CSR and COO formats");
  CreateSparseFormat(on_format);
  ufeat = feat(ufeat, "ufeat");
  efeat = feat(efeat, "efeat");
  TORCH_CHECK(out.defined() && out.is_cuda() && out.is_contiguous() &&
                  out.scalar_type() == torch::kFloat32,
              "SpMM: out must be a contiguous float32 GPU tensor");
  check_reduce_operands(op, ufeat, efeat, out, u_target, "SpMM");
  const Broadcast bc = make_broadcast(op, ufeat, efeat, out);
  TORCH_CHECK(out.numel() >= out.size(0) * bc.out_len, "SpMM: out is too small");
  for (const torch::Tensor* arg : {&argu, &arge})
    TORCH_CHECK(!arg->defined() || arg->numel() == 0 ||
                    (arg->is_cuda() && arg->scalar_type() == torch::kInt64 &&
                     arg->numel() >= out.size(0) * bc.out_len),
                "SpMM: arg tensors must be int64 GPU tensors as large as out");
  const StructureArgs s = reduce_structure(
      *this, coo_.get(), on_format == kCOO ? nullptr : &compressed(on_format),
      on_format, u_target, "SpMM");
  torch::Tensor ws = reduce_workspace(s, out);
  GS_CALL(gs_spmm(s.format, s.a, s.b, s.num_major, s.nnz, s.edge_map,
                  op_code(op), reduce_code(reduce), (const float*)fptr(ufeat),
                  (const float*)fptr(efeat), (float*)out.data_ptr(),
                  argu.defined() ? mptr(argu) : nullptr,
                  arge.defined() ? mptr(arge) : nullptr, (int)u_target,
                  bc.lhs_len, bc.rhs_len, bc.out_len, cptr(bc.lhs_off),
                  cptr(bc.rhs_off), out.size(0), ws.data_ptr(), (size_t)ws.numel(),
                  cur_stream()));
}

void Graph::FusedESquareSum(const std::string& op, const std::string& reduce,
                            torch::Tensor ufeat, torch::Tensor efeat,
                            torch::Tensor out, torch::Tensor argu,
                            torch::Tensor arge, int64_t u_target,
                            int64_t on_format) {
  if (num_edges_ <= 0) return;
  TORCH_CHECK(reduce == "sum", "FusedESquareSum only sums");
  CreateSparseFormat(on_format);
  efeat = feat(efeat, "efeat");
  TORCH_CHECK(efeat.scalar_type() == torch::kFloat32 &&
                  out.scalar_type() == torch::kFloat32,
              "FusedESquareSum needs float32 tensors");
  check_reduce_operands("copy_rhs", torch::Tensor(), efeat, out, u_target, "FusedESquareSum");
  int64_t len = 1;
  for (int64_t i = 1; i < efeat.dim(); ++i) len *= efeat.size(i);
  TORCH_CHECK(out.numel() >= out.size(0) * len, "FusedESquareSum: out is too small");
  const StructureArgs s = reduce_structure(
      *this, coo_.get(), on_format == kCOO ? nullptr : &compressed(on_format),
      on_format, u_target, "FusedESquareSum");
  torch::Tensor ws = reduce_workspace(s, out);
  GS_CALL(gs_e_square_sum(s.format, s.a, s.b, s.num_major, s.nnz, s.edge_map,
                          (const float*)fptr(efeat), (float*)out.data_ptr(),
                          (int)u_target, len, out.size(0), ws.data_ptr(),
                          (size_t)ws.numel(), cur_stream()));
}

void Graph::FusedEDivUSum(const std::string& op, const std::string& reduce,
                          torch::Tensor ufeat, torch::Tensor efeat,
                          torch::Tensor out, torch::Tensor argu,
                          torch::Tensor arge, int64_t u_target,
                          int64_t on_format) {
  if (num_edges_ <= 0) return;
  TORCH_CHECK(reduce == "sum", "FusedEDivUSum only sums");
  CreateSparseFormat(on_format);
  ufeat = feat(ufeat, "ufeat");
  efeat = feat(efeat, "efeat");
  TORCH_CHECK(efeat.scalar_type() == torch::kFloat32 &&
                  ufeat.scalar_type() == torch::kFloat32 &&
                  out.scalar_type() == torch::kFloat32,
              "FusedEDivUSum needs float32 tensors");
  check_reduce_operands("div", ufeat, efeat, out, u_target, "FusedEDivUSum");
  int64_t len = 1;
  for (int64_t i = 1; i < efeat.dim(); ++i) len *= efeat.size(i);
  TORCH_CHECK(ufeat.numel() / std::max<int64_t>(ufeat.size(0), 1) == len,
              "FusedEDivUSum: ufeat and efeat must have the same feature length");
  TORCH_CHECK(out.numel() >= out.size(0) * len, "FusedEDivUSum: out is too small");
  const StructureArgs s = reduce_structure(
      *this, coo_.get(), on_format == kCOO ? nullptr : &compressed(on_format),
      on_format, u_target, "FusedEDivUSum");
  torch::Tensor ws = reduce_workspace(s, out);
  GS_CALL(gs_e_div_u_sum(s.format, s.a, s.b, s.num_major, s.nnz, s.edge_map,
                         (const float*)fptr(ufeat), (const float*)fptr(efeat),
                         (float*)out.data_ptr(), (int)u_target, len, out.size(0),
                         ws.data_ptr(), (size_t)ws.numel(), cur_stream()));
}

}  // namespace gs
