// membership.hip -- slicing across the compressed axis: keep the edges whose
// minor id (row id of a CSC, or any id array of a COO) belongs to a picked set
// and relabel that id to its position in the set.
//
//   count: hash the picked ids (smallest position wins for repeated ids), flag
//          every edge, exclusive-scan the flags; out_indptr[c] =
//          prefix[indptr[c]] needs no per-column pass.
//   fill : kept edge e goes to position prefix[e], edge order preserved.
#include "common.h"
#include "hashtable.h"
#include "scan.h"

namespace gs {

struct MemberWs {
  uint64_t* table;  // [2 * num_picked + 2]
  int64_t* prefix;  // [nnz + 1]
  void* scan_ws;
  size_t scan_ws_bytes;
  size_t total;
};

static MemberWs carve_member(void* ws, int64_t nnz, int64_t num_picked) {
  Carver c(ws);
  MemberWs w;
  w.table = c.take<uint64_t>((size_t)(2 * num_picked + 2));
  w.prefix = c.take<int64_t>((size_t)nnz + 1);
  w.scan_ws_bytes = scan_workspace_bytes(nnz + 1);
  w.scan_ws = c.take<char>(w.scan_ws_bytes);
  w.total = c.total();
  return w;
}

__global__ __launch_bounds__(kBlock) void member_insert_kernel(
    const int64_t* __restrict__ picked, int64_t n, uint64_t* table, uint64_t cap) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const uint64_t key = (uint64_t)picked[i];
  if (key > kMaxPackedKey) return;  // cannot equal any admissible id
  table_insert_min(table, cap, key, (uint64_t)i);
}

__global__ __launch_bounds__(kBlock) void member_flag_kernel(
    const int64_t* __restrict__ ids, int64_t nnz,
    const uint64_t* __restrict__ table, uint64_t cap,
    int64_t* __restrict__ flags) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e > nnz) return;
  int64_t f = 0;
  if (e < nnz) {
    const uint64_t key = (uint64_t)ids[e];
    f = (key <= kMaxPackedKey && table_find(table, cap, key) < cap) ? 1 : 0;
  }
  flags[e] = f;  // flags[nnz] = 0 so that the scan leaves the total there
}

__global__ __launch_bounds__(kBlock) void member_indptr_kernel(
    const int64_t* __restrict__ indptr, int64_t num_major,
    const int64_t* __restrict__ prefix, int64_t nnz,
    int64_t* __restrict__ out_indptr, int64_t* __restrict__ out_total) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c == 0 && out_total) *out_total = prefix[nnz];
  if (indptr == nullptr || c > num_major) return;
  out_indptr[c] = prefix[indptr[c]];
}

__global__ __launch_bounds__(kBlock) void member_fill_kernel(
    const int64_t* __restrict__ ids, int64_t nnz,
    const uint64_t* __restrict__ table, uint64_t cap,
    const int64_t* __restrict__ prefix, const int64_t* __restrict__ indptr,
    int64_t num_major, const int64_t* __restrict__ edge_major,
    int64_t* __restrict__ out_major, int64_t* __restrict__ out_minor,
    int64_t* __restrict__ out_select) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= nnz) return;
  const int64_t pos = prefix[e];
  if (prefix[e + 1] == pos) return;
  const uint64_t key = (uint64_t)ids[e];
  out_minor[pos] = (int64_t)(uint32_t)table[table_find(table, cap, key)];
  out_select[pos] = e;
  if (out_major)
    out_major[pos] = edge_major ? edge_major[e] : segment_of(indptr, num_major, e);
}

}  // namespace gs

extern "C" {

size_t gs_minor_slice_workspace_bytes(int64_t nnz, int64_t num_picked) {
  if (nnz < 0 || num_picked < 0) return 0;
  return gs::carve_member(nullptr, nnz, num_picked).total;
}

int gs_minor_slice_count(const int64_t* ids, int64_t nnz, const int64_t* picked,
                         int64_t num_picked, const int64_t* indptr,
                         int64_t num_major, int64_t* out_indptr,
                         int64_t* out_total, void* workspace,
                         size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_picked >= 0 && num_major >= 0,
             "minor_slice_count: negative size");
  GS_REQUIRE((nnz == 0 || ids) && (num_picked == 0 || picked),
             "minor_slice_count: null pointer");
  GS_REQUIRE((indptr == nullptr) == (out_indptr == nullptr),
             "minor_slice_count: indptr and out_indptr go together");
  GS_REQUIRE(out_indptr || out_total, "minor_slice_count: nothing to write");
  GS_REQUIRE(num_picked <= (int64_t)kMaxPackedKey,
             "minor_slice_count: too many picked ids");
  MemberWs w = carve_member(workspace, nnz, num_picked);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("minor_slice workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  const uint64_t cap = (uint64_t)(2 * num_picked + 2);
  GS_LAUNCH("member_clear", s,
            table_fill_kernel<><<<dim3((unsigned)ceil_div((int64_t)cap, kBlock * 4)),
                                  dim3(kBlock), 0, s>>>(w.table, (int64_t)cap,
                                                        kEmptySlot));
  if (num_picked > 0)
    GS_LAUNCH("member_insert", s,
              member_insert_kernel<<<dim3((unsigned)ceil_div(num_picked, kBlock)),
                                     dim3(kBlock), 0, s>>>(picked, num_picked,
                                                           w.table, cap));
  GS_LAUNCH("member_flag", s,
            member_flag_kernel<<<dim3((unsigned)ceil_div(nnz + 1, kBlock)),
                                 dim3(kBlock), 0, s>>>(ids, nnz, w.table, cap,
                                                       w.prefix));
  int rc = exclusive_scan_i64(w.prefix, w.prefix, nnz + 1, w.scan_ws,
                              w.scan_ws_bytes, s);
  if (rc != GS_OK) return rc;
  const int64_t n = indptr ? num_major + 1 : 1;
  GS_LAUNCH("member_indptr", s,
            member_indptr_kernel<<<dim3((unsigned)ceil_div(n, kBlock)),
                                   dim3(kBlock), 0, s>>>(indptr, num_major,
                                                         w.prefix, nnz,
                                                         out_indptr, out_total));
  return GS_OK;
}

int gs_minor_slice_fill(const int64_t* ids, int64_t nnz, int64_t num_picked,
                        const int64_t* indptr, int64_t num_major,
                        const int64_t* edge_major, int64_t* out_major,
                        int64_t* out_minor, int64_t* out_select,
                        void* workspace, size_t workspace_bytes,
                        gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_picked >= 0 && num_major >= 0,
             "minor_slice_fill: negative size");
  if (nnz == 0) return GS_OK;
  GS_REQUIRE(ids, "minor_slice_fill: null ids");
  GS_REQUIRE(out_major == nullptr || edge_major != nullptr || indptr != nullptr,
             "minor_slice_fill: out_major needs edge_major or indptr");
  MemberWs w = carve_member(workspace, nnz, num_picked);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("minor_slice workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  const uint64_t cap = (uint64_t)(2 * num_picked + 2);
  GS_LAUNCH("member_fill", s,
            member_fill_kernel<<<dim3((unsigned)ceil_div(nnz, kBlock)),
                                 dim3(kBlock), 0, s>>>(
                ids, nnz, w.table, cap, w.prefix, indptr, num_major, edge_major,
                out_major, out_minor, out_select));
  return GS_OK;
}

}  // extern "C"
