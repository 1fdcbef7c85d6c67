// format.hip -- CSC <-> COO conversion kernels.
#include "common.h"

namespace gs {

// Column id of every edge: the segment of indptr that holds the edge position,
// looked up per tile of consecutive edges.
constexpr int kCooItems = 8;
constexpr int kCooTile = kBlock * kCooItems;

__global__ __launch_bounds__(kBlock) void csc2coo_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz,
    int64_t* __restrict__ out_col) {
  const int64_t e0 = (int64_t)blockIdx.x * kCooTile;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kCooTile - 1 < nnz ? e0 + kCooTile - 1 : nnz - 1;
  const SegmentSpan span = segment_span(indptr, num_cols, e0, e_last);
#pragma unroll
  for (int j = 0; j < kCooItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (e >= nnz) break;
    out_col[e] = span.segment_at(indptr, e);
  }
}

// indptr[c] = number of entries of the sorted column array that are < c.
__global__ __launch_bounds__(kBlock) void sorted_to_indptr_kernel(
    const int64_t* __restrict__ sorted, int64_t nnz, int64_t num_cols,
    int64_t* __restrict__ indptr) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (c > num_cols) return;
  int64_t lo = 0, hi = nnz;  // first position with sorted[pos] >= c
  while (lo < hi) {
    int64_t mid = (lo + hi) >> 1;
    if (sorted[mid] < c)
      lo = mid + 1;
    else
      hi = mid;
  }
  indptr[c] = lo;
}

}  // namespace gs

namespace gs {

// first[r] = smallest e with ids[e] == r (INT64_MAX for an id that does not
// occur), for ids in a small dense range [0, num_ids).  Atomics from all dies
// on a few hundred addresses would queue up at the memory side, so a
// work-group first takes the minimum over its tile of edges in LDS and then
// sends one atomic per id it met -- and only if the value in memory is not
// already smaller, which it is for every tile but the first few.
constexpr int kFirstLdsIds = 4096;
constexpr int kFirstTile = kBlock * 32;

__global__ __launch_bounds__(kBlock) void first_position_lds_kernel(
    const int64_t* __restrict__ ids, int64_t n, int64_t num_ids, long long* first) {
  __shared__ long long tile_min[kFirstLdsIds];
  for (int i = threadIdx.x; i < num_ids; i += kBlock) tile_min[i] = INT64_MAX;
  __syncthreads();
  const int64_t e0 = (int64_t)blockIdx.x * kFirstTile;
  const int64_t e1 = e0 + kFirstTile < n ? e0 + kFirstTile : n;
  for (int64_t base = e0; base < e1; base += kBlock * 8) {
    int64_t r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t e = base + j * kBlock + threadIdx.x;
      r[j] = e < e1 ? ids[e] : -1;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t e = base + j * kBlock + threadIdx.x;
      if (r[j] >= 0 && r[j] < num_ids && tile_min[r[j]] > e)
        atomicMin(&tile_min[r[j]], (long long)e);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < num_ids; i += kBlock) {
    const long long m = tile_min[i];
    if (m != INT64_MAX &&
        __hip_atomic_load(first + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > m)
      atomicMin(first + i, m);
  }
}

// The same for a range of ids too large for LDS: one atomic per edge unless a
// smaller position is already there.
__global__ __launch_bounds__(kBlock) void first_position_kernel(
    const int64_t* __restrict__ ids, int64_t n, int64_t num_ids, long long* first) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= n) return;
  const int64_t r = ids[e];
  if (r < 0 || r >= num_ids) return;
  if (__hip_atomic_load(first + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > e)
    atomicMin(first + r, (long long)e);
}

__global__ __launch_bounds__(kBlock) void fill_i64_kernel(int64_t* p, int64_t n, int64_t v) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = v;
}

}  // namespace gs

extern "C" {

int gs_csc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz,
               int64_t* out_col, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_cols >= 0 && nnz >= 0, "csc2coo: negative size");
  if (nnz == 0) return GS_OK;
  GS_REQUIRE(indptr && out_col, "csc2coo: null pointer");
  GS_REQUIRE(num_cols > 0, "csc2coo: %lld edges but no columns", (long long)nnz);
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("csc2coo", s,
            csc2coo_kernel<<<dim3((unsigned)ceil_div(nnz, kCooTile)), dim3(kBlock),
                             0, s>>>(indptr, num_cols, nnz, out_col));
  return GS_OK;
}

int gs_sorted_to_indptr(const int64_t* sorted_ids, int64_t nnz, int64_t num_cols,
                        int64_t* out_indptr, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_cols >= 0 && nnz >= 0, "sorted_to_indptr: negative size");
  GS_REQUIRE(out_indptr && (nnz == 0 || sorted_ids),
             "sorted_to_indptr: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("sorted_to_indptr", s,
            sorted_to_indptr_kernel<<<dim3((unsigned)ceil_div(num_cols + 1, kBlock)),
                                      dim3(kBlock), 0, s>>>(sorted_ids, nnz,
                                                            num_cols, out_indptr));
  return GS_OK;
}

int gs_first_position(const int64_t* ids, int64_t n, int64_t num_ids,
                      int64_t* out_first, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0 && num_ids >= 0, "first_position: negative size");
  if (num_ids == 0) return GS_OK;
  GS_REQUIRE(out_first && (n == 0 || ids), "first_position: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("first_position_init", s,
            fill_i64_kernel<<<dim3((unsigned)ceil_div(num_ids, kBlock)), dim3(kBlock), 0,
                              s>>>(out_first, num_ids, INT64_MAX));
  if (n > 0 && num_ids <= kFirstLdsIds)
    GS_LAUNCH("first_position", s,
              first_position_lds_kernel<<<dim3((unsigned)ceil_div(n, kFirstTile)),
                                          dim3(kBlock), 0, s>>>(ids, n, num_ids,
                                                                (long long*)out_first));
  else if (n > 0)
    GS_LAUNCH("first_position", s,
              first_position_kernel<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0,
                                      s>>>(ids, n, num_ids, (long long*)out_first));
  return GS_OK;
}

}  // extern "C"
