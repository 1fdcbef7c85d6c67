// format.hip -- CSC <-> COO conversion kernels.
#include "common.h"

namespace gs {

// Column id of every edge: the segment of indptr that holds the edge position.
__global__ __launch_bounds__(kBlock) void csc2coo_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz,
    int64_t* __restrict__ out_col) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= nnz) return;
  out_col[e] = segment_of(indptr, num_cols, e);
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
            csc2coo_kernel<<<dim3((unsigned)ceil_div(nnz, kBlock)), dim3(kBlock),
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

}  // extern "C"
