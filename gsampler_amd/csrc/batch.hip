// batch.hip -- small super-batch bookkeeping kernels.
#include "common.h"

namespace gs {

__global__ __launch_bounds__(kBlock) void decode_batch_ids_kernel(
    const int64_t* __restrict__ encoded, int64_t n, int64_t stride,
    int64_t* __restrict__ orig, int64_t* __restrict__ batch) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t v = encoded[i];
  const int64_t b = v / stride;
  if (batch) batch[i] = b;
  if (orig) orig[i] = v - b * stride;
}

// Batch b's piece is indptr[offset[b] .. offset[b+1]] (inclusive) rebased to 0,
// written at out[offset[b] - offset[0] + b ...]: the pieces tile the output, one
// thread per output element.  An element finds its batch among the pieces'
// start positions offset[b] - offset[0] + b, which increase strictly.
__global__ __launch_bounds__(kBlock) void split_indptr_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ offset,
    int64_t num_batches, int64_t out_len, int64_t* __restrict__ out) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= out_len) return;
  const int64_t first = offset[0];
  int64_t lo = 0, hi = num_batches;  // the batch lies in [lo, hi)
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (offset[mid] - first + mid <= p)
      lo = mid;
    else
      hi = mid;
  }
  const int64_t begin = offset[lo];
  const int64_t j = p - (begin - first + lo);
  out[p] = indptr[begin + j] - indptr[begin];
}

}  // namespace gs

extern "C" {

int gs_decode_batch_ids(const int64_t* encoded, int64_t n, int64_t stride,
                        int64_t* out_orig, int64_t* out_batch,
                        gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0, "decode_batch_ids: negative size");
  GS_REQUIRE(stride > 0, "decode_batch_ids: stride must be positive, got %lld",
             (long long)stride);
  if (n == 0) return GS_OK;
  GS_REQUIRE(encoded, "decode_batch_ids: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("decode_batch_ids", s,
            decode_batch_ids_kernel<<<dim3((unsigned)ceil_div(n, kBlock)),
                                      dim3(kBlock), 0, s>>>(encoded, n, stride,
                                                            out_orig, out_batch));
  return GS_OK;
}

int gs_split_indptr(const int64_t* indptr, const int64_t* offset,
                    int64_t num_batches, int64_t out_len, int64_t* out,
                    gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_batches >= 0 && out_len >= 0, "split_indptr: negative size");
  if (num_batches == 0 || out_len == 0) return GS_OK;
  GS_REQUIRE(indptr && offset && out, "split_indptr: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("split_indptr", s,
            split_indptr_kernel<<<dim3((unsigned)ceil_div(out_len, kBlock)),
                                  dim3(kBlock), 0, s>>>(indptr, offset,
                                                        num_batches, out_len, out));
  return GS_OK;
}

}  // extern "C"
