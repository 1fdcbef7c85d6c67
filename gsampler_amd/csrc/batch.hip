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
// written at out[offset[b] - offset[0] + b ...]: the pieces tile the output.  A
// work-group takes kSplitTile consecutive output elements; the pieces start at
// offset[b] - offset[0] + b, which increases strictly with b, so the batches of
// the tile's first and last element are looked up once per work-group (the
// position is the same in every lane: scalar loads) and an element searches
// only between them -- not at all when one piece covers the tile.
constexpr int kSplitItems = 4;
constexpr int kSplitTile = kBlock * kSplitItems;

__device__ __forceinline__ int64_t piece_of(const int64_t* __restrict__ offset, int64_t first,
                                            int64_t lo, int64_t hi, int64_t p) {
  while (hi - lo > 1) {  // the piece lies in [lo, hi)
    const int64_t mid = (lo + hi) >> 1;
    if (offset[mid] - first + mid <= p)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(kBlock) void split_indptr_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ offset,
    int64_t num_batches, int64_t out_len, int64_t* __restrict__ out) {
  const int64_t p0 = (int64_t)blockIdx.x * kSplitTile;
  if (p0 >= out_len) return;
  const int64_t p_last = p0 + kSplitTile - 1 < out_len ? p0 + kSplitTile - 1 : out_len - 1;
  const int64_t first = offset[0];
  const int64_t b_lo = piece_of(offset, first, 0, num_batches, p0);
  const int64_t b_hi = piece_of(offset, first, b_lo, num_batches, p_last);
  int64_t begin = offset[b_lo], base = indptr[begin];
#pragma unroll
  for (int i = 0; i < kSplitItems; ++i) {
    const int64_t p = p0 + i * kBlock + threadIdx.x;
    if (p > p_last) break;
    int64_t b = b_lo;
    if (b_lo != b_hi) {
      b = piece_of(offset, first, b_lo, b_hi + 1, p);
      begin = offset[b];
      base = indptr[begin];
    }
    out[p] = indptr[begin + (p - (begin - first + b))] - base;
  }
}

// distinct[b] = 1 when the seeds of batch b are pairwise different.  The
// frontier of a batch lists its keys in first-occurrence order, seeds first, so
// the seeds are distinct exactly when the last seed sits at place ns - 1.
__global__ __launch_bounds__(kBlock) void seeds_distinct_kernel(
    const int64_t* __restrict__ frontier, const int64_t* __restrict__ frontier_ptr,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t num_batches, int64_t* __restrict__ distinct) {
  const int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (b >= num_batches) return;
  const int64_t s_lo = seeds_ptr[b], ns = seeds_ptr[b + 1] - s_lo;
  const int64_t f_lo = frontier_ptr[b], nu = frontier_ptr[b + 1] - f_lo;
  int64_t ok = 1;
  if (ns > 0) ok = nu >= ns && frontier[f_lo + ns - 1] == seeds[s_lo + ns - 1];
  distinct[b] = ok;
}

}  // namespace gs

extern "C" {

int gs_batch_seeds_distinct(const int64_t* frontier, const int64_t* frontier_ptr,
                            const int64_t* seeds, const int64_t* seeds_ptr,
                            int64_t num_batches, int64_t* out_distinct,
                            gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_batches >= 0, "batch_seeds_distinct: negative size");
  if (num_batches == 0) return GS_OK;
  GS_REQUIRE(frontier_ptr && seeds_ptr && out_distinct, "batch_seeds_distinct: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("seeds_distinct", s,
            seeds_distinct_kernel<<<dim3((unsigned)ceil_div(num_batches, kBlock)), dim3(kBlock),
                                    0, s>>>(frontier, frontier_ptr, seeds, seeds_ptr,
                                            num_batches, out_distinct));
  return GS_OK;
}

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
            split_indptr_kernel<<<dim3((unsigned)ceil_div(out_len, kSplitTile)),
                                  dim3(kBlock), 0, s>>>(indptr, offset,
                                                        num_batches, out_len, out));
  return GS_OK;
}

}  // extern "C"
