// walks.hip -- uniform random walk and node2vec over CSC in-neighbours.
// One thread per walk; traces are stored step-major, out[step * N + walk], so
// that a wavefront writes 64 consecutive ids per step (the reference uses the
// same layout, src/cuda/fusion/random_walk.cu:34).  Streams: pos = walk index;
// random walk draw = step; node2vec draw = step << 32 | attempt.
#include "common.h"

#pragma clang fp contract(off)

namespace gs {

__global__ __launch_bounds__(kBlock) void random_walk_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices,
    int64_t num_cols, const int64_t* __restrict__ seeds, int64_t num_seeds,
    int64_t walk_length, PhiloxKey key, int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= num_seeds) return;
  int64_t curr = seeds[i];
  out[i] = curr;
  for (int64_t step = 1; step <= walk_length; ++step) {
    int64_t pick = -1;
    if (curr >= 0 && curr < num_cols) {
      const int64_t start = indptr[curr];
      const int64_t deg = indptr[curr + 1] - start;
      if (deg > 0)
        pick = indices[start + (int64_t)philox_bounded(key, (uint64_t)i, (uint64_t)step,
                                                        (uint64_t)deg)];
    }
    curr = pick;
    out[step * num_seeds + i] = pick;
  }
}

// Is `target` among the sorted ids ptr[0, n)?
__device__ __forceinline__ bool sorted_contains(const int64_t* ptr, int64_t n,
                                                int64_t target) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    const int64_t v = ptr[mid];
    if (v == target) return true;
    if (v < target)
      lo = mid + 1;
    else
      hi = mid;
  }
  return false;
}

constexpr uint32_t kMaxAttempts = 1u << 16;

// Second-order walk by rejection sampling (src/cuda/fusion/node2vec.cu:90-135):
// every attempt draws an integer level y = floor(u * max(p, q)) and a uniform
// candidate; the candidate is accepted outright when y < min(p, q, 1), else when
// y < h with h = p for a return to the previous node, q for a neighbour of the
// previous node, 1 otherwise.
__global__ __launch_bounds__(kBlock) void node2vec_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices,
    int64_t num_cols, const int64_t* __restrict__ seeds, int64_t num_seeds,
    int64_t walk_length, double p, double q, PhiloxKey key,
    int64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= num_seeds) return;
  const double max_scale = p > q ? p : q;
  const double reject_from = max_scale > 1.0 ? max_scale : 1.0;
  double accept_below = p < q ? p : q;
  if (accept_below > 1.0) accept_below = 1.0;
  int64_t curr = seeds[i];
  int64_t last = -1;  // no previous node before the first step
  out[i] = curr;
  for (int64_t step = 1; step <= walk_length; ++step) {
    int64_t pick = -1;
    if (curr >= 0 && curr < num_cols) {
      const int64_t start = indptr[curr];
      const int64_t deg = indptr[curr + 1] - start;
      if (deg == 1) {
        pick = indices[start];
      } else if (deg > 1) {
        for (uint32_t attempt = 0;; ++attempt) {
          const Words4 w = philox(key, (uint64_t)i, ((uint64_t)step << 32) | attempt);
          const double u = (double)((w.z >> 8) + 1u) * 0x1p-24;  // (0, 1]
          const int y = (int)floor(u * max_scale);
          const uint64_t r = ((uint64_t)w.y << 32) | w.x;
          const int64_t cand = indices[start + (int64_t)__umul64hi(r, (uint64_t)deg)];
          pick = cand;
          if (attempt + 1 >= kMaxAttempts) break;
          if ((double)y >= reject_from) continue;
          if ((double)y < accept_below) break;
          double h = 1.0;
          if (cand == last) {
            h = p;
          } else if (((double)y < q) != ((double)y < 1.0) && last >= 0 &&
                     last < num_cols) {
            // the verdict differs between a neighbour of the previous node
            // (h = q) and any other node (h = 1) only for levels between q and
            // 1; everywhere else the adjacency search would change nothing
            const int64_t ls = indptr[last];
            if (sorted_contains(indices + ls, indptr[last + 1] - ls, cand)) h = q;
          }
          if ((double)y < h) break;
        }
      }
    }
    last = curr;
    curr = pick;
    out[step * num_seeds + i] = pick;
  }
}

}  // namespace gs

extern "C" {

int gs_random_walk(const int64_t* indptr, const int64_t* indices, int64_t num_cols,
                   const int64_t* seeds, int64_t num_seeds, int64_t walk_length,
                   uint64_t seed, uint64_t call_id, int64_t* out_traces,
                   gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_seeds >= 0 && walk_length >= 0 && num_cols >= 0,
             "random_walk: negative size");
  if (num_seeds == 0) return GS_OK;
  GS_REQUIRE(indptr && seeds && out_traces, "random_walk: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("random_walk", s,
            random_walk_kernel<<<dim3((unsigned)ceil_div(num_seeds, kBlock)),
                                 dim3(kBlock), 0, s>>>(
                indptr, indices, num_cols, seeds, num_seeds, walk_length,
                make_key(seed, call_id), out_traces));
  return GS_OK;
}

int gs_node2vec(const int64_t* indptr, const int64_t* indices, int64_t num_cols,
                const int64_t* seeds, int64_t num_seeds, int64_t walk_length,
                double p, double q, uint64_t seed, uint64_t call_id,
                int64_t* out_traces, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_seeds >= 0 && walk_length >= 0 && num_cols >= 0,
             "node2vec: negative size");
  GS_REQUIRE(p > 0.0 && q > 0.0, "node2vec: p and q must be positive");
  if (num_seeds == 0) return GS_OK;
  GS_REQUIRE(indptr && seeds && out_traces, "node2vec: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("node2vec", s,
            node2vec_kernel<<<dim3((unsigned)ceil_div(num_seeds, kBlock)),
                              dim3(kBlock), 0, s>>>(
                indptr, indices, num_cols, seeds, num_seeds, walk_length, p, q,
                make_key(seed, call_id), out_traces));
  return GS_OK;
}

}  // extern "C"
