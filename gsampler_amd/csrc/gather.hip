// gather.hip -- row gather out[i, :] = table[ids[i], :] for rows of any byte
// length: node features of a sampled frontier, labels, edge data behind an
// edge index.  The table may live in device memory or in pinned host memory
// (read over the host link by the same loads).
#include "common.h"

namespace gs {

typedef uint32_t vec16 __attribute__((ext_vector_type(4)));
typedef uint32_t vec8 __attribute__((ext_vector_type(2)));

constexpr int kGatherRows = 4;  // rows a lane group keeps in flight

// A group of L lanes copies a row as vectors of type V (L = the power of two at
// or above the vectors per row, at most 64, so short rows do not idle lanes);
// it takes kGatherRows rows per trip and issues their loads together.  Output
// rows are written once and never read by this kernel: non-temporal stores keep
// them from displacing table rows that the next ids hit again (frontiers of
// neighbouring mini-batches share their high-degree nodes).
template <typename V, int L>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(
    const V* __restrict__ table, int64_t num_rows, int64_t vec_per_row,
    const int64_t* __restrict__ ids, int64_t n, V* __restrict__ out,
    unsigned long long* bad_count) {
  const int lane = threadIdx.x % L;
  const int64_t group = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / L;
  const int64_t base = group * kGatherRows;
  if (base >= n) return;
  int64_t src[kGatherRows];
#pragma unroll
  for (int u = 0; u < kGatherRows; ++u) {
    src[u] = -1;
    if (base + u < n) {
      const int64_t id = ids[base + u];
      if (id >= 0 && id < num_rows)
        src[u] = id * vec_per_row;
      else if (lane == 0 && bad_count != nullptr)
        atomicAdd(bad_count, 1ull);
    }
  }
  for (int64_t j = lane; j < vec_per_row; j += L) {
    V v[kGatherRows];
#pragma unroll
    for (int u = 0; u < kGatherRows; ++u) {
      v[u] = V(0);
      if (src[u] >= 0) v[u] = table[src[u] + j];
    }
#pragma unroll
    for (int u = 0; u < kGatherRows; ++u)
      if (base + u < n)
        __builtin_nontemporal_store(v[u], out + (base + u) * vec_per_row + j);
  }
}

// Rows of a single vector (edge data, labels, id arrays): consecutive lanes take
// consecutive output positions, kGatherRows of them per thread a block apart,
// so that stores and the id loads are coalesced.
template <typename V>
__global__ __launch_bounds__(kBlock) void gather_scalar_kernel(
    const V* __restrict__ table, int64_t num_rows, const int64_t* __restrict__ ids,
    int64_t n, V* __restrict__ out, unsigned long long* bad_count) {
  const int64_t base = (int64_t)blockIdx.x * (kBlock * kGatherRows) + threadIdx.x;
  int64_t id[kGatherRows];
#pragma unroll
  for (int u = 0; u < kGatherRows; ++u) {
    const int64_t i = base + u * kBlock;
    id[u] = i < n ? ids[i] : 0;
  }
  V v[kGatherRows];
#pragma unroll
  for (int u = 0; u < kGatherRows; ++u) {
    const bool ok = id[u] >= 0 && id[u] < num_rows;
    v[u] = V(0);
    if (ok)
      v[u] = table[id[u]];
    else if (base + u * kBlock < n && bad_count != nullptr)
      atomicAdd(bad_count, 1ull);
  }
#pragma unroll
  for (int u = 0; u < kGatherRows; ++u) {
    const int64_t i = base + u * kBlock;
    if (i < n) __builtin_nontemporal_store(v[u], out + i);
  }
}

__global__ void gather_clear_kernel(unsigned long long* bad_count) { *bad_count = 0; }

template <typename V>
static int gather_launch(const void* table, int64_t num_rows, int64_t row_bytes,
                         const int64_t* ids, int64_t n, void* out,
                         unsigned long long* bad_count, hipStream_t s) {
  const int64_t vpr = row_bytes / (int64_t)sizeof(V);
  if (vpr == 1) {
    const int64_t blocks = ceil_div(n, (int64_t)kBlock * kGatherRows);
    GS_REQUIRE(blocks < ((int64_t)1 << 31), "gather_rows: %lld rows need too many work-groups",
               (long long)n);
    GS_LAUNCH("gather_rows", s,
              gather_scalar_kernel<V><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(
                  (const V*)table, num_rows, ids, n, (V*)out, bad_count));
    return GS_OK;
  }
  int lanes = 1;
  while (lanes < kWave && lanes < vpr) lanes *= 2;
  const int64_t groups = ceil_div(n, (int64_t)kGatherRows);
  const int64_t blocks = ceil_div(groups * lanes, (int64_t)kBlock);
  GS_REQUIRE(blocks < ((int64_t)1 << 31), "gather_rows: %lld rows need too many work-groups",
             (long long)n);
#define GS_GATHER(L)                                                            \
  case L:                                                                       \
    GS_LAUNCH("gather_rows", s,                                                 \
              gather_rows_kernel<V, L><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>( \
                  (const V*)table, num_rows, vpr, ids, n, (V*)out, bad_count)); \
    break
  switch (lanes) {
    GS_GATHER(1);
    GS_GATHER(2);
    GS_GATHER(4);
    GS_GATHER(8);
    GS_GATHER(16);
    GS_GATHER(32);
    GS_GATHER(64);
  }
#undef GS_GATHER
  return GS_OK;
}

}  // namespace gs

extern "C" int gs_gather_rows(const void* table, int64_t num_rows, int64_t row_bytes,
                              const int64_t* ids, int64_t n, void* out,
                              int64_t* bad_count, void* stream) {
  using namespace gs;
  GS_REQUIRE(num_rows >= 0 && row_bytes >= 0 && n >= 0, "gather_rows: negative size");
  hipStream_t s = (hipStream_t)stream;
  if (bad_count != nullptr)
    GS_LAUNCH("gather_clear", s,
              gather_clear_kernel<<<dim3(1), dim3(1), 0, s>>>((unsigned long long*)bad_count));
  if (n == 0 || row_bytes == 0) return GS_OK;
  GS_REQUIRE(table && ids && out, "gather_rows: null pointer");
  // widest vector that divides the row length and that both bases are aligned to
  const uintptr_t bits = (uintptr_t)table | (uintptr_t)out | (uintptr_t)row_bytes;
  unsigned long long* bad = (unsigned long long*)bad_count;
  if (bits % 16 == 0) return gather_launch<vec16>(table, num_rows, row_bytes, ids, n, out, bad, s);
  if (bits % 8 == 0) return gather_launch<vec8>(table, num_rows, row_bytes, ids, n, out, bad, s);
  if (bits % 4 == 0) return gather_launch<uint32_t>(table, num_rows, row_bytes, ids, n, out, bad, s);
  if (bits % 2 == 0) return gather_launch<uint16_t>(table, num_rows, row_bytes, ids, n, out, bad, s);
  return gather_launch<uint8_t>(table, num_rows, row_bytes, ids, n, out, bad, s);
}
