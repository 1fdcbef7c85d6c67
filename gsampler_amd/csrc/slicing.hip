// slicing.hip -- per-column counts and the CSC column slice.
#include "common.h"
#include "scan.h"

#include <mutex>

namespace gs {

// Scan scratch of gs_csc_col_count_static: one tile sum per kScanTile counts,
// held by every device the library runs on until the process ends.
constexpr int64_t kStaticScanTiles = 65536;  // 512 KiB
constexpr int64_t kStaticCountMaxItems = kStaticScanTiles * kScanTile - 1;
static __device__ __align__(256) int64_t scratch[kStaticScanTiles];

// Device address of `scratch` on the current device.  The array's name is only
// a host-side handle; every device has its own copy at its own address, looked
// up once per device.
constexpr int kMaxDevices = 64;
static int static_scratch(int64_t** out) {
  static std::mutex mutex;
  static int64_t* ptr[kMaxDevices] = {};
  int dev = -1;
  GS_HIP(hipGetDevice(&dev));
  GS_REQUIRE(dev >= 0 && dev < kMaxDevices, "col_count_static: device %d not supported", dev);
  std::lock_guard<std::mutex> lock(mutex);
  if (ptr[dev] == nullptr) {
    void* p = nullptr;
    GS_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    GS_REQUIRE(p != nullptr, "col_count_static: no device address for the scratch array");
    ptr[dev] = (int64_t*)p;
  }
  *out = ptr[dev];
  return GS_OK;
}

// One work-group of kCountThreads threads per tile of the scan that follows
// (kScanTile consecutive columns): writes the output counts and the tile's sum,
// so that the scan only has its down sweep left to turn the counts into
// sub_indptr in place.
constexpr int kCountThreads = 1024;
constexpr int kCountItems = kScanTile / kCountThreads;
__global__ __launch_bounds__(kCountThreads) void col_count_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ column_ids, int64_t num_items, int64_t fanout,
    int replace, int64_t* __restrict__ counts, int64_t* __restrict__ tile_sums,
    int64_t* __restrict__ col_span) {
  __shared__ int64_t smem[kCountThreads / kWave + 1];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + threadIdx.x;
  int64_t cnt[kCountItems], sum = 0;
#pragma unroll
  for (int k = 0; k < kCountItems; ++k) {
    const int64_t i = base + k * kCountThreads;
    cnt[k] = 0;
    if (i < num_items) {
      int64_t in_start;
      const int64_t deg =
          column_degree(indptr, num_cols, column_ids ? column_ids[i] : i, &in_start);
      if (col_span) col_span[i] = pack_span(in_start, deg);
      if (fanout < 0)
        cnt[k] = deg;
      else if (replace)
        cnt[k] = deg == 0 ? 0 : fanout;
      else
        cnt[k] = deg < fanout ? deg : fanout;
    }
    sum += cnt[k];
  }
#pragma unroll
  for (int k = 0; k < kCountItems; ++k) {
    const int64_t i = base + k * kCountThreads;
    if (i <= num_items) counts[i] = cnt[k];  // counts[num_items] = 0: the scan leaves the total there
  }
  int64_t total;
  block_exclusive_sum<int64_t, kCountThreads>(sum, smem, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Up to kSmallCountItems columns: one work-group counts and scans in a single
// launch (every thread asks for its eight columns' pointers at once), where the
// tiled pair of launches above costs a small sampling step one launch more per
// layer than it has work for.
constexpr int kSmallCountPer = 8;
constexpr int64_t kSmallCountItems = (int64_t)kCountThreads * kSmallCountPer - 1;
__global__ __launch_bounds__(kCountThreads) void col_count_small_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ column_ids, int64_t num_items, int64_t fanout,
    int replace, int64_t* __restrict__ sub_indptr, int64_t* total_mirror,
    int64_t* __restrict__ col_span) {
  __shared__ int64_t smem[kCountThreads / kWave + 1];
  // thread t owns columns t * 8 .. t * 8 + 7: its prefix sums leave in one run
  const int64_t base = (int64_t)threadIdx.x * kSmallCountPer;
  int64_t cnt[kSmallCountPer], sum = 0;
#pragma unroll
  for (int k = 0; k < kSmallCountPer; ++k) {
    const int64_t i = base + k;
    cnt[k] = 0;
    if (i < num_items) {
      int64_t in_start;
      const int64_t deg =
          column_degree(indptr, num_cols, column_ids ? column_ids[i] : i, &in_start);
      if (col_span) col_span[i] = pack_span(in_start, deg);
      if (fanout < 0)
        cnt[k] = deg;
      else if (replace)
        cnt[k] = deg == 0 ? 0 : fanout;
      else
        cnt[k] = deg < fanout ? deg : fanout;
    }
    sum += cnt[k];
  }
  int64_t total;
  int64_t run = block_exclusive_sum<int64_t, kCountThreads>(sum, smem, &total);
#pragma unroll
  for (int k = 0; k < kSmallCountPer; ++k) {
    const int64_t i = base + k;
    if (i <= num_items) sub_indptr[i] = run;
    run += cnt[k];
  }
  if (threadIdx.x == 0 && total_mirror) *total_mirror = total;
}

// Edge-parallel slice: thread e owns output edge e, finds its column by binary
// search in sub_indptr (L2-resident; skipped when its whole tile lies in one
// column) and copies one row id.  Load balance is
// independent of the degree distribution; reads within a column and all
// writes are coalesced.
constexpr int kSliceItems = 4;
constexpr int kSliceTile = kBlock * kSliceItems;

__global__ __launch_bounds__(kBlock) void col_slice_fill_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices, const int64_t* __restrict__ column_ids,
    int64_t num_items, const int64_t* __restrict__ sub_indptr, int64_t nnz,
    const int64_t* __restrict__ batch_ptr, int64_t num_batches,
    int64_t encode_stride, int64_t* __restrict__ out_coo_col,
    int64_t* __restrict__ out_indices, int64_t* __restrict__ out_select) {
  const int64_t e0 = (int64_t)blockIdx.x * kSliceTile;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kSliceTile - 1 < nnz ? e0 + kSliceTile - 1 : nnz - 1;
  // columns that the tile touches: one search per work-group (on the scalar
  // unit) instead of one per edge; a long column covers whole tiles
  const SegmentSpan span = segment_span(sub_indptr, num_items, e0, e_last);
  if (span.lo == span.hi && e0 + kSliceTile <= nnz &&
      (((uintptr_t)out_indices | (uintptr_t)out_select | (uintptr_t)out_coo_col) & 15) == 0) {
    // a whole tile out of one column: two edges (16 bytes) per lane and
    // instruction; the source run is only aligned to 8 bytes
    struct Pair {
      int64_t v[2];
    };
    const int64_t col = span.lo;
    const int64_t c = column_ids ? column_ids[col] : col;
    const int64_t shift = indptr[c] - sub_indptr[col];
    int64_t add = 0;
    if (batch_ptr != nullptr && encode_stride > 0)
      add = segment_of(batch_ptr, num_batches, col) * encode_stride;
    constexpr int kVecs = kSliceItems / 2;
    Pair rows[kVecs];
#pragma unroll
    for (int j = 0; j < kVecs; ++j)
      __builtin_memcpy(&rows[j], indices + e0 + shift + (j * kBlock + (int)threadIdx.x) * 2,
                       sizeof(Pair));
#pragma unroll
    for (int j = 0; j < kVecs; ++j) {
      const int64_t e = e0 + (j * kBlock + (int)threadIdx.x) * 2;
      const Pair r{{rows[j].v[0] + add, rows[j].v[1] + add}};
      const Pair p{{e + shift, e + shift + 1}};
      __builtin_memcpy(__builtin_assume_aligned(out_indices + e, 16), &r, sizeof(Pair));
      __builtin_memcpy(__builtin_assume_aligned(out_select + e, 16), &p, sizeof(Pair));
      if (out_coo_col) {
        const Pair cc{{col, col}};
        __builtin_memcpy(__builtin_assume_aligned(out_coo_col + e, 16), &cc, sizeof(Pair));
      }
    }
    return;
  }
  int64_t item[kSliceItems], in_pos[kSliceItems], row[kSliceItems];
#pragma unroll
  for (int j = 0; j < kSliceItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    item[j] = -1;
    if (e >= nnz) continue;
    item[j] = span.segment_at(sub_indptr, e);
    const int64_t c = column_ids ? column_ids[item[j]] : item[j];
    in_pos[j] = indptr[c] + (e - sub_indptr[item[j]]);
  }
#pragma unroll
  for (int j = 0; j < kSliceItems; ++j)
    if (item[j] >= 0) row[j] = indices[in_pos[j]];
#pragma unroll
  for (int j = 0; j < kSliceItems; ++j) {
    if (item[j] < 0) continue;
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (batch_ptr != nullptr && encode_stride > 0)
      row[j] += segment_of(batch_ptr, num_batches, item[j]) * encode_stride;
    out_indices[e] = row[j];
    out_select[e] = in_pos[j];
    if (out_coo_col) out_coo_col[e] = item[j];
  }
}

// Per-edge values of the slice: out[sub_indptr[i] + k] = values[indptr[c_i] + k].
// The edges of a sliced column are a run of the parent's edges, so the values
// come straight from the parent's array; the edge positions the slice kernel
// wrote (8 bytes per edge) are not read back.
// (Four bytes in and out per edge: a work-group takes eight edges per thread,
// so the look-ups at its head are paid once per 2048 edges; four, sixteen and
// thirty-two per thread all measured slower.)
constexpr int kValueItems = 8;
constexpr int kValueTile = kBlock * kValueItems;
template <typename T>
__global__ __launch_bounds__(kBlock) void col_slice_values_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ column_ids, int64_t num_items,
    const int64_t* __restrict__ sub_indptr, int64_t nnz, const T* __restrict__ values,
    T* __restrict__ out) {
  const int64_t e0 = (int64_t)blockIdx.x * kValueTile;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kValueTile - 1 < nnz ? e0 + kValueTile - 1 : nnz - 1;
  const SegmentSpan span = segment_span(sub_indptr, num_items, e0, e_last);
  // one column covers the tile (columns of a slice worth copying are long): its
  // offset is the same for every edge
  int64_t shift = 0;
  if (span.lo == span.hi) {
    const int64_t c = column_ids ? column_ids[span.lo] : span.lo;
    shift = indptr[c] - sub_indptr[span.lo];
  }
  if (span.lo == span.hi && e0 + kValueTile <= nnz && ((uintptr_t)out & 15) == 0) {
    // a whole tile out of one column: 16 bytes per lane and instruction; the
    // source run starts wherever the column does, so its vectors are only
    // aligned to the value size (the loads are issued as such)
    constexpr int kPer = 16 / (int)sizeof(T), kVecs = kValueItems / kPer;
    struct Vec {
      T v[kPer];
    };
    const T* from = values + e0 + shift;
    T* to = out + e0;
    Vec held[kVecs];
#pragma unroll
    for (int j = 0; j < kVecs; ++j)
      __builtin_memcpy(&held[j], from + (j * kBlock + (int)threadIdx.x) * kPer, sizeof(Vec));
#pragma unroll
    for (int j = 0; j < kVecs; ++j)
      __builtin_memcpy(__builtin_assume_aligned(to + (j * kBlock + (int)threadIdx.x) * kPer, 16),
                       &held[j], sizeof(Vec));
    return;
  }
  int64_t src[kValueItems];
#pragma unroll
  for (int j = 0; j < kValueItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    src[j] = -1;
    if (e >= nnz) continue;
    if (span.lo == span.hi) {
      src[j] = e + shift;
    } else {
      const int64_t item = span.segment_at(sub_indptr, e);
      const int64_t c = column_ids ? column_ids[item] : item;
      src[j] = indptr[c] + (e - sub_indptr[item]);
    }
  }
  T v[kValueItems];
#pragma unroll
  for (int j = 0; j < kValueItems; ++j)
    if (src[j] >= 0) v[j] = values[src[j]];
#pragma unroll
  for (int j = 0; j < kValueItems; ++j)
    if (src[j] >= 0) out[e0 + j * kBlock + threadIdx.x] = v[j];
}

}  // namespace gs

extern "C" {

int gs_csc_col_slice_values(const int64_t* indptr, const int64_t* column_ids, int64_t num_items,
                            const int64_t* sub_indptr, int64_t nnz, const void* values,
                            int64_t value_bytes, void* out_values, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items >= 0 && nnz >= 0, "col_slice_values: negative size");
  GS_REQUIRE(value_bytes == 4 || value_bytes == 8,
             "col_slice_values: values of 4 or 8 bytes, got %lld (gather by edge position instead)",
             (long long)value_bytes);
  if (nnz == 0 || num_items == 0) return GS_OK;
  GS_REQUIRE(indptr && sub_indptr && values && out_values, "col_slice_values: null pointer");
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)ceil_div(nnz, kValueTile));
  if (value_bytes == 4)
    GS_LAUNCH("col_slice_values", s,
              col_slice_values_kernel<uint32_t><<<grid, dim3(kBlock), 0, s>>>(
                  indptr, column_ids, num_items, sub_indptr, nnz, (const uint32_t*)values,
                  (uint32_t*)out_values));
  else
    GS_LAUNCH("col_slice_values", s,
              col_slice_values_kernel<uint64_t><<<grid, dim3(kBlock), 0, s>>>(
                  indptr, column_ids, num_items, sub_indptr, nnz, (const uint64_t*)values,
                  (uint64_t*)out_values));
  return GS_OK;
}

int gs_csc_col_count(const int64_t* indptr, int64_t num_cols,
                     const int64_t* column_ids, int64_t num_items,
                     int64_t fanout, int replace, int64_t* sub_indptr,
                     int64_t* total_mirror, int64_t* out_col_span, void* workspace,
                     size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items >= 0 && num_cols >= 0, "col_count: negative size");
  GS_REQUIRE(indptr && sub_indptr, "col_count: null pointer");
  GS_REQUIRE(column_ids != nullptr || num_items <= num_cols,
             "col_count: %lld items but the matrix has %lld columns",
             (long long)num_items, (long long)num_cols);
  hipStream_t s = as_stream(stream);
  const int64_t n = num_items + 1;
  if (workspace == nullptr || workspace_bytes < scan_workspace_bytes(n)) {
    set_error("col_count: workspace too small: %zu < %zu", workspace_bytes,
              scan_workspace_bytes(n));
    return GS_ERR_WORKSPACE;
  }
  if (num_items <= kSmallCountItems) {
    GS_LAUNCH("col_count", s,
              col_count_small_kernel<<<dim3(1), dim3(kCountThreads), 0, s>>>(
                  indptr, num_cols, column_ids, num_items, fanout, replace, sub_indptr,
                  total_mirror, out_col_span));
    return GS_OK;
  }
  GS_LAUNCH("col_count", s,
            col_count_kernel<<<dim3((unsigned)ceil_div(n, kScanTile)), dim3(kCountThreads),
                               0, s>>>(indptr, num_cols, column_ids, num_items,
                                       fanout, replace, sub_indptr,
                                       (int64_t*)workspace, out_col_span));
  return exclusive_scan_i64(sub_indptr, sub_indptr, n, workspace,
                            workspace_bytes, s, /*sums_ready=*/true, total_mirror);
}

int gs_csc_col_count_static(const int64_t* indptr, int64_t num_cols,
                            const int64_t* column_ids, int64_t num_items,
                            int64_t fanout, int replace, int64_t* sub_indptr,
                            gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items >= 0 && num_cols >= 0, "col_count_static: negative size");
  GS_REQUIRE(num_items <= kStaticCountMaxItems,
             "col_count_static: %lld items exceed the fixed scratch (at most %lld); "
             "use gs_csc_col_count with a workspace",
             (long long)num_items, (long long)kStaticCountMaxItems);
  int64_t* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != GS_OK) return rc;
  return gs_csc_col_count(indptr, num_cols, column_ids, num_items, fanout, replace,
                          sub_indptr, nullptr, nullptr, ws,
                          (size_t)kStaticScanTiles * sizeof(int64_t), stream);
}

int gs_csc_col_slice_fill(const int64_t* indptr, int64_t num_cols,
                          const int64_t* indices, const int64_t* column_ids,
                          int64_t num_items, const int64_t* sub_indptr,
                          int64_t nnz, const int64_t* batch_ptr,
                          int64_t num_batches, int64_t encode_stride,
                          int64_t* out_coo_col, int64_t* out_indices,
                          int64_t* out_select, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items >= 0 && nnz >= 0, "col_slice_fill: negative size");
  if (nnz == 0 || num_items == 0) return GS_OK;
  GS_REQUIRE(indptr && indices && sub_indptr && out_indices && out_select,
             "col_slice_fill: null pointer");
  GS_REQUIRE(batch_ptr == nullptr || num_batches > 0,
             "col_slice_fill: batch_ptr given but num_batches = %lld",
             (long long)num_batches);
  (void)num_cols;  // ids were validated by the count phase
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("col_slice_fill", s,
            col_slice_fill_kernel<<<dim3((unsigned)ceil_div(nnz, kSliceTile)),
                                    dim3(kBlock), 0, s>>>(
                indptr, indices, column_ids, num_items, sub_indptr, nnz,
                batch_ptr, num_batches, encode_stride, out_coo_col, out_indices,
                out_select));
  return GS_OK;
}

}  // extern "C"
