// sort.hip -- per-segment key sort (row ids inside every column), the
// prerequisite of node2vec's connectivity test, and the stable sort of edges by
// column (or row) id that turns an edge list into a compressed format.  Ids
// below 2^32 (every graph's ids) are sorted per segment by the kernels of
// segsort.hip and over an edge list by those of coosort.hip; for wider or
// unbounded keys and for lists of 2^32 edges and more this file adapts rocPRIM's
// radix sorts to the workspace convention and limits the sorted bits to what
// the ids need.
#include "common.h"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_segmented_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

namespace gs {

// segsort.hip
size_t segsort_workspace_bytes(int64_t nnz, int64_t num_segments, int key_bits);
int segsort_run(const int64_t* indptr, int64_t num_segments, const int64_t* keys_in,
                int64_t* keys_out, int64_t nnz, int key_bits, void* workspace, hipStream_t s);

// coosort.hip
size_t coosort_workspace_bytes(int64_t nnz, int id_bits);
int coosort_run(const int64_t* major, int64_t nnz, int id_bits, int64_t* sorted_major,
                int64_t* perm, void* workspace, hipStream_t s);

static int id_bits(int64_t num_ids) {
  int bits = 1;
  while (bits < 63 && ((int64_t)1 << bits) < num_ids) ++bits;
  return bits;
}

// Segment and key in one word: (segment << key_bits) | key.  A plain radix sort
// of these words over the bits they use sorts every segment, because the input
// is already grouped by segment; it moves every key a fixed number of times
// whatever the segment sizes are, where a segmented sort of millions of short
// segments and a few hubs spends its time on scheduling them.
constexpr int kPackItems = 8;
constexpr int kPackTile = kBlock * kPackItems;

__global__ __launch_bounds__(kBlock) void pack_segment_keys_kernel(
    const int64_t* __restrict__ indptr, int64_t num_segments,
    const int64_t* __restrict__ keys, int64_t nnz, int key_bits,
    uint64_t* __restrict__ packed) {
  const int64_t e0 = (int64_t)blockIdx.x * kPackTile;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kPackTile - 1 < nnz ? e0 + kPackTile - 1 : nnz - 1;
  const SegmentSpan span = segment_span(indptr, num_segments, e0, e_last);
#pragma unroll
  for (int j = 0; j < kPackItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (e > e_last) break;
    packed[e] = ((uint64_t)span.segment_at(indptr, e) << key_bits) | (uint64_t)keys[e];
  }
}

__global__ __launch_bounds__(kBlock) void unpack_segment_keys_kernel(
    int64_t* __restrict__ keys, int64_t nnz, int key_bits) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= nnz) return;
  keys[e] = (int64_t)((uint64_t)keys[e] & (((uint64_t)1 << key_bits) - 1));
}

// Bits of the packed word, or 0 when segment and key do not fit one word (or
// the key range is not known): then the segmented sort over all 64 bits runs.
static int packed_bits(int64_t num_segments, int64_t key_bound, int* key_bits) {
  if (key_bound <= 0) return 0;
  *key_bits = id_bits(key_bound);
  const int total = *key_bits + id_bits(num_segments);
  return total <= 64 ? total : 0;
}

// Whether the kernels of segsort.hip take the call: ids known to lie below 2^32,
// positions inside a segment that fit 32 bits.
static bool native_segment_sort(int64_t nnz, int64_t key_bound) {
  return key_bound > 0 && key_bound <= (int64_t(1) << 32) && nnz < (int64_t(1) << 32);
}

// Whether the kernels of coosort.hip take the call: ids and positions of 32 bits.
static bool native_coo_sort(int64_t nnz, int64_t num_major) {
  return nnz > 0 && nnz < (int64_t(1) << 32) && num_major <= (int64_t(1) << 32);
}

static size_t segmented_temp_bytes(int64_t nnz, int64_t num_segments) {
  size_t bytes = 0;
  const int64_t* k = nullptr;
  int64_t* o = nullptr;
  (void)rocprim::segmented_radix_sort_keys(nullptr, bytes, k, o, (size_t)(nnz > 0 ? nnz : 1),
                                           (unsigned)(num_segments > 0 ? num_segments : 1),
                                           k, k, 0, 64);
  return align_up(bytes, 256);
}

static size_t packed_temp_bytes(int64_t nnz, int bits) {
  size_t bytes = 0;
  const uint64_t* k = nullptr;
  uint64_t* o = nullptr;
  (void)rocprim::radix_sort_keys(nullptr, bytes, k, o, (size_t)(nnz > 0 ? nnz : 1), 0u,
                                 (unsigned)bits);
  return align_up(bytes, 256);
}

}  // namespace gs

extern "C" {

size_t gs_segment_sort_workspace_bytes(int64_t nnz, int64_t num_segments, int64_t key_bound) {
  using namespace gs;
  if (nnz < 0 || num_segments < 0) return 0;
  if (native_segment_sort(nnz, key_bound))
    return segsort_workspace_bytes(nnz, num_segments, id_bits(key_bound));
  int key_bits = 0;
  const int bits = packed_bits(num_segments, key_bound, &key_bits);
  if (bits == 0) return segmented_temp_bytes(nnz, num_segments);
  return align_up((size_t)(nnz > 0 ? nnz : 1) * sizeof(uint64_t), 256) + packed_temp_bytes(nnz, bits);
}

// keys_out[seg] = sorted(keys_in[seg]) for every segment of indptr; in and out
// must not alias.  key_bound: every key lies in [0, key_bound) (the number of
// rows, for the row ids of a column); 0 = not known.
// SortIndicesCUDA, src/cuda/sort_indices.cu:11-37.
int gs_segment_sort_i64(const int64_t* indptr, int64_t num_segments,
                        const int64_t* keys_in, int64_t* keys_out, int64_t nnz,
                        int64_t key_bound, void* workspace, size_t workspace_bytes,
                        gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_segments >= 0, "segment_sort: negative size");
  if (nnz == 0 || num_segments == 0) return GS_OK;
  GS_REQUIRE(indptr && keys_in && keys_out, "segment_sort: null pointer");
  GS_REQUIRE(keys_in != keys_out, "segment_sort: in-place sorting is not supported");
  size_t need = gs_segment_sort_workspace_bytes(nnz, num_segments, key_bound);
  if (workspace == nullptr || workspace_bytes < need) {
    set_error("segment_sort workspace too small: %zu < %zu", workspace_bytes, need);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  if (native_segment_sort(nnz, key_bound))
    return segsort_run(indptr, num_segments, keys_in, keys_out, nnz, id_bits(key_bound),
                       workspace, s);
  int key_bits = 0;
  const int bits = packed_bits(num_segments, key_bound, &key_bits);
  if (bits == 0) {
    size_t bytes = workspace_bytes;
    ProfScope ps("segment_sort", s);
    GS_HIP(rocprim::segmented_radix_sort_keys(workspace, bytes, keys_in, keys_out,
                                              (size_t)nnz, (unsigned)num_segments,
                                              indptr, indptr + 1, 0, 64, s));
    return GS_OK;
  }
  uint64_t* packed = (uint64_t*)workspace;
  const size_t packed_bytes = align_up((size_t)nnz * sizeof(uint64_t), 256);
  void* temp = (char*)workspace + packed_bytes;
  size_t temp_bytes = workspace_bytes - packed_bytes;
  const dim3 grid((unsigned)ceil_div(nnz, kBlock));
  GS_LAUNCH("segment_sort_pack", s,
            pack_segment_keys_kernel<<<dim3((unsigned)ceil_div(nnz, kPackTile)), dim3(kBlock), 0,
                                       s>>>(indptr, num_segments, keys_in, nnz, key_bits, packed));
  {
    ProfScope ps("segment_sort", s);
    GS_HIP(rocprim::radix_sort_keys(temp, temp_bytes, packed, (uint64_t*)keys_out, (size_t)nnz,
                                    0u, (unsigned)bits, s));
  }
  GS_LAUNCH("segment_sort_unpack", s,
            unpack_segment_keys_kernel<<<grid, dim3(kBlock), 0, s>>>(keys_out, nnz, key_bits));
  return GS_OK;
}


size_t gs_coo_sort_workspace_bytes(int64_t nnz, int64_t num_major) {
  if (nnz < 0) return 0;
  if (gs::native_coo_sort(nnz, num_major))
    return gs::coosort_workspace_bytes(nnz, gs::id_bits(num_major));
  size_t bytes = 0;
  const int64_t* k = nullptr;
  int64_t* o = nullptr;
  (void)rocprim::radix_sort_pairs(nullptr, bytes, k, o, rocprim::counting_iterator<int64_t>(0), o,
                                  (size_t)(nnz > 0 ? nnz : 1), 0u, (unsigned)gs::id_bits(num_major));
  return gs::align_up(bytes, 256);
}

// Where in the workspace of gs_coo_sort, in bytes, the 32-bit gave-up flag of the
// library's own sort kernels sits for a call of these sizes, or -1 when the call
// is served by rocPRIM, which has none.
int64_t gs_coo_sort_flag_offset(int64_t nnz, int64_t num_major) {
  return gs::native_coo_sort(nnz, num_major) ? 0 : -1;
}

// Stable sort of the edge positions 0..nnz-1 by major[position]: sorted_major
// receives the ids in order, perm the positions.  Only the low bits that ids
// below num_major can have are sorted (COOSort, src/cuda/format_transform.cu:
// 65-84, does the same through cub): three 8-bit passes instead of eight for a
// few million columns.  Ids must lie in [0, num_major).
int gs_coo_sort(const int64_t* major, int64_t nnz, int64_t num_major,
                int64_t* sorted_major, int64_t* perm, void* workspace,
                size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_major >= 0, "coo_sort: negative size");
  if (nnz == 0) return GS_OK;
  GS_REQUIRE(major && sorted_major && perm, "coo_sort: null pointer");
  GS_REQUIRE(major != sorted_major, "coo_sort: in-place sorting is not supported");
  size_t need = gs_coo_sort_workspace_bytes(nnz, num_major);
  if (workspace == nullptr || workspace_bytes < need) {
    set_error("coo_sort workspace too small: %zu < %zu", workspace_bytes, need);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  if (native_coo_sort(nnz, num_major))
    return coosort_run(major, nnz, id_bits(num_major), sorted_major, perm, workspace, s);
  size_t bytes = workspace_bytes;
  ProfScope ps("coo_sort", s);
  GS_HIP(rocprim::radix_sort_pairs(workspace, bytes, major, sorted_major,
                                   rocprim::counting_iterator<int64_t>(0), perm, (size_t)nnz,
                                   0u, (unsigned)id_bits(num_major), s));
  return GS_OK;
}

}  // extern "C"
