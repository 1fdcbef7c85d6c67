// listlabels.hip -- frontier and labels of a matrix whose rows are positions
// in a short list of ids (what a row slice by a few hundred picked ids leaves
// behind): one work-group, everything in LDS.
//
// Every edge of local row l carries the same key list_ids[l], so the listed
// ids, ordered by the first edge that uses each, give the same first-occurrence
// frontier as the edges themselves would (seeds first); the labels of the
// edges are then two gathers by local row and by column.
#include "common.h"

namespace gs {

constexpr int kLabelThreads = 1024;
constexpr int kLabelMaxKeys = GS_LIST_LABELS_MAX_KEYS;
constexpr int kLabelSlots = 2 * kLabelMaxKeys;  // open addressing, at most half full
constexpr int kLabelIdBits = 12;                // list positions in the low bits of a sort key
constexpr uint32_t kLabelEmpty = 0xFFFFFFFFu;
static_assert(kLabelMaxKeys <= (1 << kLabelIdBits), "a list position must fit the sort key");
static_assert(kLabelMaxKeys == 2 * kLabelThreads, "two keys per thread");

__device__ __forceinline__ uint32_t label_slot(int64_t key) {
  return (uint32_t)(((uint64_t)key * 0x9E3779B97F4A7C15ull) >> 40) & (kLabelSlots - 1);
}

__global__ __launch_bounds__(kLabelThreads) void list_labels_kernel(
    const int64_t* __restrict__ seeds, int num_seeds, const int64_t* __restrict__ list_ids,
    const int64_t* __restrict__ first_pos, int num_ids, int64_t* __restrict__ out_frontier,
    int64_t* __restrict__ out_count, int64_t* out_count_mirror,
    int64_t* __restrict__ out_list_label, int64_t* __restrict__ out_seed_label) {
  __shared__ uint64_t order[kLabelMaxKeys];   // (first position, list position), sorted
  __shared__ int64_t keys[kLabelMaxKeys];     // seeds ++ used list ids in order of first use
  __shared__ uint32_t table[kLabelSlots];     // slot -> smallest position of the key that owns it
  __shared__ int32_t rank[kLabelMaxKeys];     // rank of a first occurrence
  __shared__ int32_t wave_sum[kLabelThreads / kWave];
  __shared__ int used_ids;
  const int t = threadIdx.x;

  // 1. list positions by first use; ids that no edge uses sort to the end
  int m = 1;
  while (m < num_ids) m <<= 1;
  if (t == 0) used_ids = 0;
  for (int i = t; i < m; i += kLabelThreads) {
    uint64_t k = ~0ull;
    if (i < num_ids) {
      const int64_t f = first_pos[i];
      const uint64_t when = f == INT64_MAX ? (1ull << 51) : (uint64_t)f;
      k = (when << kLabelIdBits) | (uint64_t)i;
    }
    order[i] = k;
  }
  for (int i = t; i < kLabelSlots; i += kLabelThreads) table[i] = kLabelEmpty;
  __syncthreads();
  for (int k = 2; k <= m; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = t; i < m; i += kLabelThreads) {
        const int other = i ^ j;
        if (other > i) {
          const uint64_t a = order[i], b = order[other];
          const bool up = (i & k) == 0;
          if ((a > b) == up) {
            order[i] = b;
            order[other] = a;
          }
        }
      }
      __syncthreads();
    }
  int mine_used = 0;
  for (int i = t; i < num_ids; i += kLabelThreads)
    mine_used += (order[i] >> kLabelIdBits) < (1ull << 51);
  if (mine_used) atomicAdd(&used_ids, mine_used);
  __syncthreads();
  const int n = num_seeds + used_ids;

  // 2. keys, and the smallest position of every distinct key
  for (int i = t; i < n; i += kLabelThreads)
    keys[i] = i < num_seeds
                  ? seeds[i]
                  : list_ids[order[i - num_seeds] & ((1ull << kLabelIdBits) - 1ull)];
  __syncthreads();
  for (int i = t; i < n; i += kLabelThreads) {
    const int64_t key = keys[i];
    uint32_t slot = label_slot(key);
    while (true) {
      uint32_t cur = table[slot];
      if (cur == kLabelEmpty) {
        cur = atomicCAS(&table[slot], kLabelEmpty, (uint32_t)i);
        if (cur == kLabelEmpty) break;  // the slot is this key's now
      }
      if (keys[cur] == key) {
        atomicMin(&table[slot], (uint32_t)i);
        break;
      }
      slot = (slot + 1) & (kLabelSlots - 1);
    }
  }
  __syncthreads();

  // 3. first occurrences in order -> frontier; two consecutive positions per thread
  int first_at[2], flags = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = 2 * t + j;
    first_at[j] = -1;
    if (i >= n) continue;
    const int64_t key = keys[i];
    uint32_t slot = label_slot(key);
    while (keys[table[slot]] != key) slot = (slot + 1) & (kLabelSlots - 1);
    first_at[j] = (int)table[slot];
    flags |= (first_at[j] == i) << j;
  }
  const int own = (flags & 1) + (flags >> 1);
  int incl = own;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int o = __shfl_up(incl, d, kWave);
    if (lane_id() >= d) incl += o;
  }
  if (lane_id() == kWave - 1) wave_sum[t / kWave] = incl;
  __syncthreads();
  int before = incl - own, total = 0;
  for (int w = 0; w < kLabelThreads / kWave; ++w) {
    if (w < t / kWave) before += wave_sum[w];
    total += wave_sum[w];
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = 2 * t + j;
    if (!((flags >> j) & 1)) continue;
    const int r = before + (j == 1 ? (flags & 1) : 0);
    rank[i] = r;
    out_frontier[r] = keys[i];
  }
  if (t == 0) {
    if (out_count) *out_count = total;
    if (out_count_mirror) *out_count_mirror = total;
  }
  __syncthreads();

  // 4. labels
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = 2 * t + j;
    if (i >= n) continue;
    const int64_t label = rank[first_at[j]];
    if (i < num_seeds)
      out_seed_label[i] = label;
    else
      out_list_label[order[i - num_seeds] & ((1ull << kLabelIdBits) - 1ull)] = label;
  }
  for (int i = used_ids + t; i < num_ids; i += kLabelThreads)  // ids that no edge uses
    out_list_label[order[i] & ((1ull << kLabelIdBits) - 1ull)] = 0;
}

}  // namespace gs

extern "C" int gs_list_labels(const int64_t* seeds, int64_t num_seeds, const int64_t* list_ids,
                              const int64_t* first_pos, int64_t num_ids,
                              int64_t* out_frontier, int64_t* out_count,
                              int64_t* out_count_mirror, int64_t* out_list_label,
                              int64_t* out_seed_label, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_seeds >= 0 && num_ids >= 0, "list_labels: negative size");
  GS_REQUIRE(num_seeds + num_ids <= kLabelMaxKeys,
             "list_labels: %lld seeds + %lld listed ids exceed %d keys; use gs_unique_count / "
             "gs_unique_relabel",
             (long long)num_seeds, (long long)num_ids, kLabelMaxKeys);
  GS_REQUIRE(num_seeds == 0 || (seeds && out_seed_label), "list_labels: null seeds");
  GS_REQUIRE(num_ids == 0 || (list_ids && first_pos && out_list_label),
             "list_labels: null list");
  GS_REQUIRE(num_seeds + num_ids == 0 || out_frontier, "list_labels: null out_frontier");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("list_labels", s,
            list_labels_kernel<<<dim3(1), dim3(kLabelThreads), 0, s>>>(
                seeds, (int)num_seeds, list_ids, first_pos, (int)num_ids, out_frontier,
                out_count, out_count_mirror, out_list_label, out_seed_label));
  return GS_OK;
}
