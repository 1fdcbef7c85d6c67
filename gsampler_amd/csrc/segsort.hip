// segsort.hip -- the ids of every segment (the row ids of every column) sorted,
// for ids below 2^32 (SortIndicesCUDA, src/cuda/sort_indices.cu:11-37, which
// calls cub's segmented radix sort).
//
// The input is already grouped by segment, so only the ids inside a segment have
// to move, and most segments are short:
//   leaf       a work-group takes the segments that start inside its window of
//              2048 positions and are at most 2048 long (4096 ids at most), and
//              sorts each of them in LDS, 32 bits per id, with a comparator
//              network that works on every segment of the tile at once: one read
//              and one write of the ids
//   partition  a longer segment is split by the next 11 bits of its ids into 2048
//              bins that lie in id order (tiles of 4096 ids: histogram, scan per
//              segment, scatter as contiguous runs); bins of at most 2048 ids are
//              leaves of the next round, longer ones are split again.  After the
//              last bits every bin holds one value and is in place.
// Which segments are long, how many there are and where their bins start stays
// on the device: every launch is sized by a bound and work-groups without work
// leave at once, so the host never waits.
// The leaf pass is bound by the instructions of its network (a segment of n ids
// takes log2(n) (log2(n) + 1) / 2 steps, 66 for 2048), not by memory or by the
// barriers between the steps: sixteen ids per thread in 256-thread work-groups,
// eight tiles to a compute unit, ran 2.5 times slower than eight ids per thread.
#include "common.h"

namespace gs {

constexpr int kSortSmall = 2048;                     // longest segment a leaf sorts
constexpr int kSortTile = 2 * kSortSmall;            // ids a tile holds
constexpr int kSortThreads = 512;
constexpr int kSortItems = kSortTile / kSortThreads; // ids per thread
constexpr int kSplitTile = 4096;                     // ids a work-group of the partition passes takes
constexpr int kSplitThreads = 512;
constexpr int kSplitItems = kSplitTile / kSplitThreads;
constexpr int kDigitBits = 11;
constexpr int kDigitBins = 1 << kDigitBits;
constexpr int kFan = kDigitBins + 1;  // pointer entries of a split segment: its bins, then what lies behind it

// A list of segments: segment j is [ptr[j], ptr[j + 1]), ptr has *n + 1 entries.
// stride == 0: the caller's pointer array.  stride == kFan: entries j * kFan + b,
// b < 2048, are the bins of split segment j; entry j * kFan + 2048 is the gap
// between that segment and the next split one, which is not to be touched.
struct SegList {
  const int64_t* ptr;
  const int64_t* n;
  int stride;
  __device__ __forceinline__ bool is_gap(int64_t j) const {
    return stride != 0 && j % stride == stride - 1;
  }
};

// Number of entries of ptr[0..n) that are below x (ptr non-decreasing), by a
// whole wavefront: 64 probes a round.
__device__ __forceinline__ int64_t wave_count_below(const int64_t* __restrict__ ptr, int64_t n,
                                                    int64_t x) {
  int64_t lo = 0, hi = n;  // entries before lo are below x, entries from hi on are not
  while (lo < hi) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t c = lo + (int64_t)lane_id() * step;
    const bool below = c < hi && ptr[c] < x;
    const int hits = __popcll(__ballot(below));  // `below` is monotone over the lanes
    const int64_t first_not = lo + (int64_t)hits * step;
    if (hits > 0) lo += (int64_t)(hits - 1) * step + 1;
    if (first_not < hi) hi = first_not;
  }
  return lo;
}

__device__ __forceinline__ int bits_for(uint32_t len) {  // smallest k with 2^k >= len
  return len <= 1 ? 0 : 32 - __clz((int)(len - 1));
}

// ------------------------------------------------------------------- leaf
// first[b] = the first segment of the list that starts at or behind position
// b * 2048 (the list's length when none does): where the window of work-group b
// begins in the list.  One thread per window searches the list; the leaf
// work-groups then start with two loads instead of a search of their own.
__global__ __launch_bounds__(kBlock) void segsort_windows_kernel(SegList list, int64_t windows,
                                                                int64_t* __restrict__ first) {
  const int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (b > windows) return;
  const int64_t n = *list.n, x = b * kSortSmall;
  int64_t lo = 0, hi = n;  // entries before lo start before x, entries from hi on do not
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (list.ptr[mid] < x)
      lo = mid + 1;
    else
      hi = mid;
  }
  first[b] = lo;
}

// A segment of at most kRankMax ids needs no network: every id counts the ids
// of its segment that go before it and is written to that place at once.
// 16 KB of LDS per work-group (the segment marks of the set-up share it with the
// ids) and 256 threads let eight tiles share a compute unit: the passes of the
// network are a chain of barriers, and what hides one tile's waits is the
// other tiles.
constexpr uint32_t kRankMax = 32;
static_assert(kSortItems % 8 == 0, "a thread scans whole 16-byte groups of marks");
template <typename SrcT>
__global__ __launch_bounds__(kSortThreads) void segsort_leaf_kernel(
    SegList list, const int64_t* __restrict__ first, const SrcT* __restrict__ src,
    int64_t* __restrict__ dst) {
  __shared__ __align__(16) uint32_t key[kSortTile];
  // during the set-up: at a segment's first id, start << 1 | skip, and where it ends
  uint16_t* mark = reinterpret_cast<uint16_t*>(key);
  uint16_t* end_at = mark + kSortTile;
  __shared__ uint32_t wave_max[kSortThreads / kWave];
  __shared__ int max_phase;
  __shared__ uint32_t tile_end;
  // segments that start inside the window
  const int64_t j_lo = first[blockIdx.x], j_hi = first[blockIdx.x + 1];
  if (j_lo >= j_hi) return;
  const int wave = threadIdx.x / kWave;
  constexpr int kQuads = kSortItems / 8;  // 16-byte groups of marks per thread
  uint4* my_marks = reinterpret_cast<uint4*>(mark) + threadIdx.x * kQuads;
#pragma unroll
  for (int q = 0; q < kQuads; ++q) my_marks[q] = make_uint4(0, 0, 0, 0);
  if (threadIdx.x == 0) {
    max_phase = 0;
    tile_end = 0;
  }
  const int64_t e_lo = list.ptr[j_lo];
  __syncthreads();
  {
    // (the tile's end and the longest network go to LDS once per wavefront: a
    // window of short segments would otherwise send hundreds of atomics to the
    // same two words, which LDS takes one after another)
    uint32_t my_end = 0;
    int my_phase = 0;
    for (int64_t j = j_lo + threadIdx.x; j < j_hi; j += kSortThreads) {
      const int64_t s = list.ptr[j], t = list.ptr[j + 1];
      if (t <= s) continue;
      const uint32_t ls = (uint32_t)(s - e_lo);  // < 2048: s and e_lo lie in the window
      const bool skip = list.is_gap(j) || t - s > kSortSmall;
      mark[ls] = (uint16_t)(ls << 1 | (skip ? 1u : 0u));
      if (!skip) {
        const uint32_t le = (uint32_t)(t - e_lo);  // <= 4096
        end_at[ls] = (uint16_t)le;
        my_end = max(my_end, le);
        if (le - ls > kRankMax) my_phase = max(my_phase, bits_for(le - ls));
      }
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
      my_end = max(my_end, (uint32_t)__shfl_xor((int)my_end, d, kWave));
      my_phase = max(my_phase, __shfl_xor(my_phase, d, kWave));
    }
    if (lane_id() == 0 && my_end != 0) {
      atomicMax(&tile_end, my_end);
      if (my_phase != 0) atomicMax(&max_phase, my_phase);
    }
  }
  __syncthreads();
  const uint32_t count = tile_end;
  if (count == 0) return;  // nothing to sort in this window
  // running maximum of the marks: every id learns where its segment starts
  {
    uint32_t h[kSortItems], run = 0;
#pragma unroll
    for (int q = 0; q < kQuads; ++q) {
      const uint4 v = my_marks[q];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        h[8 * q + 2 * x] = max(w[x] & 0xFFFFu, run);
        h[8 * q + 2 * x + 1] = max(w[x] >> 16, h[8 * q + 2 * x]);
        run = h[8 * q + 2 * x + 1];
      }
    }
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t o = __shfl_up(run, d, kWave);
      if (lane_id() >= d) run = max(run, o);
    }
    if (lane_id() == kWave - 1) wave_max[wave] = run;
    uint32_t before = __shfl_up(run, 1, kWave);
    if (lane_id() == 0) before = 0;
    __syncthreads();
    for (int x = 0; x < wave; ++x) before = max(before, wave_max[x]);
#pragma unroll
    for (int q = 0; q < kSortItems; ++q) h[q] = max(h[q], before);
#pragma unroll
    for (int q = 0; q < kQuads; ++q)
      my_marks[q] = make_uint4(h[8 * q] | h[8 * q + 1] << 16, h[8 * q + 2] | h[8 * q + 3] << 16,
                               h[8 * q + 4] | h[8 * q + 5] << 16, h[8 * q + 6] | h[8 * q + 7] << 16);
  }
  __syncthreads();
  // id i of the tile: segment [lo, lo + len) in tile positions (len == 0: none) and
  // the phases it needs, in one word: lo | len << 12 | need << 25
  uint32_t seg[kSortItems], value[kSortItems];
#pragma unroll
  for (int r = 0; r < kSortItems; ++r) {
    const uint32_t i = r * kSortThreads + threadIdx.x;
    seg[r] = 0;
    value[r] = 0;
    if (i < count) {
      const uint32_t v = mark[i];
      if (!(v & 1u)) {
        const uint32_t lo = v >> 1, hi = end_at[lo];
        if (i < hi) {
          seg[r] = lo | (hi - lo) << 12 | (uint32_t)bits_for(hi - lo) << 25;
          value[r] = (uint32_t)src[e_lo + i];
        }
      }
    }
  }
  __syncthreads();  // the marks have been read: their memory now holds the ids
#pragma unroll
  for (int r = 0; r < kSortItems; ++r)
    if (seg[r] != 0) key[r * kSortThreads + threadIdx.x] = value[r];
  __syncthreads();
  // short segments: place = ids of the segment that are smaller, or equal and earlier
#pragma unroll
  for (int r = 0; r < kSortItems; ++r) {
    const uint32_t lo = seg[r] & 0xFFFu, len = (seg[r] >> 12) & 0x1FFFu;
    if (len == 0 || len > kRankMax) continue;
    const uint32_t il = r * kSortThreads + threadIdx.x - lo;
    uint32_t before = 0;
    for (uint32_t t = 0; t < len; ++t) {
      const uint32_t v = key[lo + t];
      before += (v < value[r] || (v == value[r] && t < il)) ? 1u : 0u;
    }
    dst[e_lo + lo + before] = (int64_t)value[r];
    seg[r] = 0;  // done
  }
  // Longer ones: comparators that only ever put the smaller id first.  Phase k
  // makes sorted runs of 2^k out of runs of 2^(k-1) (mirror step, then halving
  // steps).  A partner past the end of the segment counts as larger than anything.
  const int phases = max_phase;
  for (int k = 1; k <= phases; ++k) {
    for (int step = k - 1; step >= 0; --step) {
      const uint32_t flip = step == k - 1 ? (1u << k) - 1u : 1u << step;
#pragma unroll
      for (int r = 0; r < kSortItems; ++r) {
        if ((uint32_t)k > seg[r] >> 25) continue;  // sorted after as many phases as it needs
        const uint32_t lo = seg[r] & 0xFFFu, len = (seg[r] >> 12) & 0x1FFFu;
        const uint32_t i = r * kSortThreads + threadIdx.x;
        const uint32_t il = i - lo, pl = il ^ flip;
        if (pl > il && pl < len) {
          const uint32_t a = key[i], b = key[lo + pl];
          if (a > b) {
            key[i] = b;
            key[lo + pl] = a;
          }
        }
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int r = 0; r < kSortItems; ++r) {
    const uint32_t i = r * kSortThreads + threadIdx.x;
    if (seg[r] != 0) dst[e_lo + i] = (int64_t)key[i];
  }
}

// ------------------------------------------------------------------- which segments are long
struct LongSegments {
  int64_t* count;   // [1] how many
  int64_t* lo;      // [bound] first id
  int64_t* hi;      // [bound] one past the last id
};

__device__ __forceinline__ bool is_long(const SegList& l, int64_t j, int64_t n) {
  return j < n && !l.is_gap(j) && l.ptr[j + 1] - l.ptr[j] > kSortSmall;
}

// per chunk of `chunk` entries: how many long segments
__global__ __launch_bounds__(kBlock) void segsort_count_long_kernel(SegList list, int chunk,
                                                                    int32_t* __restrict__ chunk_cnt) {
  __shared__ int32_t total;
  const int64_t n = *list.n;
  const int64_t j0 = (int64_t)blockIdx.x * chunk;
  if (j0 >= n) return;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int32_t mine = 0;
  for (int64_t j = j0 + threadIdx.x; j < j0 + chunk; j += kBlock) mine += is_long(list, j, n) ? 1 : 0;
  if (mine) atomicAdd(&total, mine);
  __syncthreads();
  if (threadIdx.x == 0) chunk_cnt[blockIdx.x] = total;
}

// one work-group: chunk counts -> chunk offsets; the number of long segments;
// the size and the last entry of the next round's pointer array
constexpr int kChunkScanThreads = 1024;
__global__ __launch_bounds__(kChunkScanThreads) void segsort_scan_chunks_kernel(
    SegList list, int chunk, const int32_t* __restrict__ chunk_cnt, int64_t* __restrict__ chunk_off,
    int64_t* __restrict__ long_count, int64_t* __restrict__ next_n, int64_t* __restrict__ next_ptr,
    int64_t nnz) {
  __shared__ int64_t smem[kChunkScanThreads / kWave + 1];
  const int64_t n = *list.n;
  const int64_t chunks = ceil_div_dev(n, chunk);
  int64_t carry = 0;
  for (int64_t base = 0; base < chunks; base += kChunkScanThreads) {
    const int64_t c = base + threadIdx.x;
    const int64_t v = c < chunks ? chunk_cnt[c] : 0;
    int64_t total;
    const int64_t at = carry + block_exclusive_sum<int64_t, kChunkScanThreads>(v, smem, &total);
    if (c < chunks) chunk_off[c] = at;
    carry += total;
  }
  if (threadIdx.x == 0) {
    *long_count = carry;
    *next_n = carry * kFan;
    next_ptr[carry * kFan] = nnz;
  }
}

// per chunk: the long segments in order
__global__ __launch_bounds__(kBlock) void segsort_list_long_kernel(
    SegList list, int chunk, const int64_t* __restrict__ chunk_off, LongSegments out) {
  __shared__ int32_t smem[kBlock / kWave + 1];
  const int64_t n = *list.n;
  const int64_t j0 = (int64_t)blockIdx.x * chunk;
  if (j0 >= n) return;
  int64_t at = chunk_off[blockIdx.x];
  for (int64_t base = 0; base < chunk; base += kBlock) {
    const int64_t j = j0 + base + threadIdx.x;
    const bool yes = base + threadIdx.x < chunk && is_long(list, j, n);
    int32_t total;
    const int32_t rank = block_exclusive_sum<int32_t>(yes ? 1 : 0, smem, &total);
    if (yes) {
      out.lo[at + rank] = list.ptr[j];
      out.hi[at + rank] = list.ptr[j + 1];
    }
    at += total;
  }
}

__global__ __launch_bounds__(kBlock) void segsort_zero_kernel(const int64_t* __restrict__ long_count,
                                                             uint32_t* __restrict__ cnt) {
  const int64_t words = *long_count * kDigitBins;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < words;
       i += (int64_t)gridDim.x * kBlock)
    cnt[i] = 0;
}

// ------------------------------------------------------------------- partition
// The long segments that a tile of positions [t0, t1) meets, one after the
// other (a few at most): `first` is the first whose end lies behind t0.
__device__ __forceinline__ int64_t first_long_behind(const LongSegments& s, int64_t count,
                                                     int64_t t0, int64_t* slot) {
  if (threadIdx.x < kWave) {
    const int64_t c = wave_count_below(s.hi, count, t0 + 1);  // ends at or before t0
    if (lane_id() == 0) *slot = c;
  }
  __syncthreads();
  return *slot;
}

template <typename SrcT>
__global__ __launch_bounds__(kSplitThreads) void segsort_hist_kernel(
    const SrcT* __restrict__ src, int64_t nnz, LongSegments segs, int shift,
    uint32_t* __restrict__ cnt) {
  __shared__ uint32_t hist[kDigitBins];
  __shared__ int64_t slot;
  const int64_t count = *segs.count;
  const int64_t t0 = (int64_t)blockIdx.x * kSplitTile;
  if (count == 0 || t0 >= nnz) return;
  const int64_t t1 = t0 + kSplitTile < nnz ? t0 + kSplitTile : nnz;
  for (int64_t s = first_long_behind(segs, count, t0, &slot); s < count; ++s) {
    const int64_t lo = segs.lo[s], hi = segs.hi[s];
    if (lo >= t1) break;
    const int64_t a = lo > t0 ? lo : t0, b = hi < t1 ? hi : t1;
    for (int i = threadIdx.x; i < kDigitBins; i += kSplitThreads) hist[i] = 0;
    __syncthreads();
    for (int64_t e = a + threadIdx.x; e < b; e += kSplitThreads)
      atomicAdd(&hist[((uint32_t)src[e] >> shift) & (kDigitBins - 1)], 1u);
    __syncthreads();
    for (int i = threadIdx.x; i < kDigitBins; i += kSplitThreads) {
      const uint32_t c = hist[i];
      if (c) atomicAdd(&cnt[s * kDigitBins + i], c);
    }
    __syncthreads();
  }
}

// per long segment: bin counts -> where every bin starts (the next round's
// pointer entries); the counters start again at zero as the scatter's cursors
__global__ __launch_bounds__(kBlock) void segsort_bins_kernel(LongSegments segs,
                                                             uint32_t* __restrict__ cnt,
                                                             int64_t* __restrict__ next_ptr) {
  __shared__ uint32_t smem[kBlock / kWave + 1];
  const int64_t s = blockIdx.x;
  if (s >= *segs.count) return;
  constexpr int kPer = kDigitBins / kBlock;
  uint32_t* mine = cnt + s * kDigitBins + threadIdx.x * kPer;
  uint32_t c[kPer], sum = 0;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    c[i] = mine[i];
    sum += c[i];
    mine[i] = 0;
  }
  uint32_t total;
  uint32_t run = block_exclusive_sum<uint32_t>(sum, smem, &total);
  const int64_t lo = segs.lo[s];
  int64_t* out = next_ptr + s * kFan + threadIdx.x * kPer;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    out[i] = lo + run;
    run += c[i];
  }
  if (threadIdx.x == 0) next_ptr[s * kFan + kDigitBins] = segs.hi[s];
}

template <typename SrcT, typename DstT>
__global__ __launch_bounds__(kSplitThreads) void segsort_scatter_kernel(
    const SrcT* __restrict__ src, DstT* __restrict__ dst, int64_t nnz, LongSegments segs,
    int shift, uint32_t* cursor, const int64_t* __restrict__ next_ptr) {
  __shared__ uint32_t hist[kDigitBins];    // counts, then where a bin starts in the tile
  __shared__ uint32_t run_at[kDigitBins];  // where the tile's run of a bin goes, from the segment's first id
  __shared__ uint32_t stage[kSplitTile];
  __shared__ uint32_t scan_smem[kSplitThreads / kWave + 1];
  __shared__ int64_t slot;
  const int64_t count = *segs.count;
  const int64_t t0 = (int64_t)blockIdx.x * kSplitTile;
  if (count == 0 || t0 >= nnz) return;
  const int64_t t1 = t0 + kSplitTile < nnz ? t0 + kSplitTile : nnz;
  constexpr int kPer = kDigitBins / kSplitThreads;
  for (int64_t s = first_long_behind(segs, count, t0, &slot); s < count; ++s) {
    const int64_t lo = segs.lo[s], hi = segs.hi[s];
    if (lo >= t1) break;
    const int64_t a = lo > t0 ? lo : t0, b = hi < t1 ? hi : t1;
    const uint32_t m = (uint32_t)(b - a);
    for (int i = threadIdx.x; i < kDigitBins; i += kSplitThreads) hist[i] = 0;
    __syncthreads();
    uint32_t k[kSplitItems], place[kSplitItems];
#pragma unroll
    for (int r = 0; r < kSplitItems; ++r) {
      const int64_t e = a + r * kSplitThreads + threadIdx.x;
      k[r] = (uint32_t)src[e < b ? e : b - 1];
    }
#pragma unroll
    for (int r = 0; r < kSplitItems; ++r)
      if (a + r * kSplitThreads + threadIdx.x < b)
        place[r] = atomicAdd(&hist[(k[r] >> shift) & (kDigitBins - 1)], 1u);
    __syncthreads();
    {
      const uint32_t bin0 = threadIdx.x * kPer;
      uint32_t c[kPer], sum = 0;
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        c[i] = hist[bin0 + i];
        sum += c[i];
      }
      uint32_t total;
      uint32_t run = block_exclusive_sum<uint32_t, kSplitThreads>(sum, scan_smem, &total);
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        hist[bin0 + i] = run;
        run += c[i];
        if (c[i]) {
          const uint32_t taken = atomicAdd(&cursor[s * kDigitBins + bin0 + i], c[i]);
          run_at[bin0 + i] = (uint32_t)(next_ptr[s * kFan + bin0 + i] - lo) + taken;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSplitItems; ++r)
      if (a + r * kSplitThreads + threadIdx.x < b)
        stage[hist[(k[r] >> shift) & (kDigitBins - 1)] + place[r]] = k[r];
    __syncthreads();
    for (uint32_t j = threadIdx.x; j < m; j += kSplitThreads) {
      const uint32_t v = stage[j];
      const uint32_t bin = (v >> shift) & (kDigitBins - 1);
      dst[lo + run_at[bin] + (j - hist[bin])] = (DstT)v;
    }
    __syncthreads();
  }
}

__global__ void segsort_init_kernel(int64_t* n_dev, int64_t num_segments) { *n_dev = num_segments; }

// ------------------------------------------------------------------- host
struct SegSortWs {
  int64_t* n;          // [kMaxLevels + 1] segments of every round's list
  int64_t* long_count; // [kMaxLevels]
  int32_t* chunk_cnt;
  int64_t* chunk_off;
  int64_t* long_lo;
  int64_t* long_hi;
  uint32_t* cnt;
  int64_t* ptr[2];
  int64_t* window;     // [windows + 1] first segment of every leaf window
  uint32_t* tmp[2];
  int64_t long_bound, chunk_bound;
  size_t total;
};
constexpr int kMaxLevels = 3;  // 32 bits, 11 at a time

static SegSortWs carve_segsort(void* ws, int64_t nnz, int64_t num_segments, int levels) {
  Carver c(ws);
  SegSortWs w;
  // a long segment has more than kSortSmall ids
  w.long_bound = nnz / (kSortSmall + 1) + 1;
  const int64_t chunks0 = ceil_div(num_segments > 0 ? num_segments : 1, kSortSmall);
  w.chunk_bound = chunks0 > w.long_bound ? chunks0 : w.long_bound;
  w.n = c.take<int64_t>(kMaxLevels + 1);
  w.long_count = c.take<int64_t>(kMaxLevels);
  w.chunk_cnt = c.take<int32_t>((size_t)w.chunk_bound);
  w.chunk_off = c.take<int64_t>((size_t)w.chunk_bound);
  w.long_lo = c.take<int64_t>((size_t)w.long_bound);
  w.long_hi = c.take<int64_t>((size_t)w.long_bound);
  w.cnt = c.take<uint32_t>((size_t)w.long_bound * kDigitBins);
  for (int i = 0; i < 2; ++i) w.ptr[i] = c.take<int64_t>((size_t)w.long_bound * kFan + 1);
  w.window = c.take<int64_t>((size_t)ceil_div(nnz > 0 ? nnz : 1, kSortSmall) + 2);
  const size_t ids = (size_t)(nnz > 0 ? nnz : 1);
  w.tmp[0] = levels >= 2 ? c.take<uint32_t>(ids) : nullptr;
  w.tmp[1] = levels >= 3 ? c.take<uint32_t>(ids) : nullptr;
  w.total = c.total();
  return w;
}

int segsort_levels(int key_bits) { return (key_bits + kDigitBits - 1) / kDigitBits; }

size_t segsort_workspace_bytes(int64_t nnz, int64_t num_segments, int key_bits) {
  return carve_segsort(nullptr, nnz, num_segments, segsort_levels(key_bits)).total;
}

// keys_out[segment] = sorted(keys_in[segment]) for ids below 2^key_bits, key_bits <= 32,
// nnz < 2^32.
int segsort_run(const int64_t* indptr, int64_t num_segments, const int64_t* keys_in,
                int64_t* keys_out, int64_t nnz, int key_bits, void* workspace,
                hipStream_t s) {
  const int levels = segsort_levels(key_bits);
  const SegSortWs w = carve_segsort(workspace, nnz, num_segments, levels);
  const dim3 leaf_grid((unsigned)ceil_div(nnz, kSortSmall));
  const dim3 tile_grid((unsigned)ceil_div(nnz, kSplitTile));
  GS_LAUNCH("segsort_init", s, segsort_init_kernel<<<dim3(1), dim3(1), 0, s>>>(w.n, num_segments));
  SegList list{indptr, w.n, 0};
  const int64_t windows = ceil_div(nnz, kSortSmall);
  const dim3 window_grid((unsigned)ceil_div(windows + 1, kBlock));
  GS_LAUNCH("segsort_windows", s,
            segsort_windows_kernel<<<window_grid, dim3(kBlock), 0, s>>>(list, windows, w.window));
  GS_LAUNCH("segsort_leaf", s,
            segsort_leaf_kernel<int64_t><<<leaf_grid, dim3(kSortThreads), 0, s>>>(
                list, w.window, keys_in, keys_out));
  const uint32_t* src32 = nullptr;
  for (int level = 0; level < levels; ++level) {
    const int chunk = level == 0 ? kSortSmall : kFan;
    const dim3 chunk_grid(
        (unsigned)(level == 0 ? ceil_div(num_segments, kSortSmall) : w.long_bound));
    int64_t* next_ptr = w.ptr[level % 2];
    const LongSegments segs{w.long_count + level, w.long_lo, w.long_hi};
    GS_LAUNCH("segsort_find_long", s,
              segsort_count_long_kernel<<<chunk_grid, dim3(kBlock), 0, s>>>(list, chunk,
                                                                           w.chunk_cnt));
    GS_LAUNCH("segsort_find_long", s,
              segsort_scan_chunks_kernel<<<dim3(1), dim3(kChunkScanThreads), 0, s>>>(
                  list, chunk, w.chunk_cnt, w.chunk_off, w.long_count + level, w.n + level + 1,
                  next_ptr, nnz));
    GS_LAUNCH("segsort_find_long", s,
              segsort_list_long_kernel<<<chunk_grid, dim3(kBlock), 0, s>>>(list, chunk,
                                                                          w.chunk_off, segs));
    GS_LAUNCH("segsort_find_long", s,
              segsort_zero_kernel<<<dim3(1024), dim3(kBlock), 0, s>>>(segs.count, w.cnt));
    const int shift = key_bits > kDigitBits * (level + 1) ? key_bits - kDigitBits * (level + 1) : 0;
    const bool last = level == levels - 1;
    uint32_t* dst32 = last ? nullptr : w.tmp[level % 2];
    if (level == 0)
      GS_LAUNCH("segsort_hist", s,
                segsort_hist_kernel<int64_t><<<tile_grid, dim3(kSplitThreads), 0, s>>>(
                    keys_in, nnz, segs, shift, w.cnt));
    else
      GS_LAUNCH("segsort_hist", s,
                segsort_hist_kernel<uint32_t><<<tile_grid, dim3(kSplitThreads), 0, s>>>(
                    src32, nnz, segs, shift, w.cnt));
    GS_LAUNCH("segsort_bins", s,
              segsort_bins_kernel<<<dim3((unsigned)w.long_bound), dim3(kBlock), 0, s>>>(
                  segs, w.cnt, next_ptr));
#define GS_SCATTER(SrcT, DstT, from, to)                                                   \
  GS_LAUNCH("segsort_scatter", s,                                                          \
            segsort_scatter_kernel<SrcT, DstT><<<tile_grid, dim3(kSplitThreads), 0, s>>>(  \
                from, to, nnz, segs, shift, w.cnt, next_ptr))
    if (level == 0 && last)
      GS_SCATTER(int64_t, int64_t, keys_in, keys_out);
    else if (level == 0)
      GS_SCATTER(int64_t, uint32_t, keys_in, dst32);
    else if (last)
      GS_SCATTER(uint32_t, int64_t, src32, keys_out);
    else
      GS_SCATTER(uint32_t, uint32_t, src32, dst32);
#undef GS_SCATTER
    if (last) break;
    list = SegList{next_ptr, w.n + level + 1, kFan};
    GS_LAUNCH("segsort_windows", s,
              segsort_windows_kernel<<<window_grid, dim3(kBlock), 0, s>>>(list, windows, w.window));
    GS_LAUNCH("segsort_leaf", s,
              segsort_leaf_kernel<uint32_t><<<leaf_grid, dim3(kSortThreads), 0, s>>>(
                  list, w.window, dst32, keys_out));
    src32 = dst32;
  }
  return GS_OK;
}

}  // namespace gs
