// common.h -- shared device/host helpers for the gfx950 sampling kernels.
// wave64 everywhere: a wavefront is 64 lanes, sub-wave "groups" are power-of-two
// slices of one wavefront.
#ifndef GSAMPLER_CSRC_COMMON_H_
#define GSAMPLER_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/gsampler_hip.h"

namespace gs {

// ------------------------------------------------------------ error plumbing
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what, const char* file, int line);

#define GS_REQUIRE(cond, ...)     \
  do {                            \
    if (!(cond)) {                \
      gs::set_error(__VA_ARGS__); \
      return GS_ERR_INVALID;      \
    }                             \
  } while (0)

#define GS_HIP(expr)                                                    \
  do {                                                                  \
    hipError_t e__ = (expr);                                            \
    if (e__ != hipSuccess) return gs::hip_fail(e__, #expr, __FILE__, __LINE__); \
  } while (0)

// Call right after a kernel launch.
#define GS_LAUNCH_CHECK() GS_HIP(hipGetLastError())

inline hipStream_t as_stream(gs_stream_t s) { return (hipStream_t)s; }

// Compute units of the current device (256 on the part this is written for).
int num_compute_units();

// Optional per-kernel timing (gs_profile_*): while enabled, every launch that
// sits inside a ProfScope is bracketed by two HIP events on its own stream.
bool profile_enabled();
void profile_begin(const char* name, hipStream_t stream);
void profile_end(hipStream_t stream);
struct ProfScope {
  hipStream_t stream;
  bool on;
  ProfScope(const char* name, hipStream_t s) : stream(s), on(profile_enabled()) {
    if (on) profile_begin(name, s);
  }
  ~ProfScope() {
    if (on) profile_end(stream);
  }
};
// Usage: GS_LAUNCH("name", stream, kernel<<<grid, block, 0, stream>>>(args));
#define GS_LAUNCH(name, stream, ...)   \
  do {                                 \
    {                                  \
      gs::ProfScope ps__(name, stream); \
      __VA_ARGS__;                     \
    }                                  \
    GS_LAUNCH_CHECK();                 \
  } while (0)

constexpr int kWave = 64;
constexpr int kBlock = 256;  // 4 waves; the default block for flat kernels

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__device__ __forceinline__ int64_t ceil_div_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Carves aligned sub-buffers out of a caller-supplied workspace.
struct Carver {
  char* base;
  size_t used;
  explicit Carver(void* p) : base((char*)p), used(0) {}
  template <typename T>
  T* take(size_t count) {
    used = align_up(used, 256);
    T* r = (T*)(base ? base + used : nullptr);
    used += count * sizeof(T);
    return r;
  }
  size_t total() const { return align_up(used, 256); }
};

// ------------------------------------------------------------------- Philox
// Philox4x32-10 (Salmon et al., SC'11).  One call yields four 32-bit words.
struct PhiloxKey {
  uint32_t k0, k1;
};

__host__ __device__ inline PhiloxKey make_key(uint64_t seed, uint64_t call_id) {
  uint64_t k = seed + call_id * 0x9E3779B97F4A7C15ull;
  PhiloxKey r;
  r.k0 = (uint32_t)k;
  r.k1 = (uint32_t)(k >> 32);
  return r;
}

struct Words4 {
  uint32_t x, y, z, w;
};

__device__ __forceinline__ Words4 philox(PhiloxKey key, uint64_t pos,
                                         uint64_t draw) {
  uint32_t c0 = (uint32_t)draw, c1 = (uint32_t)(draw >> 32);
  uint32_t c2 = (uint32_t)pos, c3 = (uint32_t)(pos >> 32);
  uint32_t k0 = key.k0, k1 = key.k1;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return Words4{c0, c1, c2, c3};
}

// Integer in [0, n): floor(r64 * n / 2^64) with r64 = w1:w0.
__device__ __forceinline__ uint64_t philox_bounded(PhiloxKey key, uint64_t pos,
                                                   uint64_t draw, uint64_t n) {
  Words4 w = philox(key, pos, draw);
  uint64_t r = ((uint64_t)w.y << 32) | w.x;
  return __umul64hi(r, n);
}

// ------------------------------------------------------------- wave helpers
__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

// The first active lane's value, in every lane.
__device__ __forceinline__ int64_t wave_uniform_first(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Inclusive scan across the 64 lanes of a wavefront.
template <typename T>
__device__ __forceinline__ T wave_inclusive_sum(T v) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    T o = __shfl_up(v, d, kWave);
    if (lane_id() >= d) v += o;
  }
  return v;
}

// Exclusive block scan for blocks of kThreads threads.  `total` receives the
// block sum in every thread.  smem must hold kThreads / kWave + 1 elements.
template <typename T, int kThreads = kBlock>
__device__ __forceinline__ T block_exclusive_sum(T v, T* smem, T* total) {
  const int wave = threadIdx.x / kWave;
  T inc = wave_inclusive_sum(v);
  if (lane_id() == kWave - 1) smem[wave] = inc;
  __syncthreads();
  T base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kThreads / kWave; ++w) {
    T s = smem[w];
    if (w < wave) base += s;
    sum += s;
  }
  __syncthreads();
  *total = sum;
  return base + inc - v;
}

// Largest b in [0, n) with ptr[b] <= x, for a non-decreasing ptr[0..n] whose
// first element is <= x (segment lookup in a [n+1] offsets array).
__device__ __forceinline__ int64_t segment_of(const int64_t* ptr, int64_t n,
                                              int64_t x) {
  int64_t lo = 0, hi = n;  // answer in [lo, hi)
  while (hi - lo > 1) {
    int64_t mid = (lo + hi) >> 1;
    if (ptr[mid] <= x)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

// The same look-up by a whole wavefront, 64 probes a round (three rounds for
// 2^18 segments where the one-lane search takes eighteen dependent loads).
__device__ __forceinline__ int64_t wave_segment_of(const int64_t* __restrict__ ptr, int64_t n,
                                                   int64_t x) {
  int64_t lo = 0, hi = n;  // ptr[lo] <= x; hi == n or ptr[hi] > x
  while (hi - lo > 1) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t c = lo + (int64_t)(lane_id() + 1) * step;
    const bool ok = c < hi && ptr[c] <= x;
    const int hits = __popcll(__ballot(ok));  // ok is monotone over the lanes
    const int64_t next_hi = lo + (int64_t)(hits + 1) * step;
    lo += (int64_t)hits * step;
    if (next_hi < hi) hi = next_hi;
  }
  return lo;
}

// Segments that a tile of consecutive positions [p0, p_last] touches.  The two
// look-ups run once per wavefront on the scalar unit (p0 and p_last are the
// same in every lane); a position of the tile is then searched only among the
// segments in between, and not at all when one segment covers the tile.
struct SegmentSpan {
  int64_t lo, hi;
  __device__ __forceinline__ int64_t segment_at(const int64_t* __restrict__ ptr,
                                                int64_t p) const {
    return lo == hi ? lo : lo + segment_of(ptr + lo, hi - lo + 1, p);
  }
};
__device__ __forceinline__ SegmentSpan segment_span(const int64_t* __restrict__ ptr, int64_t n,
                                                    int64_t p0, int64_t p_last) {
  SegmentSpan s;
  s.lo = segment_of(ptr, n, wave_uniform_first(p0));
  s.hi = segment_of(ptr, n, wave_uniform_first(p_last));
  return s;
}

// What a sampler stores as the column of an edge: the column's position among
// the call's columns or, with the offsets of the call's batches of columns, its
// position inside its batch -- which is the label the column gets in a block
// whose batch has distinct seeds, so that the relabel pass has nothing left to do
// for the column side.
struct ColumnLabels {
  const int64_t* batch_ptr;  // [num_batches + 1], null: positions in the call
  int64_t num_batches;
  __device__ __forceinline__ int64_t of(int64_t item) const {
    return batch_ptr ? item - batch_ptr[segment_of(batch_ptr, num_batches, item)] : item;
  }
  // The same for a wavefront whose lanes hold neighbouring columns, the first of
  // them `wave_first` (the same value in every lane): the batch of that column is
  // searched once, on the scalar unit, and a lane walks on from there -- nearly
  // always not at all.
  __device__ __forceinline__ int64_t of_near(int64_t item, int64_t wave_first) const {
    if (batch_ptr == nullptr) return item;
    int64_t b = segment_of(batch_ptr, num_batches, wave_uniform_first(wave_first));
    while (b + 1 < num_batches && batch_ptr[b + 1] <= item) ++b;
    return item - batch_ptr[b];
  }
};

// A column slice that is not written out.  Edge v of the slice A[:, cols] is
// edge  indptr[cols[c]] + (v - sub_indptr[c])  of the parent, where c is the
// position with sub_indptr[c] <= v < sub_indptr[c + 1] (sub_indptr = the
// exclusive scan of the picked columns' degrees).  key_offset[c], when given, is
// added to the ids of column c's edges (ids of a super-batch are told apart as
// id + batch * stride).  A view with sub_indptr == nullptr is no view: edge v is
// edge v of the arrays at hand.
struct SliceView {
  const int64_t* sub_indptr;
  const int64_t* cols;
  const int64_t* indptr;
  const int64_t* key_offset;
  int64_t n;
  __device__ __forceinline__ bool on() const { return sub_indptr != nullptr; }

  // A run of consecutive slice edges [first, last], the same for every lane of
  // the wavefront: the columns it touches are looked up once, on the scalar
  // unit.  Columns worth slicing are long, so a run nearly always lies inside
  // one column or across the border of two neighbours: an edge's place in the
  // parent is then its number plus one of two distances, chosen by which side
  // of the border it is on, and nothing is searched or loaded per edge.  A run
  // over up to 64 columns keeps one column per lane (where it starts inside the
  // run, its distance, its offset) and an edge finds its column by a search over
  // the lanes with shuffles; only beyond that does an edge search the pointer.
  struct Run {
    SegmentSpan span;
    int64_t first;            // first edge of the run
    int64_t split;            // first edge of the second column (none: beyond every edge)
    int64_t shift[2], offset[2];
    int count;                // columns held by the lanes (0: none are)
    int32_t lane_start;       // this lane's column: first edge, relative to `first`, not below 0
    int64_t lane_shift, lane_offset;
    // At most two neighbouring columns.  Callers branch on this once per run,
    // around their whole loop over the run's edges, not per edge: a branch
    // between a load and its use keeps the loads of an unrolled loop from being
    // in flight together.
    __device__ __forceinline__ bool near() const { return span.hi - span.lo <= 1; }
    // for near() runs
    __device__ __forceinline__ int64_t place(int64_t v) const {
      return v + (v < split ? shift[0] : shift[1]);
    }
    __device__ __forceinline__ int64_t id_offset(int64_t v) const {
      return v < split ? offset[0] : offset[1];
    }
    __device__ __forceinline__ int64_t column(int64_t v) const {
      return v < split ? span.lo : span.hi;
    }
  };
  // Every lane of the wavefront must call this, with the same arguments.
  __device__ __forceinline__ Run run(int64_t first, int64_t last) const {
    Run r;
    // the column of the first edge by a search; the last edge is nearly always
    // in the same column, which one more look at the pointer tells
    const int64_t first_u = wave_uniform_first(first), last_u = wave_uniform_first(last);
    r.first = first_u;
    r.span.lo = segment_of(sub_indptr, n, first_u);
    r.span.hi = r.span.lo;
    if (sub_indptr[r.span.lo + 1] <= last_u)
      r.span.hi = r.span.lo + segment_of(sub_indptr + r.span.lo, n - r.span.lo, last_u);
    r.split = INT64_MAX;
    r.shift[0] = r.shift[1] = r.offset[0] = r.offset[1] = 0;
    r.count = 0;
    r.lane_start = 0;
    r.lane_shift = r.lane_offset = 0;
    if (r.near()) {
      r.shift[0] = indptr[cols[r.span.lo]] - sub_indptr[r.span.lo];
      if (key_offset) r.offset[0] = key_offset[r.span.lo];
      if (r.span.hi != r.span.lo) {
        r.split = sub_indptr[r.span.hi];
        r.shift[1] = indptr[cols[r.span.hi]] - r.split;
        if (key_offset) r.offset[1] = key_offset[r.span.hi];
      }
    } else if (r.span.hi - r.span.lo < kWave) {
      r.count = (int)(r.span.hi - r.span.lo) + 1;
      const int64_t c = r.span.lo + (lane_id() < r.count ? lane_id() : r.count - 1);
      const int64_t start = sub_indptr[c];
      r.lane_start = start > first_u ? (int32_t)(start - first_u) : 0;
      r.lane_shift = indptr[cols[c]] - start;
      if (key_offset) r.lane_offset = key_offset[c];
    }
    return r;
  }
  // Position in the parent of edge v of a run that is not near(): *col = its
  // column position, *offset = what to add to its id.  Every lane of the
  // wavefront must call this together (it shuffles), with v inside the run.
  __device__ __forceinline__ int64_t position(const Run& r, int64_t v, int64_t* col,
                                              int64_t* offset) const {
    if (r.count > 0) {  // the same in every lane
      const int32_t x = (int32_t)(v - r.first);
      int i = 0;  // the last column that starts at or before the edge
#pragma unroll
      for (int step = kWave / 2; step >= 1; step >>= 1) {
        const int probe = i + step;
        const int32_t s = __shfl(r.lane_start, probe < r.count ? probe : r.count - 1, kWave);
        i = (probe < r.count && s <= x) ? probe : i;
      }
      *col = r.span.lo + i;
      *offset = key_offset ? (int64_t)__shfl((long long)r.lane_offset, i, kWave) : 0;
      return v + (int64_t)__shfl((long long)r.lane_shift, i, kWave);
    }
    const int64_t c = r.span.lo + segment_of(sub_indptr + r.span.lo, r.span.hi - r.span.lo + 1, v);
    *col = c;
    *offset = key_offset ? key_offset[c] : 0;
    return indptr[cols[c]] + (v - sub_indptr[c]);
  }
};
inline SliceView no_view() { return SliceView{nullptr, nullptr, nullptr, nullptr, 0}; }

__device__ __forceinline__ int64_t column_degree(const int64_t* indptr,
                                                 int64_t num_cols, int64_t c,
                                                 int64_t* in_start) {
  if (c < 0 || c >= num_cols) {
    *in_start = 0;
    return 0;
  }
  int64_t b = indptr[c];
  *in_start = b;
  return indptr[c + 1] - b;
}

// What the count pass of a slice or a sampler can leave behind for the fill pass
// of the same columns, one word per requested column: where the column starts
// (low 40 bits) and how long it is (24 bits above), so that the fill pass reads
// its columns' spans in a stream instead of looking up each column's pointer pair
// again -- a 128-byte line of the matrix's column pointer per column.  A start or
// a length that does not fit is kSpanLookUp: look the pair up after all.
constexpr int kSpanStartBits = 40;
constexpr uint64_t kSpanLookUp = ~0ull;
__device__ __forceinline__ int64_t pack_span(int64_t start, int64_t deg) {
  const bool fits = ((uint64_t)start >> kSpanStartBits) == 0 && deg >= 0 && deg < (1 << 24) - 1;
  return (int64_t)(fits ? ((uint64_t)deg << kSpanStartBits) | (uint64_t)start : kSpanLookUp);
}
// Degree and start of requested column `item`: from its span when there is one,
// else from the column pointer.
__device__ __forceinline__ int64_t column_span(const int64_t* __restrict__ col_span,
                                               const int64_t* __restrict__ column_ids,
                                               const int64_t* __restrict__ indptr,
                                               int64_t num_cols, int64_t item,
                                               int64_t* in_start) {
  if (col_span != nullptr) {
    const uint64_t span = (uint64_t)col_span[item];
    if (span != kSpanLookUp) {
      *in_start = (int64_t)(span & ((1ull << kSpanStartBits) - 1ull));
      return (int64_t)(span >> kSpanStartBits);
    }
  }
  return column_degree(indptr, num_cols, column_ids ? column_ids[item] : item, in_start);
}

}  // namespace gs

#endif  // GSAMPLER_CSRC_COMMON_H_
