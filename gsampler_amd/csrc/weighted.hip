// weighted.hip -- weighted sampling: per column (individual) and over a list
// (collective / layer-wise), with and without replacement.
//
// Without replacement: Efraimidis-Spirakis in exponential-clock form.  Item i
// gets key (-log2 u_i) / w_i, the K smallest keys win (same ranking as the K
// largest u^(1/w)).  The key uses correctly rounded double operations only, so
// the CPU check computes bit-identical keys; ties break to the smaller index.
// With replacement: integer CDF (weights quantised against the exact maximum,
// integer prefix sums are order-independent) and a binary search per pick.
#include "common.h"
#include "scan.h"

// The sampling keys must come out bit-identical to the CPU check: no implicit
// fusing of a multiply into a neighbouring add anywhere in this file.
#pragma clang fp contract(off)

#include <cstdlib>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_segmented_radix_sort.hpp>

namespace gs {

// ------------------------------------------------------------ key arithmetic
// x / y for finite normal y > 0 from fused multiply-adds only: a bit-trick
// reciprocal estimate (12 % off at worst), six Newton steps, one residual
// correction.  Hardware division is avoided because its last bit need not
// agree between a GPU and a CPU; every operation here is a correctly rounded
// IEEE operation, so the result is reproducible anywhere (it lies within an
// ulp or two of the true quotient, which is all a sampling key needs).
__device__ __forceinline__ double det_div(double x, double y) {
  double r = __longlong_as_double(0x7FDE623822FC16E6ll - __double_as_longlong(y));
#pragma unroll
  for (int i = 0; i < 6; ++i) r = __fma_rn(r, __fma_rn(-y, r, 1.0), r);
  const double q = __dmul_rn(x, r);
  return __fma_rn(__fma_rn(-y, q, x), r, q);
}

__device__ __forceinline__ double neg_log2_unit(uint64_t r64) {
  const uint64_t v = (r64 >> 12) + 1;  // [1, 2^52]: exact as a double
  int e = 63 - __clzll((long long)v);
  double m = ldexp((double)(long long)v, -e);  // [1, 2)
  if (m > 0x1.6a09e667f3bcdp+0) {
    m = __dmul_rn(m, 0.5);
    e += 1;
  }
  const double s = det_div(__dsub_rn(m, 1.0), __dadd_rn(m, 1.0));
  const double s2 = __dmul_rn(s, s);
  double p = 0x1.1964ec6fc9491p-3;
  p = __fma_rn(p, s2, 0x1.3703c1f4d0ffep-3);
  p = __fma_rn(p, s2, 0x1.5b9ac9b743f0dp-3);
  p = __fma_rn(p, s2, 0x1.89f3b1694cffep-3);
  p = __fma_rn(p, s2, 0x1.c68f568d31761p-3);
  p = __fma_rn(p, s2, 0x1.0c9a84994022dp-2);
  p = __fma_rn(p, s2, 0x1.484b13d7c02a9p-2);
  p = __fma_rn(p, s2, 0x1.a61762a7adedap-2);
  p = __fma_rn(p, s2, 0x1.2776c50ef9bfep-1);
  p = __fma_rn(p, s2, 0x1.ec709dc3a03fep-1);
  p = __fma_rn(p, s2, 0x1.71547652b82fep+1);
  return __fma_rn(-s, p, (double)(52 - e));
}

__device__ __forceinline__ double weighted_key(PhiloxKey key, uint64_t pos,
                                               uint64_t draw, float w) {
  if (!(w > 0.0f)) return __longlong_as_double(0x7ff0000000000000ll);  // +inf
  const Words4 wd = philox(key, pos, draw);
  const uint64_t r = ((uint64_t)wd.y << 32) | wd.x;
  return det_div(neg_log2_unit(r), (double)w);
}

__global__ void weighted_key_probe_kernel(PhiloxKey key, uint64_t pos,
                                          uint64_t draw, float w, uint64_t r64,
                                          double* out) {
  out[0] = neg_log2_unit(r64);
  out[1] = weighted_key(key, pos, draw, w);
}

__device__ __forceinline__ bool key_less(double ka, int64_t ia, double kb,
                                         int64_t ib) {
  return ka < kb || (ka == kb && ia < ib);
}

// -------------------------------------------- per column, without replacement
// One wavefront per requested column.  Every lane keeps the K smallest keys of
// the edges it visits (lane l sees offsets l, l + 64, ...) as a sorted list in
// LDS, laid out [slot][thread] so that a wavefront touches consecutive banks.
// The 64 sorted lists are then merged by K rounds of a wavefront arg-min.
__global__ __launch_bounds__(kBlock) void sample_weighted_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ indices, const float* __restrict__ probs,
    const int64_t* __restrict__ column_ids, int64_t num_items, int fanout,
    PhiloxKey key, const int64_t* __restrict__ sub_indptr,
    int64_t* __restrict__ out_coo_col, int64_t* __restrict__ out_indices,
    int64_t* __restrict__ out_select, ColumnLabels labels) {
  extern __shared__ __align__(8) unsigned char smem[];
  const int nthreads = blockDim.x;
  double* lkey = (double*)smem;                               // [fanout][nthreads]
  int* lidx = (int*)(smem + (size_t)fanout * nthreads * sizeof(double));
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int64_t item = ((int64_t)blockIdx.x * nthreads + tid) / kWave;
  if (item >= num_items) return;
  const int64_t c = column_ids ? column_ids[item] : item;
  int64_t in_start;
  const int64_t deg = column_degree(indptr, num_cols, c, &in_start);
  if (deg == 0) return;
  const int64_t out_start = sub_indptr[item];
  const int K = fanout;

  if (deg <= K) {  // whole column, original order, zero weights included
    for (int64_t j = lane; j < deg; j += kWave) {
      const int64_t p = in_start + j;
      out_indices[out_start + j] = indices ? indices[p] : p;
      out_select[out_start + j] = p;
      if (out_coo_col) out_coo_col[out_start + j] = labels.of(item);
    }
    return;
  }

  int cnt = 0;
  for (int64_t j = lane; j < deg; j += kWave) {
    const double k = weighted_key(key, (uint64_t)item, (uint64_t)j, probs[in_start + j]);
    // offsets grow along a lane, so an equal key never displaces a kept one
    if (cnt == K && !(k < lkey[(K - 1) * nthreads + tid])) continue;
    int s = cnt < K ? cnt : K - 1;
    while (s > 0 && k < lkey[(s - 1) * nthreads + tid]) {
      lkey[s * nthreads + tid] = lkey[(s - 1) * nthreads + tid];
      lidx[s * nthreads + tid] = lidx[(s - 1) * nthreads + tid];
      --s;
    }
    lkey[s * nthreads + tid] = k;
    lidx[s * nthreads + tid] = (int)(j / kWave);  // j = lane + 64 * (stored value)
    if (cnt < K) ++cnt;
  }

  int head = 0;
  int64_t mine = -1;  // lane r keeps the winner of round r
  for (int r = 0; r < K; ++r) {
    double k = __longlong_as_double(0x7ff0000000000000ll);
    int64_t off = INT64_MAX;
    if (head < cnt) {
      k = lkey[head * nthreads + tid];
      off = (int64_t)lidx[head * nthreads + tid] * kWave + lane;
    }
    double bk = k;
    int64_t bo = off;
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
      const double ok = __shfl_xor(bk, d, kWave);
      const int64_t oo = __shfl_xor(bo, d, kWave);
      if (key_less(ok, oo, bk, bo)) {
        bk = ok;
        bo = oo;
      }
    }
    if (off == bo) ++head;  // offsets are unique, so exactly one lane advances
    if (lane == r) mine = bo;
  }
  if (lane < K) {
    const int64_t p = in_start + mine;
    out_indices[out_start + lane] = indices ? indices[p] : p;
    out_select[out_start + lane] = p;
    if (out_coo_col) out_coo_col[out_start + lane] = labels.of(item);
  }
}

// ----------------------------------------------- per column, with replacement
__device__ __forceinline__ uint64_t quantise(float w, double scale) {
  return w > 0.0f ? (uint64_t)__dmul_rn((double)w, scale) : 0ull;
}

// First position in cdf[0, n) whose value exceeds t, clamped to n - 1.
__device__ __forceinline__ int64_t cdf_search(const uint64_t* cdf, int64_t n,
                                              uint64_t t) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (cdf[mid] > t)
      hi = mid;
    else
      lo = mid + 1;
  }
  return lo < n ? lo : n - 1;
}

// One wavefront per column: exact max of the weights, integer CDF into the
// scratch slice of the column, then one binary search per output slot.
__global__ __launch_bounds__(kBlock) void sample_weighted_replace_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ indices, const float* __restrict__ probs,
    const int64_t* __restrict__ column_ids, int64_t num_items, int64_t fanout,
    PhiloxKey key, const int64_t* __restrict__ sub_indptr,
    const int64_t* __restrict__ cdf_offsets, uint64_t* cdf_scratch,
    int64_t* __restrict__ out_coo_col, int64_t* __restrict__ out_indices,
    int64_t* __restrict__ out_select, ColumnLabels labels) {
  const int lane = lane_id();
  const int64_t item = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  if (item >= num_items) return;
  const int64_t c = column_ids ? column_ids[item] : item;
  int64_t in_start;
  const int64_t deg = column_degree(indptr, num_cols, c, &in_start);
  if (deg == 0) return;
  const int64_t out_start = sub_indptr[item];
  uint64_t* cdf = cdf_scratch + (cdf_offsets ? cdf_offsets[item] : in_start);

  float wmax = 0.0f;
  for (int64_t j = lane; j < deg; j += kWave) {
    const float w = probs[in_start + j];
    if (w > wmax) wmax = w;
  }
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    const float o = __shfl_xor(wmax, d, kWave);
    if (o > wmax) wmax = o;
  }
  const double scale = wmax > 0.0f ? det_div(2147483648.0, (double)wmax) : 0.0;
  uint64_t carry = 0;
  for (int64_t base = 0; base < deg; base += kWave) {
    const int64_t j = base + lane;
    uint64_t q = (j < deg && wmax > 0.0f) ? quantise(probs[in_start + j], scale) : 0ull;
    q = wave_inclusive_sum(q);
    if (j < deg) cdf[j] = carry + q;
    carry += __shfl(q, kWave - 1, kWave);
  }
  const uint64_t total = carry;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  for (int64_t j = lane; j < fanout; j += kWave) {
    const uint64_t t = total > 0 ? philox_bounded(key, (uint64_t)item, (uint64_t)j, total) : 0ull;
    // the scratch was written by other lanes of this wavefront: read past L1
    int64_t lo = 0, hi = deg;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      const uint64_t v = __hip_atomic_load(cdf + mid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (v > t)
        hi = mid;
      else
        lo = mid + 1;
    }
    const int64_t p = in_start + (lo < deg ? lo : deg - 1);
    out_indices[out_start + j] = indices ? indices[p] : p;
    out_select[out_start + j] = p;
    if (out_coo_col) out_coo_col[out_start + j] = labels.of(item);
  }
}

// ------------------------------------------- persistent packed CDF of a matrix
// One 64-bit entry per edge, built once per (matrix, weights):
//   cdf[0]      = row_bits, the number of low bits of an entry that hold a row id
//                 (0: no row ids packed, the sampler reads them from `indices`)
//   cdf[e + 1]  = share(e) << row_bits | row id of edge e
// share(e) is the part of its column's mass that lies at or before edge e, in
// units of 2^-cb (cb = min(62, 64 - row_bits)): the weights of a column are
// quantised to 31 bits against the column's exact maximum (integers, so their
// prefix sums G do not depend on the order of additions), and
//   share(e) = floor(G(e) * 2^cb / T)   for G(e) < T = the column's total,
//   share(e) = 2^cb - 1                 from the last positive item on
// (0 everywhere in a column without positive weights).  Item j of a column
// owns [share(j - 1), share(j)); a draw is a search for the item whose interval
// holds a point, over 8-byte entries, and the row id of the item arrives with
// the entry that ends the search: a pick costs the lines of its search and
// nothing else.  (Row ids and prefix sums in arrays of their own cost a random
// 128-byte line per pick for the row id and two for the ends of the column's
// slice of a global prefix sum.)
// Both passes take tiles of consecutive edges and look the tile's first and
// last column up once, on the scalar unit; an edge then searches only among
// the columns of its tile instead of all of them.
constexpr int kCdfItems = 8;
constexpr int kCdfTile = kBlock * kCdfItems;
constexpr int kCdfMaxRowBits = 32;

// Column maxima: the tile's maxima are first taken in LDS (integer atomics on
// the bit patterns: positive floats order like their bits), then every column
// the tile touches sends one atomic to memory.  With one atomic per edge the
// pass ran at the rate of the memory-side atomic units.
constexpr int kCdfSegs = 4096;

__global__ __launch_bounds__(kBlock) void cdf_colmax_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const float* __restrict__ probs, int64_t nnz, unsigned int* colmax_bits) {
  __shared__ unsigned int tile_max[kCdfSegs];
  const int64_t e0 = (int64_t)blockIdx.x * kCdfTile;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kCdfTile - 1 < nnz ? e0 + kCdfTile - 1 : nnz - 1;
  float w[kCdfItems];
#pragma unroll
  for (int j = 0; j < kCdfItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    w[j] = e <= e_last ? probs[e] : 0.0f;
  }
  const SegmentSpan span = segment_span(indptr, num_cols, e0, e_last);
  const int64_t nseg = span.hi - span.lo + 1;
  const bool in_lds = nseg <= kCdfSegs;
  if (in_lds) {
    for (int64_t j = threadIdx.x; j < nseg; j += kBlock) tile_max[j] = 0u;
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < kCdfItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (e > e_last || !(w[j] > 0.0f)) continue;
    const int64_t c = span.segment_at(indptr, e);
    if (in_lds) atomicMax(&tile_max[c - span.lo], __float_as_uint(w[j]));
    else atomicMax(colmax_bits + c, __float_as_uint(w[j]));
  }
  if (!in_lds) return;
  __syncthreads();
  for (int64_t j = threadIdx.x; j < nseg; j += kBlock)
    if (tile_max[j] != 0u) atomicMax(colmax_bits + span.lo + j, tile_max[j]);
}

// prefix[e] = quantised weight of edge e (the device-wide scan that follows
// turns it into the sum of all quantised weights before e); prefix[nnz] = 0.
__global__ __launch_bounds__(kBlock) void cdf_quantise_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const float* __restrict__ probs, int64_t nnz,
    const unsigned int* __restrict__ colmax_bits, int64_t* __restrict__ prefix) {
  const int64_t e0 = (int64_t)blockIdx.x * kCdfTile;
  if (e0 > nnz) return;
  if (e0 == nnz) {  // prefix[nnz] = 0 closes the exclusive scan
    if (threadIdx.x == 0) prefix[nnz] = 0;
    return;
  }
  const int64_t e_last = e0 + kCdfTile - 1 < nnz ? e0 + kCdfTile - 1 : nnz - 1;
  const SegmentSpan span = segment_span(indptr, num_cols, e0, e_last);
#pragma unroll
  for (int j = 0; j < kCdfItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (e > e_last) break;
    uint64_t q = 0;
    const float wmax = __uint_as_float(colmax_bits[span.segment_at(indptr, e)]);
    if (wmax > 0.0f) q = quantise(probs[e], det_div(2147483648.0, (double)wmax));
    prefix[e] = (int64_t)q;
  }
  if (e_last == nnz - 1 && threadIdx.x == 0) prefix[nnz] = 0;
}

__global__ __launch_bounds__(kBlock) void cdf_zero_kernel(unsigned int* p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// floor(a * 2^bits / t) for a < t < 2^63, by shift and subtract: exact integer
// arithmetic, so the CPU check (a 128-bit division) agrees to the bit.
__device__ __forceinline__ uint64_t scale_share(uint64_t a, uint64_t t, int bits) {
  uint64_t rem = a, q = 0;
  for (int i = 0; i < bits; ++i) {
    rem <<= 1;
    q <<= 1;
    if (rem >= t) {
      rem -= t;
      q |= 1ull;
    }
  }
  return q;
}

// prefix[] (global exclusive prefix sums of the quantised weights) -> entries.
__global__ __launch_bounds__(kBlock) void cdf_pack_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ indices, int64_t nnz,
    const int64_t* __restrict__ prefix, int row_bits, uint64_t* __restrict__ cdf) {
  const int64_t e0 = (int64_t)blockIdx.x * kCdfTile;
  if (blockIdx.x == 0 && threadIdx.x == 0) cdf[0] = (uint64_t)row_bits;
  if (e0 >= nnz) return;
  const int64_t e_last = e0 + kCdfTile - 1 < nnz ? e0 + kCdfTile - 1 : nnz - 1;
  const SegmentSpan span = segment_span(indptr, num_cols, e0, e_last);
  const int cb = 64 - row_bits < 62 ? 64 - row_bits : 62;
  const uint64_t full = (1ull << cb) - 1ull;
  const uint64_t row_mask = row_bits ? (~0ull >> (64 - row_bits)) : 0ull;
#pragma unroll
  for (int j = 0; j < kCdfItems; ++j) {
    const int64_t e = e0 + j * kBlock + threadIdx.x;
    if (e > e_last) break;
    const int64_t c = span.segment_at(indptr, e);
    const uint64_t base = (uint64_t)prefix[indptr[c]];
    const uint64_t t = (uint64_t)prefix[indptr[c + 1]] - base;
    const uint64_t a = (uint64_t)prefix[e + 1] - base;
    const uint64_t share = a == t ? (t ? full : 0ull) : scale_share(a, t, cb);
    const uint64_t row = row_bits ? ((uint64_t)indices[e] & row_mask) : 0ull;
    cdf[e + 1] = (share << row_bits) | row;
  }
}

// Search state of one draw over a column's entries col[1 .. deg] (col[j] is the
// entry of item j - 1, so its share is the point where item j starts): the
// item whose interval holds x is the last j in [0, deg) with start(j) <= x, for
// start(0) = 0 <= x < start(deg) = the column's mass.  Shares of weights are
// close to a straight line, so guesses interpolate; every other step (mode 1)
// or every step after kInterpolations guesses (mode 2) is a plain bisection,
// which bounds the worst case for any weights; mode 0 only bisects.  The entry
// that last lowered `hi` stays at hand: when the search ends it is the entry
// of the item found, row id included.
constexpr int kInterpolations = 8;
// Search mode of the CDF sampler: 0 bisection, 1 alternating, 2 interpolation
// first (the fastest on prefix sums of real weights, which are nearly linear).
constexpr int kCdfSearchMode = 2;
struct CdfSearch {
  int64_t lo, hi;
  uint64_t a_lo, a_hi, x, e_hi;
  int guesses;
  bool flip;
  __device__ __forceinline__ void begin(int64_t deg, uint64_t mass, uint64_t point) {
    lo = 0;
    hi = deg;
    a_lo = 0;
    a_hi = mass;
    e_hi = 0;  // the column's last entry, which nobody has read yet
    x = point;
    guesses = 0;
    flip = true;
  }
  __device__ __forceinline__ bool done() const { return hi - lo <= 1; }
  __device__ __forceinline__ int64_t probe_at() {
    constexpr int mode = kCdfSearchMode;
    bool interpolate = false;
    if (hi - lo > 8) {
      if (mode == 1) interpolate = flip;
      if (mode == 2) interpolate = guesses < kInterpolations;
    }
    flip = !flip;
    if (!interpolate) return (lo + hi) >> 1;
    ++guesses;
    // (a guess: the hardware's approximate reciprocal will do, and where a probe
    // lands never changes which item the search ends at)
    const double frac = (double)(x - a_lo) * __builtin_amdgcn_rcp((double)(a_hi - a_lo));
    int64_t mid = lo + (int64_t)(frac * (double)(hi - lo));
    if (mid <= lo) mid = lo + 1;
    if (mid >= hi) mid = hi - 1;
    return mid;
  }
  __device__ __forceinline__ void narrow(int64_t mid, uint64_t entry, int row_bits) {
    const uint64_t v = entry >> row_bits;
    if (v <= x) {
      lo = mid;
      a_lo = v;
    } else {
      hi = mid;
      a_hi = v;
      e_hi = entry;
    }
  }
};

// Leaves the item in s.lo and its interval in [s.a_lo, s.a_hi); its entry is in
// s.e_hi unless the search ended at the column's last item without having
// looked at it (s.hi == deg).  `mass` is what the column's shares add up to.
__device__ __forceinline__ void cdf_locate(CdfSearch& s, const uint64_t* __restrict__ col,
                                           int64_t deg, uint64_t mass, int row_bits,
                                           uint64_t x) {
  s.begin(deg, mass, x);
  while (!s.done()) {
    const int64_t mid = s.probe_at();
    s.narrow(mid, col[mid], row_bits);
  }
}

constexpr int kMaxCdfFanout = 64;

// One lane per requested column.
// Without replacement: successive weighted sampling.  Draw j takes a uniform
// point r of the mass that is still there and maps it past the intervals of the
// items already taken (x = r + the lengths of all taken intervals that start at
// or before x, found by iterating from x = r), so no draw repeats an item and
// a column costs exactly fanout searches whatever its weights look like; when
// the positive mass runs out, zero-weight items follow in index order.
// An earlier version let a group of lanes search independent points of the
// whole mass at once and skipped repeats: columns whose degree or effective
// number of items is close to the fan-out then need several rounds, every round
// costs the whole wavefront a Philox block and a search per lane, and the
// bookkeeping of repeats alone was half of the kernel's time.
// With replacement: one independent point of the whole mass per output slot.
// Streams: pos = column position, draw = output slot.
// The taken intervals live in registers: every access runs over all KMAX slots
// with a predicate instead of indexing.
// (Fan-out 10 takes 134 registers left alone: capped at 128 it runs four wavefronts
// per SIMD instead of three, 342 against 362 us on 592 K columns; the same cap for 15
// and 16 spills more than it gains.)
template <int KMAX>
__global__ __launch_bounds__(kBlock, KMAX <= 10 ? 4 : 1) void sample_weighted_cdf_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const int64_t* __restrict__ indices, const uint64_t* __restrict__ cdf,
    const int64_t* __restrict__ column_ids, int64_t num_items, int fanout,
    int replace, PhiloxKey key, const int64_t* __restrict__ sub_indptr,
    int64_t* __restrict__ out_coo_col, int64_t* __restrict__ out_indices,
    int64_t* __restrict__ out_select, ColumnLabels labels,
    const int64_t* __restrict__ col_span) {
  const int64_t item = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (item >= num_items) return;
  // (asked for here, so that its loads travel with the ones below)
  const int64_t col_label =
      out_coo_col ? labels.of_near(item, item - lane_id()) : item;
  const int row_bits = (int)cdf[0];  // the same word for every lane: a scalar load
  const uint64_t row_mask = row_bits ? (~0ull >> (64 - row_bits)) : 0ull;
  int64_t in_start;
  const int64_t deg = column_span(col_span, column_ids, indptr, num_cols, item, &in_start);
  if (deg == 0) return;
  const int64_t out_start = sub_indptr[item];
  const uint64_t* col = cdf + in_start;  // col[j], 1 <= j <= deg: entry of item j - 1
  // A column's shares add up to 2^cb - 1, or to 0 when it has no positive weight.
  // Which of the two is in the column's last entry, one more random line that a
  // column longer than the fan-out only reads when a search ends at its last item
  // (in a column without mass the first search does: every share is 0).
  const int cb = 64 - row_bits < 62 ? 64 - row_bits : 62;
  const uint64_t full = (1ull << cb) - 1ull;
  auto row_of = [&](int64_t off, uint64_t entry) -> int64_t {
    if (row_bits) return (int64_t)(entry & row_mask);
    return indices ? indices[in_start + off] : in_start + off;
  };
  // The picks of a column wait in registers (offset and row id) and leave
  // together at the end, so that a lane's outputs reach each array back to
  // back and the wavefront fills whole lines where pick-by-pick stores leave
  // partial lines to be evicted and reopened (measured on 3.5 M columns with
  // fanout 5: 33 M write requests and 1.8 ms pick by pick, 1.2 ms held).  What
  // does not fit the registers is written pick by pick: columns of 2^32 or
  // more items (no graph seen so far has one, nothing forbids it) and fanouts
  // above KMAX, which only occur with replacement.
  const bool hold = deg <= 0xFFFFFFFFll && fanout <= KMAX;
  uint32_t held[KMAX], held_row[KMAX];
#pragma unroll
  for (int i = 0; i < KMAX; ++i) held[i] = held_row[i] = 0;
  int taken = 0;
  auto pick = [&](int64_t off, uint64_t entry) {
    if (!hold) {
      const int64_t p = in_start + off;
      out_indices[out_start + taken] = row_of(off, entry);
      out_select[out_start + taken] = p;
      if (out_coo_col) out_coo_col[out_start + taken] = col_label;
    }
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i == taken) {
        held[i] = (uint32_t)off;
        held_row[i] = (uint32_t)(entry & row_mask);
      }
    ++taken;
  };
  CdfSearch s;
  if (replace) {
    bool mass = true;
    for (int j = 0; j < fanout; ++j) {
      if (mass) {
        cdf_locate(s, col, deg, full, row_bits,
                   philox_bounded(key, (uint64_t)item, (uint64_t)j, full));
        if (s.hi == deg) {
          s.e_hi = col[deg];
          mass = (s.e_hi >> row_bits) != 0;
        }
      }
      if (mass) pick(s.lo, s.e_hi);
      else pick(deg - 1, s.e_hi);  // no positive weight: the last item
    }
  } else if (deg <= fanout) {  // whole column, original order, zero weights included
    for (int64_t j = 0; j < deg; ++j) pick(j, col[j + 1]);
  } else {
    uint64_t start[KMAX], len[KMAX];
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
      start[i] = ~0ull;  // never at or before a point
      len[i] = 0;
    }
    uint64_t removed = 0;
    while (taken < fanout && removed < full) {
      const uint64_t r =
          philox_bounded(key, (uint64_t)item, (uint64_t)taken, full - removed);
      uint64_t x = r;
      for (int round = 0; round <= taken; ++round) {
        uint64_t skipped = 0;
#pragma unroll
        for (int i = 0; i < KMAX; ++i) skipped += start[i] <= x ? len[i] : 0ull;
        if (r + skipped == x) break;
        x = r + skipped;
      }
      cdf_locate(s, col, deg, full, row_bits, x);
      if (s.hi == deg) {  // ended at the last item without having read its entry
        s.e_hi = col[deg];
        if ((s.e_hi >> row_bits) == 0) break;  // a column without mass
      }
#pragma unroll
      for (int i = 0; i < KMAX; ++i)
        if (i == taken) {
          start[i] = s.a_lo;
          len[i] = s.a_hi - s.a_lo;
        }
      removed += s.a_hi - s.a_lo;
      pick(s.lo, s.e_hi);
    }
    // fewer than fanout items have positive weight: zero-weight items in order
    if (taken < fanout) {
      uint64_t before = 0;
      for (int64_t off = 0; taken < fanout && off < deg; ++off) {
        const uint64_t entry = col[off + 1], here = entry >> row_bits;
        if (here == before) pick(off, entry);
        before = here;
      }
    }
  }
  if (!hold) return;
  if (!row_bits) {
    int64_t row[KMAX];
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i < taken) row[i] = indices ? indices[in_start + held[i]] : in_start + held[i];
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i < taken) out_indices[out_start + i] = row[i];
  } else {
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i < taken) out_indices[out_start + i] = (int64_t)held_row[i];
  }
#pragma unroll
  for (int i = 0; i < KMAX; ++i)
    if (i < taken) out_select[out_start + i] = in_start + held[i];
  if (out_coo_col) {
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i < taken) out_coo_col[out_start + i] = col_label;
  }
}

template <int KMAX>
static int launch_weighted_cdf(const int64_t* indptr, int64_t num_cols,
                               const int64_t* indices, const int64_t* cdf,
                               const int64_t* column_ids, int64_t num_items,
                               int fanout, int replace, PhiloxKey key,
                               const int64_t* sub_indptr, int64_t* out_coo_col,
                               int64_t* out_indices, int64_t* out_select,
                               ColumnLabels labels, const int64_t* col_span, hipStream_t s) {
  GS_LAUNCH("sample_weighted_cdf", s,
            sample_weighted_cdf_kernel<KMAX><<<dim3((unsigned)ceil_div(num_items, kBlock)),
                                               dim3(kBlock), 0, s>>>(
                indptr, num_cols, indices, (const uint64_t*)cdf, column_ids, num_items,
                fanout, replace, key, sub_indptr, out_coo_col, out_indices, out_select, labels,
                col_span));
  return GS_OK;
}

// ------------------------------------------------------------ list sampling
__global__ __launch_bounds__(kBlock) void list_keys_kernel(
    const float* __restrict__ probs, int64_t n, PhiloxKey key,
    uint64_t* __restrict__ keys, int64_t* __restrict__ iota) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  // non-negative doubles (and +inf) order like their bit patterns
  keys[i] = (uint64_t)__double_as_longlong(weighted_key(key, (uint64_t)i, 0, probs[i]));
  iota[i] = i;
}

// Per segment: number of picks (replace: K for a non-empty segment; else
// min(K, n_b)).  One extra thread writes the trailing 0 for the scan.
__global__ void list_counts_kernel(const int64_t* __restrict__ range, int64_t n,
                                   int64_t nseg, int64_t num_picks, int replace,
                                   int64_t* __restrict__ counts) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > nseg) return;
  int64_t cnt = 0;
  if (b < nseg) {
    const int64_t nb = range ? range[b + 1] - range[b] : n;
    cnt = replace ? (nb > 0 ? num_picks : 0) : (nb < num_picks ? nb : num_picks);
  }
  counts[b] = cnt;
}

// The same for at most kBlock - 1 segments, with the running sum: one launch
// instead of counts + scan.
__global__ __launch_bounds__(kBlock) void list_offsets_kernel(
    const int64_t* __restrict__ range, int64_t n, int64_t nseg, int64_t num_picks, int replace,
    int64_t* __restrict__ out_range) {
  __shared__ int64_t smem[kBlock / kWave + 1];
  const int64_t b = threadIdx.x;
  int64_t cnt = 0;
  if (b < nseg) {
    const int64_t nb = range ? range[b + 1] - range[b] : n;
    cnt = replace ? (nb > 0 ? num_picks : 0) : (nb < num_picks ? nb : num_picks);
  }
  int64_t total;
  const int64_t before = block_exclusive_sum(cnt, smem, &total);
  if (b <= nseg) out_range[b] = before;
}

// Copies the first out_range[b+1] - out_range[b] sorted values of every
// segment; a segment that is taken whole keeps its original order.
__global__ __launch_bounds__(kBlock) void list_take_kernel(
    const int64_t* __restrict__ sorted_vals, const int64_t* __restrict__ range,
    int64_t n, int64_t nseg, int64_t num_picks,
    const int64_t* __restrict__ out_range, int64_t total,
    int64_t* __restrict__ out_index) {
  const int64_t o = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (o >= total) return;
  const int64_t b = nseg == 1 ? 0 : segment_of(out_range, nseg, o);
  const int64_t lo = range ? range[b] : 0;
  const int64_t nb = (range ? range[b + 1] : n) - lo;
  const int64_t k = o - out_range[b];
  out_index[o] = nb <= num_picks ? lo + k : sorted_vals[lo + k];
}

// Integer CDF of a list segment by segment is a device-wide problem; segments
// are handled one wavefront each (layer-wise samplers have few, long segments
// at most a few hundred thousand items long).
__global__ __launch_bounds__(kBlock) void list_replace_kernel(
    const float* __restrict__ probs, const int64_t* __restrict__ range,
    int64_t n, int64_t nseg, int64_t num_picks, PhiloxKey key,
    const int64_t* __restrict__ out_range, uint64_t* cdf_scratch,
    int64_t* __restrict__ out_index) {
  const int lane = lane_id();
  const int64_t b = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  if (b >= nseg) return;
  const int64_t lo = range ? range[b] : 0, hi = range ? range[b + 1] : n;
  const int64_t nb = hi - lo;
  if (nb == 0) return;
  uint64_t* cdf = cdf_scratch + lo;
  float wmax = 0.0f;
  for (int64_t j = lane; j < nb; j += kWave) {
    const float w = probs[lo + j];
    if (w > wmax) wmax = w;
  }
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    const float o = __shfl_xor(wmax, d, kWave);
    if (o > wmax) wmax = o;
  }
  const double scale = wmax > 0.0f ? det_div(2147483648.0, (double)wmax) : 0.0;
  uint64_t carry = 0;
  for (int64_t base = 0; base < nb; base += kWave) {
    const int64_t j = base + lane;
    uint64_t q = (j < nb && wmax > 0.0f) ? quantise(probs[lo + j], scale) : 0ull;
    q = wave_inclusive_sum(q);
    if (j < nb) cdf[j] = carry + q;
    carry += __shfl(q, kWave - 1, kWave);
  }
  const uint64_t total = carry;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  const int64_t out_start = out_range[b];
  for (int64_t k = lane; k < num_picks; k += kWave) {
    const uint64_t t = total > 0 ? philox_bounded(key, (uint64_t)b, (uint64_t)k, total) : 0ull;
    int64_t l = 0, h = nb;
    while (l < h) {
      const int64_t mid = (l + h) >> 1;
      const uint64_t v = __hip_atomic_load(cdf + mid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (v > t)
        h = mid;
      else
        l = mid + 1;
    }
    out_index[out_start + k] = lo + (l < nb ? l : nb - 1);
  }
}

// Zeroes n 32-bit words (a kernel rather than a memset so that callers may
// capture the launches in a HIP graph).
__global__ __launch_bounds__(kBlock) void table_fill_kernel32(uint32_t* __restrict__ words,
                                                              int64_t n) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (; i < n; i += stride) words[i] = 0u;
}

// ---------------------------------------------- the K smallest keys by selection
// Without replacement the pick is "the K smallest keys, in ascending order, ties
// to the smaller index".  Sorting all n keys for that costs sixteen launches of
// a radix sort; for K up to kSelMaxPicks the kernels below select instead:
//   keys     key of every item (kept), histogram of its top 12 bits (the
//            exponent of a non-negative double) per segment
//   refine   the bin that holds the K-th smallest key follows from that
//            histogram (every work-group scans it for itself: 4096 bins); items
//            of that bin are counted by their next 12 bits
//   emit     the same again one level down; items below the K-th item's
//            (bin, sub-bin) cell are certain picks and go to the segment's pick
//            list, items inside the cell to its candidate list
//   finish   picks + the smallest candidates of a segment are ordered by
//            (key, index) in LDS and written out (sixteen work-groups per
//            segment share the comparisons)
// The cell of the K-th item holds a handful of items unless keys repeat (items
// of weight zero all have the key +inf); a cell too large for LDS is narrowed
// by a byte-wise radix selection over its remaining key bits and indices first.
constexpr int kSelBins = 4096;
constexpr int kSelTile = 4096;  // shortest average segment the selection takes on
constexpr int64_t kSelMaxPicks = 2048;
constexpr int kFinishThreads = 1024;
constexpr int kFinishSlots = 4096;
constexpr int kFinishSplit = 16;  // work-groups that share the ordering of one segment's picks

__host__ __device__ inline bool list_can_select(int64_t n, int64_t nseg) {
  return n < (int64_t(1) << 31) && (nseg == 1 || n / nseg >= kSelTile);
}

__device__ __forceinline__ uint32_t sel_digit1(uint64_t k) { return (uint32_t)(k >> 52); }
__device__ __forceinline__ uint32_t sel_digit2(uint64_t k) {
  return (uint32_t)(k >> 40) & (kSelBins - 1);
}

// The bin of a kSelBins-bin histogram that holds the want-th smallest item
// (1-based, want <= number of items), and the number of items in the bins
// below it.  Called by the whole work-group; the result is the same in every
// thread.
__device__ __forceinline__ void find_bin(const uint32_t* __restrict__ hist, uint32_t want,
                                         uint32_t* smem, uint32_t* found, uint32_t* bin,
                                         uint32_t* below) {
  constexpr int kPer = kSelBins / kBlock;
  uint32_t c[kPer], sum = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    c[j] = hist[threadIdx.x * kPer + j];
    sum += c[j];
  }
  uint32_t total;
  uint32_t run = block_exclusive_sum(sum, smem, &total);
  const uint32_t target = want - 1;
  if (target >= run && target < run + sum) {
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      if (target >= run && target < run + c[j]) {
        found[0] = threadIdx.x * kPer + j;
        found[1] = run;
      }
      run += c[j];
    }
  }
  __syncthreads();
  *bin = found[0];
  *below = found[1];
  __syncthreads();
}

struct SelSegment {
  int64_t lo, hi;
};
__device__ __forceinline__ SelSegment sel_segment(const int64_t* __restrict__ range, int64_t n,
                                                  int64_t seg) {
  return range ? SelSegment{range[seg], range[seg + 1]} : SelSegment{0, n};
}
__device__ __forceinline__ SegmentSpan sel_span(const int64_t* __restrict__ range, int64_t nseg,
                                                int64_t i0, int64_t i_last) {
  return range ? segment_span(range, nseg, i0, i_last) : SegmentSpan{0, 0};
}

template <int kSelItems>
__global__ __launch_bounds__(kBlock) void list_keys_hist_kernel(
    const float* __restrict__ probs, const int64_t* __restrict__ range, int64_t n,
    int64_t nseg, PhiloxKey key, uint64_t* __restrict__ keys, uint32_t* hist1) {
  __shared__ uint32_t lh[kSelBins];
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * kSelItems);
  const int64_t i_last = i0 + (kBlock * kSelItems) - 1 < n ? i0 + (kBlock * kSelItems) - 1 : n - 1;
  const SegmentSpan span = sel_span(range, nseg, i0, i_last);
  for (int b = threadIdx.x; b < kSelBins; b += kBlock) lh[b] = 0;
  __syncthreads();
#pragma unroll 4
  for (int j = 0; j < kSelItems; ++j) {
    const int64_t i = i0 + j * kBlock + threadIdx.x;
    if (i >= n) break;
    // non-negative doubles (and +inf) order like their bit patterns
    const uint64_t k =
        (uint64_t)__double_as_longlong(weighted_key(key, (uint64_t)i, 0, probs[i]));
    keys[i] = k;
    const int64_t seg = span.segment_at(range, i);
    if (seg == span.lo)
      atomicAdd(&lh[sel_digit1(k)], 1u);
    else
      atomicAdd(&hist1[seg * kSelBins + sel_digit1(k)], 1u);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < kSelBins; b += kBlock)
    if (lh[b]) atomicAdd(&hist1[span.lo * kSelBins + b], lh[b]);
}

template <int kSelItems>
__global__ __launch_bounds__(kBlock) void list_refine_kernel(
    const int64_t* __restrict__ range, int64_t n, int64_t nseg, int64_t num_picks,
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ hist1, uint32_t* hist2) {
  __shared__ uint32_t lh[kSelBins];
  __shared__ uint32_t smem[kBlock / kWave + 1];
  __shared__ uint32_t found[2];
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * kSelItems);
  const int64_t i_last = i0 + (kBlock * kSelItems) - 1 < n ? i0 + (kBlock * kSelItems) - 1 : n - 1;
  const SegmentSpan span = sel_span(range, nseg, i0, i_last);
  for (int64_t seg = span.lo; seg <= span.hi; ++seg) {  // the same in every thread
    const SelSegment sg = sel_segment(range, n, seg);
    if (sg.hi - sg.lo <= num_picks) continue;  // taken whole
    uint32_t b1, below1;
    find_bin(hist1 + seg * kSelBins, (uint32_t)num_picks, smem, found, &b1, &below1);
    for (int b = threadIdx.x; b < kSelBins; b += kBlock) lh[b] = 0;
    __syncthreads();
#pragma unroll 4
    for (int j = 0; j < kSelItems; ++j) {
      const int64_t i = i0 + j * kBlock + threadIdx.x;
      if (i >= sg.lo && i < sg.hi && i <= i_last) {
        const uint64_t k = keys[i];
        if (sel_digit1(k) == b1) atomicAdd(&lh[sel_digit2(k)], 1u);
      }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < kSelBins; b += kBlock)
      if (lh[b]) atomicAdd(&hist2[seg * kSelBins + b], lh[b]);
    __syncthreads();
  }
}

template <int kSelItems>
__global__ __launch_bounds__(kBlock) void list_emit_kernel(
    const int64_t* __restrict__ range, int64_t n, int64_t nseg, int64_t num_picks,
    const uint64_t* __restrict__ keys, const uint32_t* __restrict__ hist1,
    const uint32_t* __restrict__ hist2, uint32_t* counts, uint64_t* __restrict__ win_key,
    int64_t* __restrict__ win_idx, uint64_t* __restrict__ cand_key,
    int64_t* __restrict__ cand_idx) {
  __shared__ uint32_t smem[kBlock / kWave + 1];
  __shared__ uint32_t found[2];
  __shared__ uint32_t bases[2];
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * kSelItems);
  const int64_t i_last = i0 + (kBlock * kSelItems) - 1 < n ? i0 + (kBlock * kSelItems) - 1 : n - 1;
  const SegmentSpan span = sel_span(range, nseg, i0, i_last);
  for (int64_t seg = span.lo; seg <= span.hi; ++seg) {  // the same in every thread
    const SelSegment sg = sel_segment(range, n, seg);
    if (sg.hi - sg.lo <= num_picks) continue;
    uint32_t b1, below1, b2, below2;
    find_bin(hist1 + seg * kSelBins, (uint32_t)num_picks, smem, found, &b1, &below1);
    find_bin(hist2 + seg * kSelBins, (uint32_t)num_picks - below1, smem, found, &b2, &below2);
    uint64_t k[kSelItems];
    uint32_t is_win = 0, is_cand = 0;  // one bit per item of this thread
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      const int64_t i = i0 + j * kBlock + threadIdx.x;
      k[j] = 0;
      if (i >= sg.lo && i < sg.hi && i <= i_last) {
        k[j] = keys[i];
        const uint32_t d1 = sel_digit1(k[j]), d2 = sel_digit2(k[j]);
        if (d1 < b1 || (d1 == b1 && d2 < b2))
          is_win |= 1u << j;
        else if (d1 == b1 && d2 == b2)
          is_cand |= 1u << j;
      }
    }
    uint32_t wins, cands;
    uint32_t w_at = block_exclusive_sum((uint32_t)__popc(is_win), smem, &wins);
    uint32_t c_at = block_exclusive_sum((uint32_t)__popc(is_cand), smem, &cands);
    if (threadIdx.x == 0) {
      bases[0] = wins ? atomicAdd(&counts[2 * seg], wins) : 0u;
      bases[1] = cands ? atomicAdd(&counts[2 * seg + 1], cands) : 0u;
    }
    __syncthreads();
    w_at += bases[0];
    c_at += bases[1];
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      const int64_t i = i0 + j * kBlock + threadIdx.x;
      if ((is_win >> j) & 1u) {
        if (w_at < (uint32_t)kSelMaxPicks) {  // always: fewer than num_picks items lie below the cell
          win_key[seg * kSelMaxPicks + w_at] = k[j];
          win_idx[seg * kSelMaxPicks + w_at] = i;
        }
        ++w_at;
      } else if ((is_cand >> j) & 1u) {
        if ((int64_t)c_at < sg.hi - sg.lo) {
          cand_key[sg.lo + c_at] = k[j];
          cand_idx[sg.lo + c_at] = i;
        }
        ++c_at;
      }
    }
    __syncthreads();
  }
}

// (key, index) as one number: the low 40 bits of the key (the upper 24 are the
// same for all candidates of a cell) above the 32-bit index.
__device__ __forceinline__ unsigned __int128 sel_composite(uint64_t k, int64_t i) {
  return ((unsigned __int128)(k & ((1ull << 40) - 1)) << 32) | (unsigned __int128)(uint32_t)i;
}

__global__ __launch_bounds__(kFinishThreads) void list_finish_kernel(
    const int64_t* __restrict__ range, int64_t n, int64_t num_picks,
    const uint32_t* __restrict__ counts, const uint64_t* __restrict__ win_key,
    const int64_t* __restrict__ win_idx, const uint64_t* __restrict__ cand_key,
    const int64_t* __restrict__ cand_idx, const int64_t* __restrict__ out_range,
    int64_t* __restrict__ out_index) {
  __shared__ uint64_t sk[kFinishSlots];
  __shared__ int64_t si[kFinishSlots];
  __shared__ uint32_t hist[256];
  __shared__ uint32_t chosen[2];
  __shared__ uint32_t appended;
  const int64_t seg = blockIdx.x;
  const SelSegment sg = sel_segment(range, n, seg);
  const int64_t nb = sg.hi - sg.lo, out0 = out_range[seg];
  if (nb <= num_picks) {  // taken whole, in the original order
    if (blockIdx.y == 0)
      for (int64_t k = threadIdx.x; k < nb; k += kFinishThreads) out_index[out0 + k] = sg.lo + k;
    return;
  }
  // (fewer than num_picks picks lie below the cell and no list is longer than its
  // segment; the bounds are restated here because LDS indices follow from them)
  uint32_t W = counts[2 * seg], M = counts[2 * seg + 1];
  if (W > (uint32_t)kSelMaxPicks) W = (uint32_t)kSelMaxPicks;
  if (W > (uint32_t)num_picks) W = (uint32_t)num_picks;
  if ((int64_t)M > nb) M = (uint32_t)nb;
  const uint64_t* ck = cand_key + sg.lo;
  const int64_t* ci = cand_idx + sg.lo;
  for (uint32_t t = threadIdx.x; t < W; t += kFinishThreads) {
    sk[t] = win_key[seg * kSelMaxPicks + t];
    si[t] = win_idx[seg * kSelMaxPicks + t];
  }
  uint32_t total = W + M;
  if (total <= (uint32_t)kFinishSlots) {
    for (uint32_t t = threadIdx.x; t < M; t += kFinishThreads) {
      sk[W + t] = ck[t];
      si[W + t] = ci[t];
    }
  } else {
    // the `want` smallest of the M candidates: fix the composite of the last
    // of them byte by byte, most significant first
    uint32_t want = (uint32_t)num_picks - W;
    unsigned __int128 fixed = 0;
    for (int d = 0; d < 9; ++d) {
      const int shift = 8 * (8 - d);
      for (int b = threadIdx.x; b < 256; b += kFinishThreads) hist[b] = 0;
      __syncthreads();
      for (uint32_t t = threadIdx.x; t < M; t += kFinishThreads) {
        const unsigned __int128 c = sel_composite(ck[t], ci[t]);
        if ((c >> (shift + 8)) == (fixed >> (shift + 8)))
          atomicAdd(&hist[(uint32_t)(c >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t run = 0, b = 0;
        for (; b < 255 && run + hist[b] < want; ++b) run += hist[b];
        chosen[0] = b;
        chosen[1] = run;
      }
      __syncthreads();
      fixed |= (unsigned __int128)chosen[0] << shift;
      want -= chosen[1];
      __syncthreads();
    }
    if (threadIdx.x == 0) appended = 0;
    __syncthreads();
    for (uint32_t t = threadIdx.x; t < M; t += kFinishThreads) {
      const uint64_t k = ck[t];
      const int64_t i = ci[t];
      if (sel_composite(k, i) <= fixed) {
        const uint32_t at = W + atomicAdd(&appended, 1u);
        if (at < (uint32_t)kFinishSlots) {
          sk[at] = k;
          si[at] = i;
        }
      }
    }
    total = (uint32_t)num_picks;
  }
  __syncthreads();
  // Order by (key, index): the rank of an item is the number of smaller ones.
  // The kFinishSplit work-groups of a segment all hold all items and each ranks
  // its share of them (shares go by index, so that they do not depend on the
  // order the lists were filled in): the comparisons (the square of the number
  // of items) are more than one compute unit should do alone.  Inside a
  // work-group the work is dealt out as (item, part of the others) pairs so
  // that all threads have some whatever the number of items; a thread reads
  // eight keys ahead (every lane of a wave reads the same ones: a broadcast),
  // partial ranks meet in LDS.
  __shared__ uint32_t rank_of_item[kFinishSlots];
  __shared__ uint16_t my_items[kFinishSlots];
  if (threadIdx.x == 0) appended = 0;
  for (uint32_t t = threadIdx.x; t < total; t += kFinishThreads) rank_of_item[t] = 0;
  __syncthreads();
  for (uint32_t t = threadIdx.x; t < total; t += kFinishThreads)
    if ((uint32_t)si[t] % kFinishSplit == blockIdx.y) my_items[atomicAdd(&appended, 1u)] = (uint16_t)t;
  __syncthreads();
  const uint32_t mine = appended;
  uint32_t parts = kFinishThreads / (mine ? mine : 1);
  if (parts < 1) parts = 1;
  if (parts > 8) parts = 8;
  const uint32_t per = (total + parts - 1) / parts;
  for (uint32_t w = threadIdx.x; w < mine * parts; w += kFinishThreads) {
    const uint32_t t = my_items[w % mine], part = w / mine;
    const uint64_t k = sk[t];
    const int64_t i = si[t];
    const uint32_t o_end = (part + 1) * per < total ? (part + 1) * per : total;
    uint32_t smaller = 0;
    for (uint32_t o = part * per; o < o_end; o += 8) {
      uint64_t ko[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) ko[u] = o + u < o_end ? sk[o + u] : ~0ull;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (ko[u] < k)
          ++smaller;
        else if (ko[u] == k && o + u < o_end && si[o + u] < i)
          ++smaller;
      }
    }
    atomicAdd(&rank_of_item[t], smaller);
  }
  __syncthreads();
  for (uint32_t m = threadIdx.x; m < mine; m += kFinishThreads) {
    const uint32_t t = my_items[m], r = rank_of_item[t];
    if (r < (uint32_t)num_picks) out_index[out0 + r] = si[t];
  }
}

struct ListWs {
  uint64_t *keys_in, *keys_out;  // also the CDF scratch when sampling with replacement
  int64_t *vals_in, *vals_out;
  void* sort_ws;
  size_t sort_ws_bytes;
  void* scan_ws;
  size_t scan_ws_bytes;
  // selection (list_can_select): histograms, then counters, in one block
  uint32_t* sel_block;
  size_t sel_words;
  uint32_t *hist1, *hist2, *counts;
  uint64_t* win_key;
  int64_t* win_idx;
  size_t total;
};

static size_t sort_temp_bytes(int64_t n, int64_t nseg) {
  size_t flat = 0, seg = 0;
  uint64_t* k = nullptr;
  int64_t* v = nullptr;
  (void)rocprim::radix_sort_pairs(nullptr, flat, k, k, v, v, (size_t)(n > 0 ? n : 1), 0, 64);
  const int64_t* off = nullptr;
  (void)rocprim::segmented_radix_sort_pairs(nullptr, seg, k, k, v, v, (size_t)(n > 0 ? n : 1),
                                            (unsigned)(nseg > 0 ? nseg : 1), off, off, 0, 64);
  return flat > seg ? flat : seg;
}

static ListWs carve_list(void* ws, int64_t n, int64_t nseg) {
  Carver c(ws);
  ListWs w;
  const size_t m = (size_t)(n > 0 ? n : 1);
  w.keys_in = c.take<uint64_t>(m);
  w.keys_out = c.take<uint64_t>(m);
  w.vals_in = c.take<int64_t>(m);
  w.vals_out = c.take<int64_t>(m);
  w.sort_ws_bytes = sort_temp_bytes(n, nseg);
  w.sort_ws = c.take<char>(w.sort_ws_bytes);
  w.scan_ws_bytes = scan_workspace_bytes(nseg + 1);
  w.scan_ws = c.take<char>(w.scan_ws_bytes);
  const size_t segs = list_can_select(n, nseg) ? (size_t)nseg : 0;
  w.sel_words = segs * (2 * kSelBins + 2);
  w.sel_block = c.take<uint32_t>(w.sel_words);
  w.hist1 = w.sel_block;
  w.hist2 = w.hist1 ? w.hist1 + segs * kSelBins : nullptr;
  w.counts = w.hist2 ? w.hist2 + segs * kSelBins : nullptr;
  w.win_key = c.take<uint64_t>(segs * (size_t)kSelMaxPicks);
  w.win_idx = c.take<int64_t>(segs * (size_t)kSelMaxPicks);
  w.total = c.total();
  return w;
}

}  // namespace gs

extern "C" {

int gs_weighted_key_probe(uint64_t seed, uint64_t call_id, uint64_t pos,
                          uint64_t draw, float w, uint64_t r64, double* out2,
                          gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(out2, "weighted_key_probe: null output");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("weighted_key_probe", s,
            weighted_key_probe_kernel<<<dim3(1), dim3(1), 0, s>>>(
                make_key(seed, call_id), pos, draw, w, r64, out2));
  return GS_OK;
}

size_t gs_weight_cdf_workspace_bytes(int64_t num_cols, int64_t nnz) {
  if (num_cols < 0 || nnz < 0) return 0;
  return gs::align_up((size_t)(num_cols > 0 ? num_cols : 1) * sizeof(unsigned int), 256) +
         gs::align_up((size_t)(nnz + 1) * sizeof(int64_t), 256) +
         gs::scan_workspace_bytes(nnz + 1);
}

int gs_weight_cdf_build(const int64_t* indptr, int64_t num_cols, const int64_t* indices,
                        int64_t num_rows, const float* probs, int64_t nnz, int64_t* cdf,
                        void* workspace, size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_cols >= 0 && nnz >= 0, "weight_cdf_build: negative size");
  GS_REQUIRE(cdf && (nnz == 0 || (indptr && probs)), "weight_cdf_build: null pointer");
  GS_REQUIRE(indices == nullptr || num_rows >= 0, "weight_cdf_build: negative num_rows");
  const size_t need = gs_weight_cdf_workspace_bytes(num_cols, nnz);
  if (workspace == nullptr || workspace_bytes < need) {
    set_error("weight_cdf_build workspace too small: %zu < %zu", workspace_bytes, need);
    return GS_ERR_WORKSPACE;
  }
  // bits that hold any row id below num_rows; ids too wide to share an entry
  // with a useful share stay in `indices`
  int row_bits = 0;
  if (indices != nullptr) {
    row_bits = 1;
    while (row_bits < 63 && (int64_t(1) << row_bits) < num_rows) ++row_bits;
    if (row_bits > kCdfMaxRowBits) row_bits = 0;
  }
  hipStream_t s = as_stream(stream);
  unsigned int* colmax = (unsigned int*)workspace;
  const size_t colmax_bytes =
      align_up((size_t)(num_cols > 0 ? num_cols : 1) * sizeof(unsigned int), 256);
  int64_t* prefix = (int64_t*)((char*)workspace + colmax_bytes);
  const size_t prefix_bytes = align_up((size_t)(nnz + 1) * sizeof(int64_t), 256);
  void* scan_ws = (char*)prefix + prefix_bytes;
  if (num_cols > 0)
    GS_LAUNCH("cdf_zero", s,
              cdf_zero_kernel<<<dim3((unsigned)ceil_div(num_cols, kBlock)), dim3(kBlock),
                                0, s>>>(colmax, num_cols));
  if (nnz > 0)
    GS_LAUNCH("cdf_colmax", s,
              cdf_colmax_kernel<<<dim3((unsigned)ceil_div(nnz, kCdfTile)), dim3(kBlock), 0,
                                  s>>>(indptr, num_cols, probs, nnz, colmax));
  GS_LAUNCH("cdf_quantise", s,
            cdf_quantise_kernel<<<dim3((unsigned)ceil_div(nnz + 1, kCdfTile)), dim3(kBlock),
                                  0, s>>>(indptr, num_cols, probs, nnz, colmax, prefix));
  const int rc = exclusive_scan_i64(prefix, prefix, nnz + 1, scan_ws,
                                    workspace_bytes - colmax_bytes - prefix_bytes, s);
  if (rc != GS_OK) return rc;
  GS_LAUNCH("cdf_pack", s,
            cdf_pack_kernel<<<dim3((unsigned)ceil_div(nnz > 0 ? nnz : 1, kCdfTile)),
                              dim3(kBlock), 0, s>>>(indptr, num_cols, indices, nnz, prefix,
                                                    row_bits, (uint64_t*)cdf));
  return GS_OK;
}

int gs_csc_col_sample_weighted_fill(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const float* probs, const int64_t* cdf,
    const int64_t* column_ids, int64_t num_items,
    int64_t fanout, int replace, uint64_t seed, uint64_t call_id,
    const int64_t* sub_indptr, const int64_t* col_span, const int64_t* cdf_offsets,
    void* cdf_scratch,
    int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    const int64_t* col_batch_ptr, int64_t num_col_batches, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items >= 0 && num_cols >= 0, "sample_weighted: negative size");
  GS_REQUIRE(col_batch_ptr == nullptr || num_col_batches >= 1,
             "sample_weighted: col_batch_ptr given but num_col_batches = %lld",
             (long long)num_col_batches);
  const ColumnLabels labels{col_batch_ptr, num_col_batches};
  GS_REQUIRE(fanout >= 0, "sample_weighted: negative fanout %lld", (long long)fanout);
  if (num_items == 0 || fanout == 0) return GS_OK;
  GS_REQUIRE(indptr && (probs || cdf) && sub_indptr && out_indices && out_select,
             "sample_weighted: null pointer");
  GS_REQUIRE(column_ids != nullptr || num_items <= num_cols,
             "sample_weighted: %lld items but the matrix has %lld columns",
             (long long)num_items, (long long)num_cols);
  const PhiloxKey key = make_key(seed, call_id);
  hipStream_t s = as_stream(stream);
  if (cdf != nullptr) {
    GS_REQUIRE(replace || fanout <= kMaxCdfFanout,
               "sample_weighted: fanout %lld > %d is not supported without replacement",
               (long long)fanout, kMaxCdfFanout);
    GS_REQUIRE(fanout <= INT32_MAX, "sample_weighted: fanout too large");
#define GS_CDF_ARGS                                                              \
  indptr, num_cols, indices, cdf, column_ids, num_items, (int)fanout, replace, \
      key, sub_indptr, out_coo_col, out_indices, out_select, labels, col_span, s
    // (every slot of the register arrays costs instructions in every draw whether it is
    // used or not: the common fan-outs get arrays of their own size)
    if (fanout <= 4) return launch_weighted_cdf<4>(GS_CDF_ARGS);
    if (fanout == 5) return launch_weighted_cdf<5>(GS_CDF_ARGS);
    if (fanout <= 8) return launch_weighted_cdf<8>(GS_CDF_ARGS);
    if (fanout <= 10) return launch_weighted_cdf<10>(GS_CDF_ARGS);
    if (fanout <= 12) return launch_weighted_cdf<12>(GS_CDF_ARGS);
    if (fanout <= 15) return launch_weighted_cdf<15>(GS_CDF_ARGS);
    if (fanout <= 16) return launch_weighted_cdf<16>(GS_CDF_ARGS);
    if (fanout <= 24) return launch_weighted_cdf<24>(GS_CDF_ARGS);
    if (fanout <= 32) return launch_weighted_cdf<32>(GS_CDF_ARGS);
    return launch_weighted_cdf<64>(GS_CDF_ARGS);
#undef GS_CDF_ARGS
    return GS_OK;
  }
  if (replace) {
    GS_REQUIRE(cdf_scratch, "sample_weighted: sampling with replacement needs the CDF scratch");
    GS_REQUIRE(column_ids == nullptr || cdf_offsets != nullptr,
               "sample_weighted: cdf_offsets are required with column_ids");
    GS_LAUNCH("sample_weighted_replace", s,
              sample_weighted_replace_kernel<<<dim3((unsigned)ceil_div(num_items * kWave, kBlock)),
                                               dim3(kBlock), 0, s>>>(
                  indptr, num_cols, indices, probs, column_ids, num_items, fanout,
                  key, sub_indptr, cdf_offsets, (uint64_t*)cdf_scratch, out_coo_col,
                  out_indices, out_select, labels));
    return GS_OK;
  }
  GS_REQUIRE(fanout <= 64,
             "sample_weighted: fanout %lld > 64 is not supported without replacement",
             (long long)fanout);
  const int threads = fanout <= 32 ? kBlock : kBlock / 2;
  const size_t lds = (size_t)fanout * threads * (sizeof(double) + sizeof(int));
  static bool raised = false;
  if (!raised) {
    GS_HIP(hipFuncSetAttribute((const void*)sample_weighted_kernel,
                               hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
    raised = true;
  }
  const int64_t blocks = ceil_div(num_items * kWave, threads);
  GS_LAUNCH("sample_weighted", s,
            sample_weighted_kernel<<<dim3((unsigned)blocks), dim3(threads), lds, s>>>(
                indptr, num_cols, indices, probs, column_ids, num_items,
                (int)fanout, key, sub_indptr, out_coo_col, out_indices,
                out_select, labels));
  return GS_OK;
}

size_t gs_list_sample_workspace_bytes(int64_t n, int64_t num_segments) {
  if (n < 0 || num_segments < 1) return 0;
  return gs::carve_list(nullptr, n, num_segments).total;
}

int gs_list_sample_weighted_count(const int64_t* range, int64_t n,
                                  int64_t num_segments, int64_t num_picks,
                                  int replace, int64_t* out_range,
                                  void* workspace, size_t workspace_bytes,
                                  gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0 && num_segments >= 1 && num_picks >= 0,
             "list_sample_count: bad sizes");
  GS_REQUIRE(range != nullptr || num_segments == 1,
             "list_sample_count: %lld segments need a range array", (long long)num_segments);
  GS_REQUIRE(out_range, "list_sample_count: null out_range");
  ListWs w = carve_list(workspace, n, num_segments);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("list_sample workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  if (num_segments < kBlock) {
    GS_LAUNCH("list_counts", s,
              list_offsets_kernel<<<dim3(1), dim3(kBlock), 0, s>>>(range, n, num_segments,
                                                                   num_picks, replace, out_range));
    return GS_OK;
  }
  GS_LAUNCH("list_counts", s,
            list_counts_kernel<<<dim3((unsigned)ceil_div(num_segments + 1, kBlock)),
                                 dim3(kBlock), 0, s>>>(range, n, num_segments,
                                                       num_picks, replace, out_range));
  return exclusive_scan_i64(out_range, out_range, num_segments + 1, w.scan_ws,
                            w.scan_ws_bytes, s);
}

int gs_list_sample_weighted_fill(const float* probs, const int64_t* range,
                                 int64_t n, int64_t num_segments,
                                 int64_t num_picks, int replace, uint64_t seed,
                                 uint64_t call_id, const int64_t* out_range,
                                 int64_t total_picks, int64_t* out_index,
                                 void* workspace, size_t workspace_bytes,
                                 gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0 && num_segments >= 1 && num_picks >= 0 && total_picks >= 0,
             "list_sample_fill: bad sizes");
  if (total_picks == 0 || n == 0) return GS_OK;
  GS_REQUIRE(probs && out_range && out_index, "list_sample_fill: null pointer");
  GS_REQUIRE(range != nullptr || num_segments == 1,
             "list_sample_fill: %lld segments need a range array", (long long)num_segments);
  ListWs w = carve_list(workspace, n, num_segments);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("list_sample workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  const PhiloxKey key = make_key(seed, call_id);
  hipStream_t s = as_stream(stream);
  if (replace) {
    GS_LAUNCH("list_replace", s,
              list_replace_kernel<<<dim3((unsigned)ceil_div(num_segments * kWave, kBlock)),
                                    dim3(kBlock), 0, s>>>(
                  probs, range, n, num_segments, num_picks, key, out_range,
                  w.keys_in, out_index));
    return GS_OK;
  }
  if (num_picks >= 1 && num_picks <= kSelMaxPicks && list_can_select(n, num_segments)) {
    // few items per thread while that still fills the device, else sixteen (fewer
    // work-groups meet at the same histogram bins)
    const bool deep = n >= (int64_t(1) << 21);
    const dim3 tiles((unsigned)ceil_div(n, kBlock * (deep ? 16 : 4)));
    GS_LAUNCH("list_zero", s,
              table_fill_kernel32<<<dim3((unsigned)ceil_div((int64_t)w.sel_words, kBlock * 8)),
                                    dim3(kBlock), 0, s>>>(w.sel_block, (int64_t)w.sel_words));
#define GS_SEL_LAUNCH(name, kernel, ...)                                              \
  GS_LAUNCH(name, s,                                                                  \
            if (deep) kernel<16><<<tiles, dim3(kBlock), 0, s>>>(__VA_ARGS__);         \
            else kernel<4><<<tiles, dim3(kBlock), 0, s>>>(__VA_ARGS__))
    GS_SEL_LAUNCH("list_keys", list_keys_hist_kernel, probs, range, n, num_segments, key,
                  w.keys_in, w.hist1);
    GS_SEL_LAUNCH("list_refine", list_refine_kernel, range, n, num_segments, num_picks,
                  w.keys_in, w.hist1, w.hist2);
    GS_SEL_LAUNCH("list_emit", list_emit_kernel, range, n, num_segments, num_picks, w.keys_in,
                  w.hist1, w.hist2, w.counts, w.win_key, w.win_idx, w.keys_out, w.vals_out);
#undef GS_SEL_LAUNCH
    GS_LAUNCH("list_finish", s,
              list_finish_kernel<<<dim3((unsigned)num_segments, kFinishSplit), dim3(kFinishThreads), 0, s>>>(
                  range, n, num_picks, w.counts, w.win_key, w.win_idx, w.keys_out, w.vals_out,
                  out_range, out_index));
    return GS_OK;
  }
  GS_LAUNCH("list_keys", s,
            list_keys_kernel<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, s>>>(
                probs, n, key, w.keys_in, w.vals_in));
  size_t temp = w.sort_ws_bytes;
  {
    ProfScope ps("list_sort", s);
    if (num_segments == 1) {
      GS_HIP(rocprim::radix_sort_pairs(w.sort_ws, temp, w.keys_in, w.keys_out,
                                       w.vals_in, w.vals_out, (size_t)n, 0, 64, s));
    } else {
      GS_HIP(rocprim::segmented_radix_sort_pairs(
          w.sort_ws, temp, w.keys_in, w.keys_out, w.vals_in, w.vals_out,
          (size_t)n, (unsigned)num_segments, range, range + 1, 0, 64, s));
    }
  }
  GS_LAUNCH("list_take", s,
            list_take_kernel<<<dim3((unsigned)ceil_div(total_picks, kBlock)),
                               dim3(kBlock), 0, s>>>(w.vals_out, range, n,
                                                     num_segments, num_picks,
                                                     out_range, total_picks,
                                                     out_index));
  return GS_OK;
}

}  // extern "C"
