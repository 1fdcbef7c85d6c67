// edgeops.hip -- edge-wise compute operators of layer-wise samplers:
// generalized SDDMM (a value per edge from its endpoints), generalized SpMM
// (reduce edge values onto rows or columns) and their fusions (sum of squares,
// sum of e / u, two u-op-v products in one sweep).
//
// Endpoint convention (same as the reference, src/cuda/sddmm.cu:37-38,134-135):
// on COO  src = row[e], dst = col[e]; on a compressed matrix src = indices[e]
// and dst = the segment of indptr that holds e.  Targets: 0 = src ("u"),
// 1 = edge, 2 = dst ("v").  All kernels are memory bound; features are scalar
// in every sampler that uses them, so the fast paths are the feature-length-1
// ones and the general-length paths favour simplicity.
#include "common.h"
#include "scan.h"

namespace gs {

enum { kOpAdd = 0, kOpSub, kOpMul, kOpDiv, kOpCopyLhs, kOpCopyRhs, kOpDot };
enum { kReduceSum = 0, kReduceMax, kReduceMin };

template <typename T>
__device__ __forceinline__ T apply_op(int op, const T* l, const T* r,
                                      int64_t reduce_size) {
  switch (op) {
    case kOpAdd: return l[0] + r[0];
    case kOpSub: return l[0] - r[0];
    case kOpMul: return l[0] * r[0];
    case kOpDiv: return l[0] / r[0];
    case kOpCopyLhs: return l[0];
    case kOpCopyRhs: return r[0];
    default: {
      T acc = 0;
      for (int64_t k = 0; k < reduce_size; ++k) acc += l[k] * r[k];
      return acc;
    }
  }
}

__device__ __forceinline__ int64_t pick(int target, int64_t src, int64_t eid,
                                        int64_t dst) {
  return target == 0 ? src : (target == 1 ? eid : dst);
}

struct EdgeView {
  int compressed;      // 1: (indptr, indices), 0: (row, col)
  const int64_t* a;    // row | indptr
  const int64_t* b;    // col | indices
  int64_t num_major;   // segments of indptr
  const int64_t* edge_map;
  // Segments that the edges [e_first, e_last] of one work-group touch
  // (compressed form only): looked up once, on the scalar unit.
  __device__ __forceinline__ SegmentSpan span(int64_t e_first, int64_t e_last) const {
    if (!compressed) return SegmentSpan{0, 0};
    return segment_span(a, num_major, e_first, e_last);
  }
  __device__ __forceinline__ void endpoints(const SegmentSpan& sp, int64_t e, int64_t* src,
                                            int64_t* dst, int64_t* eid) const {
    if (compressed) {
      *src = b[e];
      *dst = sp.segment_at(a, e);
    } else {
      *src = a[e];
      *dst = b[e];
    }
    *eid = edge_map ? edge_map[e] : e;
  }
};

// A work-group handles kBlock * ITEMS consecutive elements of an
// [nnz, out_len] output.  On a compressed form ITEMS = kEdgeItems, so that the
// look-up of the segments its edges touch is paid once per 2048 elements; an
// edge list needs no look-up and runs with one element per thread.
constexpr int kEdgeItems = 8;

template <int ITEMS>
__device__ __forceinline__ SegmentSpan block_edge_span(const EdgeView& g, int64_t nnz,
                                                       int64_t out_len) {
  const int64_t idx0 = (int64_t)blockIdx.x * (kBlock * ITEMS);
  int64_t idx_last = idx0 + kBlock * ITEMS - 1;
  if (idx_last > nnz * out_len - 1) idx_last = nnz * out_len - 1;
  return g.span(idx0 / out_len, idx_last / out_len);
}

// ------------------------------------------------------------------ SDDMM
template <typename T, int ITEMS>
__global__ __launch_bounds__(kBlock) void sddmm_kernel(
    EdgeView g, int64_t nnz, int op, const T* __restrict__ lhs,
    const T* __restrict__ rhs, T* __restrict__ out, int lhs_target,
    int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
    int64_t reduce_size, const int64_t* __restrict__ lhs_off,
    const int64_t* __restrict__ rhs_off) {
  const int64_t idx0 = (int64_t)blockIdx.x * (kBlock * ITEMS);
  if (idx0 >= nnz * out_len) return;
  const SegmentSpan sp = block_edge_span<ITEMS>(g, nnz, out_len);
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int64_t idx = idx0 + j * kBlock + threadIdx.x;
    if (idx >= nnz * out_len) break;
    const int64_t e = idx / out_len, f = idx - e * out_len;
    int64_t src, dst, eid;
    g.endpoints(sp, e, &src, &dst, &eid);
    const int64_t lf = lhs_off ? lhs_off[f] : f, rf = rhs_off ? rhs_off[f] : f;
    const T* l = op == kOpCopyRhs
                     ? nullptr
                     : lhs + pick(lhs_target, src, eid, dst) * lhs_len + lf * reduce_size;
    const T* r = op == kOpCopyLhs
                     ? nullptr
                     : rhs + pick(rhs_target, src, eid, dst) * rhs_len + rf * reduce_size;
    out[eid * out_len + f] = apply_op<T>(op, l, r, reduce_size);
  }
}

// Two SDDMMs (u op v) that share one edge sweep.
template <typename T, int ITEMS>
__global__ __launch_bounds__(kBlock) void fused_u_op_v_kernel(
    EdgeView g, int64_t nnz, int op, const T* __restrict__ lhs1,
    const T* __restrict__ rhs1, T* __restrict__ out1,
    const T* __restrict__ lhs2, const T* __restrict__ rhs2,
    T* __restrict__ out2, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
    int64_t reduce_size, const int64_t* __restrict__ lhs_off,
    const int64_t* __restrict__ rhs_off) {
  const int64_t idx0 = (int64_t)blockIdx.x * (kBlock * ITEMS);
  if (idx0 >= nnz * out_len) return;
  const SegmentSpan sp = block_edge_span<ITEMS>(g, nnz, out_len);
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int64_t idx = idx0 + j * kBlock + threadIdx.x;
    if (idx >= nnz * out_len) break;
    const int64_t e = idx / out_len, f = idx - e * out_len;
    int64_t src, dst, eid;
    g.endpoints(sp, e, &src, &dst, &eid);
    const int64_t lf = (lhs_off ? lhs_off[f] : f) * reduce_size;
    const int64_t rf = (rhs_off ? rhs_off[f] : f) * reduce_size;
    out1[eid * out_len + f] = apply_op<T>(op, lhs1 + src * lhs_len + lf,
                                          rhs1 + dst * rhs_len + rf, reduce_size);
    out2[eid * out_len + f] = apply_op<T>(op, lhs2 + src * lhs_len + lf,
                                          rhs2 + dst * rhs_len + rf, reduce_size);
  }
}

// ------------------------------------------------------------------- SpMM
// Value an edge contributes: kind 0 = op(u, e), 1 = e * e, 2 = e / u.
template <typename T>
__device__ __forceinline__ T edge_value(int kind, int op, const T* u, const T* e) {
  if (kind == 1) return e[0] * e[0];
  if (kind == 2) return e[0] / u[0];
  return apply_op<T>(op, u, e, 1);
}

__device__ __forceinline__ void atomic_reduce(float* addr, float v, int reduce) {
  if (reduce == kReduceSum) {
    unsafeAtomicAdd(addr, v);
    return;
  }
  unsigned int* p = (unsigned int*)addr;
  unsigned int old = *p;
  for (;;) {
    float cur = __uint_as_float(old);
    bool better = reduce == kReduceMax ? v > cur : v < cur;
    if (!better) return;
    unsigned int prev = atomicCAS(p, old, __float_as_uint(v));
    if (prev == old) return;
    old = prev;
  }
}

// Coordinate form: one thread per (edge, feature), atomics onto the output.
__global__ __launch_bounds__(kBlock) void spmm_coo_kernel(
    const int64_t* __restrict__ row, const int64_t* __restrict__ col,
    const int64_t* __restrict__ edge_map, int64_t nnz, int kind, int op,
    int reduce, const float* __restrict__ ufeat, const float* __restrict__ efeat,
    float* out, int u_target, int64_t ufeat_len, int64_t efeat_len,
    int64_t out_len, const int64_t* __restrict__ u_off,
    const int64_t* __restrict__ e_off) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= nnz * out_len) return;
  const int64_t e = idx / out_len, f = idx - e * out_len;
  const int64_t src = u_target == 0 ? row[e] : col[e];
  const int64_t dst = u_target == 0 ? col[e] : row[e];
  const int64_t eid = edge_map ? edge_map[e] : e;
  const float* u = ufeat ? ufeat + src * ufeat_len + (u_off ? u_off[f] : f) : nullptr;
  const float* ev = efeat ? efeat + eid * efeat_len + (e_off ? e_off[f] : f) : nullptr;
  atomic_reduce(out + dst * out_len + f, edge_value<float>(kind, op, u, ev), reduce);
}

// Second pass of arg-max / arg-min in coordinate form: the edge whose value
// equals the reduced output records its source and edge id.
__global__ __launch_bounds__(kBlock) void spmm_coo_arg_kernel(
    const int64_t* __restrict__ row, const int64_t* __restrict__ col,
    const int64_t* __restrict__ edge_map, int64_t nnz, int op,
    const float* __restrict__ ufeat, const float* __restrict__ efeat,
    const float* __restrict__ out, int64_t* arg_u, int64_t* arg_e, int u_target,
    int64_t ufeat_len, int64_t efeat_len, int64_t out_len,
    const int64_t* __restrict__ u_off, const int64_t* __restrict__ e_off) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= nnz * out_len) return;
  const int64_t e = idx / out_len, f = idx - e * out_len;
  const int64_t src = u_target == 0 ? row[e] : col[e];
  const int64_t dst = u_target == 0 ? col[e] : row[e];
  const int64_t eid = edge_map ? edge_map[e] : e;
  const float* u = ufeat ? ufeat + src * ufeat_len + (u_off ? u_off[f] : f) : nullptr;
  const float* ev = efeat ? efeat + eid * efeat_len + (e_off ? e_off[f] : f) : nullptr;
  if (edge_value<float>(0, op, u, ev) == out[dst * out_len + f]) {
    if (arg_u) arg_u[dst * out_len + f] = src;
    if (arg_e) arg_e[dst * out_len + f] = eid;
  }
}

// Compressed form, scalar features: a group of G lanes per segment strides over
// its edges and reduces with shuffles -- no atomics, hubs spread over a wave.
template <int G>
__global__ __launch_bounds__(kBlock) void spmm_csc_scalar_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices,
    const int64_t* __restrict__ edge_map, int64_t num_major, int kind, int op,
    int reduce, const float* __restrict__ ufeat, const float* __restrict__ efeat,
    float* __restrict__ out, int64_t* __restrict__ arg_u,
    int64_t* __restrict__ arg_e) {
  const int lane = threadIdx.x & (G - 1);
  const int64_t c = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / G;
  if (c >= num_major) return;
  const int64_t lo = indptr[c], hi = indptr[c + 1];
  // reduction starts from 0: outputs are zero-initialised accumulators
  float acc = 0.f;
  int64_t best_u = 0, best_e = 0;
  for (int64_t i = lo + lane; i < hi; i += G) {
    const int64_t eid = edge_map ? edge_map[i] : i;
    const int64_t cid = indices[i];
    const float v = edge_value<float>(kind, op, ufeat ? ufeat + cid : nullptr,
                                      efeat ? efeat + eid : nullptr);
    if (reduce == kReduceSum) {
      acc += v;
    } else if (reduce == kReduceMax ? v > acc : v < acc) {
      acc = v;
      best_u = cid;
      best_e = eid;
    }
  }
#pragma unroll
  for (int d = G / 2; d > 0; d >>= 1) {
    const float o = __shfl_down(acc, d, G);
    const int64_t ou = __shfl_down(best_u, d, G);
    const int64_t oe = __shfl_down(best_e, d, G);
    if (reduce == kReduceSum) {
      acc += o;
    } else if (reduce == kReduceMax ? o > acc : o < acc) {
      acc = o;
      best_u = ou;
      best_e = oe;
    }
  }
  if (lane == 0) {
    out[c] += acc;
    if (reduce != kReduceSum) {
      if (arg_u) arg_u[c] = best_u;
      if (arg_e) arg_e[c] = best_e;
    }
  }
}

// Compressed form, general feature length: one thread per (segment, feature).
__global__ __launch_bounds__(kBlock) void spmm_csc_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices,
    const int64_t* __restrict__ edge_map, int64_t num_major, int kind, int op,
    int reduce, const float* __restrict__ ufeat, const float* __restrict__ efeat,
    float* __restrict__ out, int64_t* __restrict__ arg_u,
    int64_t* __restrict__ arg_e, int64_t ufeat_len, int64_t efeat_len,
    int64_t out_len, const int64_t* __restrict__ u_off,
    const int64_t* __restrict__ e_off) {
  const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= num_major * out_len) return;
  const int64_t c = idx / out_len, f = idx - c * out_len;
  const int64_t uf = u_off ? u_off[f] : f, ef = e_off ? e_off[f] : f;
  float acc = 0.f;
  int64_t best_u = 0, best_e = 0;
  for (int64_t i = indptr[c]; i < indptr[c + 1]; ++i) {
    const int64_t eid = edge_map ? edge_map[i] : i;
    const int64_t cid = indices[i];
    const float v =
        edge_value<float>(kind, op, ufeat ? ufeat + cid * ufeat_len + uf : nullptr,
                          efeat ? efeat + eid * efeat_len + ef : nullptr);
    if (reduce == kReduceSum) {
      acc += v;
    } else if (reduce == kReduceMax ? v > acc : v < acc) {
      acc = v;
      best_u = cid;
      best_e = eid;
    }
  }
  out[idx] += acc;
  if (reduce != kReduceSum) {
    if (arg_u) arg_u[idx] = best_u;
    if (arg_e) arg_e[idx] = best_e;
  }
}

// ------------------------------------------------- load-balanced scalar sums
// The sums of layer-wise samplers run over slices of power-law graphs: one
// column (or row) can hold a large share of all edges.  Both kernels below are
// edge-parallel, combine inside LDS what a tile of edges adds to the same
// output, and send one atomic per (tile, output) to memory.
constexpr int kSumItems = 8;
constexpr int kSumTile = kBlock * kSumItems;
constexpr int kSumSegs = 2048;   // segments one tile can accumulate in LDS
constexpr int kCooSlots = 4096;  // combining table of the coordinate kernel
constexpr int kDies = 8;         // accelerator dies of an MI355X, one L2 each
constexpr int64_t kPrivateMinEdges = 1 << 20;

// out[i] += sum of the per-die copies; the copies were zero-filled before.
__global__ __launch_bounds__(kBlock) void spmm_fold_kernel(
    const float* __restrict__ copies, int64_t n, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  float acc = 0.f;
#pragma unroll
  for (int d = 0; d < kDies; ++d) acc += copies[d * n + i];
  if (acc != 0.f) out[i] += acc;
}

__global__ __launch_bounds__(kBlock) void spmm_zero_kernel(float* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kBlock)
    p[i] = 0.f;
}

// Per-die copies pay off when there are many edges per output row.
static size_t private_bytes(int format, int64_t nnz, int64_t num_out) {
  if (format != GS_FMT_COO || nnz < kPrivateMinEdges || num_out <= 0 ||
      num_out > nnz / 4)
    return 0;
  return (size_t)kDies * (size_t)num_out * sizeof(float);
}

// Sum of v over the wavefront if every lane is active and targets the same
// output (then *uniform is set and lane 0 should add the result).
__device__ __forceinline__ float wave_sum_if_uniform(float v, int64_t target,
                                                     bool active, bool* uniform) {
  const int64_t t0 = wave_uniform_first(target);
  *uniform = __all(active && target == t0);
  if (!*uniform) return v;
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_down(v, d, kWave);
  return v;
}

// Compressed form: tile of consecutive edges; the segments it touches are
// consecutive, so LDS accumulators are indexed directly.  On large inputs a
// work-group takes kCscRounds tiles in a row: the look-up of the columns it
// covers (two dependent chains of loads over indptr) is then paid once per
// 8192 edges.
constexpr int kCscRounds = 4;

__global__ __launch_bounds__(kBlock) void spmm_csc_sum_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices,
    const int64_t* __restrict__ edge_map, int64_t num_major, int64_t nnz,
    int kind, int op, const float* __restrict__ ufeat,
    const float* __restrict__ efeat, float* out, int rounds) {
  __shared__ float acc[kSumSegs];
  __shared__ int64_t bounds[kSumSegs + 1];
  const int64_t tile_len = (int64_t)kSumTile * rounds;
  const int64_t tile0 = (int64_t)blockIdx.x * tile_len;
  const int64_t tile_end = tile0 + tile_len < nnz ? tile0 + tile_len : nnz;
  // A lane takes quads of neighbouring edges: item i of a round is edge
  //   base + (i / 4) * 4 * kBlock + 4 * lane + i % 4,
  // so that values which come straight from the edge array arrive as 16-byte loads.
  static_assert(kSumItems % 4 == 0, "a lane takes whole quads");
  auto edge_of = [](int64_t base, int i) {
    return base + (int64_t)(i >> 2) * (4 * kBlock) + 4 * (int)threadIdx.x + (i & 3);
  };
  const bool plain = edge_map == nullptr && ufeat == nullptr && efeat != nullptr;
  auto load_round = [&](int64_t base, float (&val)[kSumItems]) {
#pragma unroll
    for (int q = 0; q < kSumItems / 4; ++q) {
      const int64_t e = edge_of(base, 4 * q);
      if (plain && e + 3 < tile_end) {
        struct Quad {
          float v[4];
        } held;
        __builtin_memcpy(&held, efeat + e, sizeof(Quad));
#pragma unroll
        for (int j = 0; j < 4; ++j)
          val[4 * q + j] = edge_value<float>(kind, op, nullptr, &held.v[j]);
        continue;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        val[4 * q + j] = 0.f;
        if (e + j < tile_end) {
          const int64_t eid = edge_map ? edge_map[e + j] : e + j;
          val[4 * q + j] = edge_value<float>(kind, op, ufeat ? ufeat + indices[e + j] : nullptr,
                                             efeat ? efeat + eid : nullptr);
        }
      }
    }
  };
  // the first round's values before anything else: their loads are in flight
  // while the columns are looked up
  float val[kSumItems];
  load_round(tile0, val);
  // both look-ups on the scalar unit; a long column covers the whole tile, and
  // then the second one is a single comparison
  const int64_t c0 = segment_of(indptr, num_major, wave_uniform_first(tile0));
  const int64_t last = wave_uniform_first(tile_end - 1);
  const int64_t c1 = indptr[c0 + 1] > last
                         ? c0
                         : c0 + segment_of(indptr + c0, num_major - c0, last);
  const int64_t nseg = c1 - c0 + 1;
  const bool in_lds = nseg <= kSumSegs;
  if (in_lds) {
    for (int64_t j = threadIdx.x; j <= nseg; j += kBlock) {
      bounds[j] = indptr[c0 + j];
      if (j < nseg) acc[j] = 0.f;
    }
    __syncthreads();
  }
  for (int r = 0; r < rounds; ++r) {
    const int64_t base = tile0 + (int64_t)r * kSumTile;
    if (base >= tile_end) break;
    if (r > 0) load_round(base, val);
    // a round that lies inside one column (any column of 2048 edges or more
    // has such rounds): the lanes add their values up first, and the
    // wavefront sends one sum
    const int64_t round_last = base + kSumTile - 1 < tile_end - 1 ? base + kSumTile - 1
                                                                : tile_end - 1;
    const int64_t s_first = in_lds ? segment_of(bounds, nseg, wave_uniform_first(base))
                                   : segment_of(indptr + c0, nseg, wave_uniform_first(base));
    const int64_t s_next = in_lds ? bounds[s_first + 1] : indptr[c0 + s_first + 1];
    if (s_next > round_last) {
      float mine = 0.f;
#pragma unroll
      for (int i = 0; i < kSumItems; ++i) mine += val[i];   // inactive slots hold 0
#pragma unroll
      for (int d = kWave / 2; d > 0; d >>= 1) mine += __shfl_down(mine, d, kWave);
      if (lane_id() == 0) {
        if (in_lds) atomicAdd(&acc[s_first], mine);
        else unsafeAtomicAdd(out + c0 + s_first, mine);
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < kSumItems; ++i) {
      const int64_t e = edge_of(base, i);
      const bool active = e < tile_end;
      int64_t seg = 0;
      if (active)
        seg = in_lds ? segment_of(bounds, nseg, e) : segment_of(indptr + c0, nseg, e);
      bool uniform;
      const float total = wave_sum_if_uniform(val[i], seg, active, &uniform);
      if (uniform) {
        if (lane_id() == 0) {
          if (in_lds) atomicAdd(&acc[seg], total);
          else unsafeAtomicAdd(out + c0 + seg, total);
        }
      } else if (active) {
        if (in_lds) atomicAdd(&acc[seg], val[i]);
        else unsafeAtomicAdd(out + c0 + seg, val[i]);
      }
    }
  }
  if (!in_lds) return;
  __syncthreads();
  for (int64_t j = threadIdx.x; j < nseg; j += kBlock)
    if (acc[j] != 0.f) unsafeAtomicAdd(out + c0 + j, acc[j]);
}

// Coordinate form: outputs arrive in any order, so the tile combines them in
// a small LDS hash table; an edge that finds no slot within a few probes adds
// to memory directly.
__global__ __launch_bounds__(kBlock) void spmm_coo_sum_kernel(
    const int64_t* __restrict__ row, const int64_t* __restrict__ col,
    const int64_t* __restrict__ edge_map, int64_t nnz, int kind, int op,
    const float* __restrict__ ufeat, const float* __restrict__ efeat, float* out,
    int u_target, int64_t copy_stride, SliceView view) {
  __shared__ long long keys[kCooSlots];
  __shared__ float vals[kCooSlots];
  for (int j = threadIdx.x; j < kCooSlots; j += kBlock) {
    keys[j] = -1;
    vals[j] = 0.f;
  }
  __syncthreads();
  // consecutive work-groups run on consecutive dies: with copy_stride > 0 every
  // die adds to a copy of its own
  out += (int64_t)(blockIdx.x % kDies) * copy_stride;
  const int64_t tile0 = (int64_t)blockIdx.x * kSumTile;
  const int64_t* dst_ids = u_target == 0 ? col : row;
  const int64_t* src_ids = u_target == 0 ? row : col;
  // all loads of the tile first, so that they are in flight together
  // (with a view: the edges of a column slice that was never written, dst_ids
  // and efeat being the parent's arrays)
  SliceView::Run vrun{};
  vrun.split = INT64_MAX;  // no view: every edge at distance 0
  if (view.on() && tile0 < nnz)
    vrun = view.run(tile0, (tile0 + kSumTile < nnz ? tile0 + kSumTile : nnz) - 1);
  int64_t dst[kSumItems];
  float val[kSumItems];
#pragma unroll
  for (int i = 0; i < kSumItems; ++i) {
    const int64_t e = tile0 + i * kBlock + threadIdx.x;
    dst[i] = -1;
    val[i] = 0.f;
    if (e < nnz && vrun.near()) {
      const int64_t p = vrun.place(e);
      dst[i] = dst_ids[p];
      const int64_t eid = edge_map ? edge_map[p] : p;
      val[i] = edge_value<float>(kind, op, ufeat ? ufeat + src_ids[p] : nullptr,
                                 efeat ? efeat + eid : nullptr);
    }
  }
  if (!vrun.near()) {
#pragma unroll
    for (int i = 0; i < kSumItems; ++i) {
      const int64_t e = tile0 + i * kBlock + threadIdx.x;
      int64_t col, offset;  // (looked up by all lanes together, a lane past the end included)
      const int64_t p = view.position(vrun, e < nnz ? e : nnz - 1, &col, &offset);
      if (e < nnz) {
        dst[i] = dst_ids[p];
        val[i] = edge_value<float>(kind, op, ufeat ? ufeat + src_ids[p] : nullptr,
                                   efeat ? efeat + (edge_map ? edge_map[p] : p) : nullptr);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kSumItems; ++i) {
    if (dst[i] < 0) continue;
    uint32_t slot =
        (uint32_t)(((uint64_t)dst[i] * 0x9E3779B97F4A7C15ull) >> 40) & (kCooSlots - 1);
    bool placed = false;
    for (int probe = 0; probe < 8 && !placed; ++probe) {
      long long k = keys[slot];
      if (k == -1) k = (long long)atomicCAS((unsigned long long*)&keys[slot],
                                            ~0ull, (unsigned long long)dst[i]);
      if (k == -1 || k == (long long)dst[i]) {
        atomicAdd(&vals[slot], val[i]);
        placed = true;
      }
      slot = (slot + 1) & (kCooSlots - 1);
    }
    if (!placed) unsafeAtomicAdd(out + dst[i], val[i]);
  }
  __syncthreads();
  for (int j = threadIdx.x; j < kCooSlots; j += kBlock)
    if (keys[j] != -1) unsafeAtomicAdd(out + keys[j], vals[j]);
}

// ------------------------------------------- coordinate sums by row ranges
// Atomic adds to device memory are executed next to the memory, at a rate far
// below what the edges stream at, and a tile of a large slice rarely adds
// twice to the same row.  Large coordinate-form sums therefore go through a
// counting sort by row range instead: (1) every tile of edges counts its edges
// per range of kRangeRows rows, (2) a scan over the (range, tile) counts gives
// every tile a private place in every range, (3) the tile writes
// (row within range, value) pairs there, (4) a work-group sums a slice of one
// range in LDS and stores its kRangeRows partial sums, (5) the partial sums of
// a range are folded into the output.  Every pass streams; none uses an atomic
// on device memory.  The floor of pass 4 is the rate of fp32 adds in LDS
// (about a quarter of the integer rate), not memory.
constexpr int kRangeShift = 13;
constexpr int kRangeRows = 1 << kRangeShift;  // 32 KB of LDS accumulators
constexpr int kMaxRanges = 1024;
constexpr int kPartThreads = 512;
constexpr int kPartItems = 8;
constexpr int kPartTile = kPartThreads * kPartItems;
constexpr int kPartMaxRounds = 8;
constexpr int kSliceEntries = 32768;  // (row, value) pairs one work-group sums
constexpr int kSliceItems = 8;
// The accumulators of a range take 64 KB of LDS, so two work-groups share a
// compute unit: 1024 threads each keep all its wavefront slots busy.
constexpr int kAccThreads = 1024;

struct RowRangePlan {
  int64_t ranges = 0, tiles = 0, max_units = 0;
  int rounds = 1;  // sub-tiles of kPartTile edges one work-group of the partition passes takes
  size_t off_offsets = 0, off_scan = 0, scan_bytes = 0, off_entries = 0,
         off_unit_start = 0, off_partial = 0, total = 0;
};

// Worth it when the slice is large and rows repeat; empty plan otherwise.
static RowRangePlan row_range_plan(int format, int64_t nnz, int64_t num_out) {
  RowRangePlan p;
  if (format != GS_FMT_COO || nnz < kPrivateMinEdges ||
      nnz >= ((int64_t)1 << 31) || num_out <= 0 || num_out > nnz / 4 ||
      ceil_div(num_out, kRangeRows) > kMaxRanges)
    return p;
  p.ranges = ceil_div(num_out, kRangeRows);
  // The (range, tile) table costs a strided 8-byte access per cell in both
  // partition passes: once there are work-groups to spare a tile grows to up
  // to eight sub-tiles, which shrinks the table by as much.
  int64_t rounds = nnz / ((int64_t)kPartTile * 8192);
  p.rounds = (int)(rounds < 1 ? 1 : rounds > kPartMaxRounds ? kPartMaxRounds : rounds);
  p.tiles = ceil_div(nnz, (int64_t)kPartTile * p.rounds);
  p.max_units = nnz / kSliceEntries + p.ranges;
  auto take = [&p](size_t bytes) {
    const size_t at = p.total;
    p.total += (bytes + 255) / 256 * 256;
    return at;
  };
  const int64_t cells = p.ranges * p.tiles + 1;
  p.off_offsets = take((size_t)cells * sizeof(int64_t));
  p.scan_bytes = scan_workspace_bytes(cells);
  p.off_scan = take(p.scan_bytes);
  p.off_entries = take((size_t)nnz * sizeof(uint2));
  p.off_unit_start = take((size_t)(p.ranges + 1) * sizeof(int64_t));
  p.off_partial = take((size_t)p.max_units * kRangeRows * sizeof(float));
  return p;
}

// counts[range * tiles + tile] = edges of the tile whose target lies in range
// Lanes of the wavefront that hold the same value (of `bits` bits) as this one,
// among the valid ones: one ballot per bit.  Many lanes of a wave meet at the
// same few counters here (a tile's edges fall into a few dozen row ranges, and
// the range that holds the hubs' rows draws most of them): the first lane of a
// set of peers sends one atomic for all of them, where 64 single ones to the
// same LDS word are taken one after another.  Every lane must call this.
constexpr int kPeerBits = 6;  // up to 64 ranges: worth the ballots (one per bit of the range)
__device__ __forceinline__ uint64_t wave_peers(int value, int bits, bool valid) {
  uint64_t peers = __ballot(valid);
  for (int b = 0; b < bits; ++b) {
    const bool bit = (value >> b) & 1;
    const uint64_t m = __ballot(bit);
    peers &= bit ? m : ~m;
  }
  return peers;
}

// With a view the edges are those of a column slice that was never written:
// dst_ids and efeat are then the parent's arrays (see SliceView).
__device__ __forceinline__ SliceView::Run view_run(const SliceView& view, int64_t tile0,
                                                   int64_t tile, int64_t nnz) {
  if (!view.on()) {  // every edge at distance 0
    SliceView::Run r{};
    r.split = INT64_MAX;
    return r;
  }
  const int64_t stop = tile0 + tile < nnz ? tile0 + tile : nnz;
  return view.run(tile0, stop - 1);
}

template <typename IdT>
__global__ __launch_bounds__(kPartThreads) void rowsum_hist_kernel(
    const IdT* __restrict__ dst_ids, int64_t nnz, int64_t num_out, int ranges, int range_bits,
    int64_t tiles, int rounds, int64_t* __restrict__ counts, SliceView view) {
  __shared__ int hist[kMaxRanges];
  for (int j = threadIdx.x; j < ranges; j += kPartThreads) hist[j] = 0;
  __syncthreads();
  for (int r = 0; r < rounds; ++r) {
    const int64_t tile0 = ((int64_t)blockIdx.x * rounds + r) * kPartTile;
    if (tile0 >= nnz) break;
    const SliceView::Run vrun = view_run(view, tile0, kPartTile, nnz);
    int64_t dst[kPartItems];
    if (vrun.near()) {  // (no view: distance 0)
#pragma unroll
      for (int i = 0; i < kPartItems; ++i) {
        const int64_t e = tile0 + i * kPartThreads + threadIdx.x;
        dst[i] = e < nnz ? (int64_t)dst_ids[vrun.place(e)] : -1;
      }
    } else {
#pragma unroll
      for (int i = 0; i < kPartItems; ++i) {
        const int64_t e = tile0 + i * kPartThreads + threadIdx.x;
        int64_t col, offset;  // (looked up by all lanes together, a lane past the end included)
        const int64_t p = view.position(vrun, e < nnz ? e : nnz - 1, &col, &offset);
        dst[i] = e < nnz ? (int64_t)dst_ids[p] : -1;
      }
    }
#pragma unroll
    for (int i = 0; i < kPartItems; ++i) {
      const bool valid = dst[i] >= 0 && dst[i] < num_out;
      const int range = valid ? (int)(dst[i] >> kRangeShift) : 0;
      if (range_bits > kPeerBits) {  // many ranges: lanes rarely meet, one atomic each
        if (valid) atomicAdd(&hist[range], 1);
        continue;
      }
      const uint64_t peers = wave_peers(range, range_bits, valid);
      if (valid && (peers & ((1ull << lane_id()) - 1ull)) == 0)  // the first of its peers
        atomicAdd(&hist[range], __popcll(peers));
    }
  }
  __syncthreads();
  for (int j = threadIdx.x; j < ranges; j += kPartThreads)
    counts[(int64_t)j * tiles + blockIdx.x] = hist[j];
  if (blockIdx.x == 0 && threadIdx.x == 0) counts[(int64_t)ranges * tiles] = 0;
}

// A sub-tile is kept small (4096 edges) so that several work-groups share a
// compute unit and the loads of one overlap the stores of another; what a tile
// sends to one range is a contiguous run, filled within a few microseconds, so
// the 8-byte stores merge into whole lines in L2.  A pair keeps its range above
// the row bits (the accumulate pass masks it off).
template <typename IdT>
__global__ __launch_bounds__(kPartThreads) void rowsum_scatter_kernel(
    const IdT* __restrict__ dst_ids, const int64_t* __restrict__ src_ids,
    const int64_t* __restrict__ edge_map, int64_t nnz, int64_t num_out, int kind,
    int op, const float* __restrict__ ufeat, const float* __restrict__ efeat,
    int ranges, int range_bits, int64_t tiles, int rounds,
    const int64_t* __restrict__ offsets, uint2* __restrict__ entries, SliceView view) {
  __shared__ unsigned cursor[kMaxRanges];  // next free place of the tile per range
  for (int j = threadIdx.x; j < ranges; j += kPartThreads)
    cursor[j] = (unsigned)offsets[(int64_t)j * tiles + blockIdx.x];
  __syncthreads();
  for (int r = 0; r < rounds; ++r) {
    const int64_t tile0 = ((int64_t)blockIdx.x * rounds + r) * kPartTile;
    if (tile0 >= nnz) break;
    const SliceView::Run vrun = view_run(view, tile0, kPartTile, nnz);
    int64_t dst[kPartItems];
    float val[kPartItems];
    const bool shifted = vrun.near();  // the same in every lane (no view: distance 0)
#pragma unroll
    for (int i = 0; i < kPartItems; ++i) {
      const int64_t e = tile0 + i * kPartThreads + threadIdx.x;
      dst[i] = -1;
      val[i] = 0.f;
      if (e < nnz && shifted) {
        const int64_t p = vrun.place(e);
        dst[i] = (int64_t)dst_ids[p];
        const int64_t eid = edge_map ? edge_map[p] : p;
        val[i] = edge_value<float>(kind, op, ufeat ? ufeat + src_ids[p] : nullptr,
                                   efeat ? efeat + eid : nullptr);
      }
    }
    if (!shifted) {
#pragma unroll
      for (int i = 0; i < kPartItems; ++i) {
        const int64_t e = tile0 + i * kPartThreads + threadIdx.x;
        int64_t col, offset;  // (looked up by all lanes together, a lane past the end included)
        const int64_t p = view.position(vrun, e < nnz ? e : nnz - 1, &col, &offset);
        if (e < nnz) {
          dst[i] = (int64_t)dst_ids[p];
          const int64_t eid = edge_map ? edge_map[p] : p;
          val[i] = edge_value<float>(kind, op, ufeat ? ufeat + src_ids[p] : nullptr,
                                     efeat ? efeat + eid : nullptr);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kPartItems; ++i) {
      const bool valid = dst[i] >= 0 && dst[i] < num_out;
      const int range = valid ? (int)(dst[i] >> kRangeShift) : 0;
      if (range_bits > kPeerBits) {
        if (valid)
          entries[atomicAdd(&cursor[range], 1u)] =
              make_uint2((unsigned)dst[i], __float_as_uint(val[i]));
        continue;
      }
      const uint64_t peers = wave_peers(range, range_bits, valid);
      const uint64_t before = peers & ((1ull << lane_id()) - 1ull);
      unsigned base = 0;
      if (valid && before == 0) base = atomicAdd(&cursor[range], (unsigned)__popcll(peers));
      // the first of the peers took places for all of them
      base = __shfl(base, valid ? __ffsll((long long)peers) - 1 : lane_id(), kWave);
      if (valid)
        entries[base + __popcll(before)] = make_uint2((unsigned)dst[i], __float_as_uint(val[i]));
    }
  }
}

// unit_start[r] = first work unit (slice of kSliceEntries pairs) of range r
__global__ __launch_bounds__(kMaxRanges) void rowsum_units_kernel(
    const int64_t* __restrict__ offsets, int ranges, int64_t tiles,
    int64_t* __restrict__ unit_start) {
  __shared__ int64_t smem[kMaxRanges / kWave + 1];
  const int r = threadIdx.x;
  int64_t units = 0;
  if (r < ranges) {
    const int64_t n = offsets[(int64_t)(r + 1) * tiles] - offsets[(int64_t)r * tiles];
    units = ceil_div_dev(n, (int64_t)kSliceEntries);
  }
  int64_t total;
  const int64_t before = block_exclusive_sum<int64_t, kMaxRanges>(units, smem, &total);
  if (r < ranges) unit_start[r] = before;
  if (r == 0) unit_start[ranges] = total;
}

__global__ __launch_bounds__(kAccThreads) void rowsum_accumulate_kernel(
    const uint2* __restrict__ entries, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ unit_start, int ranges, int64_t tiles,
    float* __restrict__ partial) {
  // Accumulators in double: this part adds doubles in LDS at twice the rate of
  // floats (602 M entries: 1.55 against 3.05 ms), and a slice's sums then carry
  // no rounding of their own before they are rounded to float once.
  __shared__ double acc[kRangeRows];
  const int64_t u = blockIdx.x;
  if (u >= unit_start[ranges]) return;
  const int64_t r = segment_of(unit_start, ranges, u);
  const int64_t range_end = offsets[(r + 1) * tiles];
  const int64_t begin = offsets[r * tiles] + (u - unit_start[r]) * kSliceEntries;
  const int64_t end = begin + kSliceEntries < range_end ? begin + kSliceEntries : range_end;
  for (int j = threadIdx.x; j < kRangeRows; j += kAccThreads) acc[j] = 0.0;
  __syncthreads();
  for (int64_t base = begin; base < end; base += kAccThreads * kSliceItems) {
    uint2 item[kSliceItems];
#pragma unroll
    for (int i = 0; i < kSliceItems; ++i) {
      const int64_t p = base + i * kAccThreads + threadIdx.x;
      item[i] = p < end ? entries[p] : make_uint2(~0u, 0u);
    }
#pragma unroll
    for (int i = 0; i < kSliceItems; ++i)
      if (item[i].x != ~0u)
        atomicAdd(&acc[item[i].x & (kRangeRows - 1)], (double)__uint_as_float(item[i].y));
  }
  __syncthreads();
  float* mine = partial + u * kRangeRows;
  for (int j = threadIdx.x; j < kRangeRows; j += kAccThreads) mine[j] = (float)acc[j];
}

// out[row] += the row's partial sums over all slices of its range.  Ranges
// differ a lot in how many slices they have (the rows of hubs sit in one range
// and draw half of the edges), so the slices of a range are dealt out over
// gridDim.y work-groups per block of rows, which add their shares atomically.
constexpr int kFoldSplit = 8;

__global__ __launch_bounds__(kBlock) void rowsum_fold_kernel(
    const float* __restrict__ partial, const int64_t* __restrict__ unit_start,
    int64_t num_out, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= num_out) return;
  const int64_t r = i >> kRangeShift;  // uniform over the work-group
  const int64_t u1 = unit_start[r + 1], step = gridDim.y;
  const float* p = partial + (i & (kRangeRows - 1));
  float acc = 0.f;
  int64_t u = unit_start[r] + blockIdx.y;
  for (; u + 7 * step < u1; u += 8 * step) {  // eight loads in flight
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = p[(u + k * step) * kRangeRows];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc += v[k];
  }
  for (; u < u1; u += step) acc += p[u * kRangeRows];
  if (acc != 0.f) unsafeAtomicAdd(out + i, acc);
}

// dst_ids32: the same ids as dst_ids in 32 bits (a matrix's narrow copy), read
// instead when given.
static int row_range_sum(const RowRangePlan& p, const int64_t* dst_ids, const int32_t* dst_ids32,
                         const int64_t* src_ids, const int64_t* edge_map,
                         int64_t nnz, int64_t num_out, int kind, int op,
                         const float* ufeat, const float* efeat, float* out,
                         void* workspace, hipStream_t s, SliceView view = no_view()) {
  char* ws = (char*)workspace;
  int64_t* offsets = (int64_t*)(ws + p.off_offsets);
  uint2* entries = (uint2*)(ws + p.off_entries);
  int64_t* unit_start = (int64_t*)(ws + p.off_unit_start);
  float* partial = (float*)(ws + p.off_partial);
  const int ranges = (int)p.ranges;
  int range_bits = 0;
  while ((1 << range_bits) < ranges) ++range_bits;
  const dim3 tiles_grid((unsigned)p.tiles);
  if (dst_ids32)
    GS_LAUNCH("rowsum_hist", s,
              rowsum_hist_kernel<int32_t><<<tiles_grid, dim3(kPartThreads), 0, s>>>(
                  dst_ids32, nnz, num_out, ranges, range_bits, p.tiles, p.rounds, offsets, view));
  else
    GS_LAUNCH("rowsum_hist", s,
              rowsum_hist_kernel<int64_t><<<tiles_grid, dim3(kPartThreads), 0, s>>>(
                  dst_ids, nnz, num_out, ranges, range_bits, p.tiles, p.rounds, offsets, view));
  int rc = exclusive_scan_i64(offsets, offsets, p.ranges * p.tiles + 1,
                              ws + p.off_scan, p.scan_bytes, s);
  if (rc != GS_OK) return rc;
  if (dst_ids32)
    GS_LAUNCH("rowsum_scatter", s,
              rowsum_scatter_kernel<int32_t><<<tiles_grid, dim3(kPartThreads), 0, s>>>(
                  dst_ids32, src_ids, edge_map, nnz, num_out, kind, op, ufeat, efeat,
                  ranges, range_bits, p.tiles, p.rounds, offsets, entries, view));
  else
    GS_LAUNCH("rowsum_scatter", s,
              rowsum_scatter_kernel<int64_t><<<tiles_grid, dim3(kPartThreads), 0, s>>>(
                  dst_ids, src_ids, edge_map, nnz, num_out, kind, op, ufeat, efeat,
                  ranges, range_bits, p.tiles, p.rounds, offsets, entries, view));
  GS_LAUNCH("rowsum_units", s,
            rowsum_units_kernel<<<dim3(1), dim3(kMaxRanges), 0, s>>>(
                offsets, ranges, p.tiles, unit_start));
  GS_LAUNCH("rowsum_accumulate", s,
            rowsum_accumulate_kernel<<<dim3((unsigned)p.max_units),
                                       dim3(kAccThreads), 0, s>>>(
                entries, offsets, unit_start, ranges, p.tiles, partial));
  GS_LAUNCH("rowsum_fold", s,
            rowsum_fold_kernel<<<dim3((unsigned)ceil_div(num_out, kBlock), kFoldSplit),
                                 dim3(kBlock), 0, s>>>(partial, unit_start,
                                                       num_out, out));
  return GS_OK;
}

static int check_view(int format, const int64_t* a, const int64_t* b,
                      int64_t num_major, int64_t nnz, const char* who) {
  GS_REQUIRE(format == GS_FMT_COO || format == GS_FMT_COMPRESSED,
             "%s: unknown format %d", who, format);
  GS_REQUIRE(nnz >= 0 && num_major >= 0, "%s: negative size", who);
  GS_REQUIRE(nnz == 0 || (a && b), "%s: null structure pointer", who);
  return GS_OK;
}

static int spmm_launch(int format, const int64_t* a, const int64_t* b,
                       int64_t num_major, int64_t nnz, const int64_t* edge_map,
                       int kind, int op, int reduce, const float* ufeat,
                       const float* efeat, float* out, int64_t* arg_u,
                       int64_t* arg_e, int u_target, int64_t ufeat_len,
                       int64_t efeat_len, int64_t out_len, const int64_t* u_off,
                       const int64_t* e_off, int64_t num_out, void* workspace,
                       size_t workspace_bytes, hipStream_t s) {
  if (nnz == 0 || out_len == 0) return GS_OK;
  const bool scalar = out_len == 1 && (ufeat == nullptr || ufeat_len == 1) &&
                      (efeat == nullptr || efeat_len == 1);
  if (scalar && reduce == kReduceSum) {
    const dim3 grid((unsigned)ceil_div(nnz, kSumTile));
    if (format == GS_FMT_COO) {
      const RowRangePlan plan = row_range_plan(format, nnz, num_out);
      if (plan.total > 0 && workspace != nullptr && workspace_bytes >= plan.total)
        return row_range_sum(plan, u_target == 0 ? b : a, nullptr, u_target == 0 ? a : b,
                             edge_map, nnz, num_out, kind, op, ufeat, efeat, out,
                             workspace, s);
      const size_t need = private_bytes(format, nnz, num_out);
      if (need > 0 && workspace != nullptr && workspace_bytes >= need) {
        float* copies = (float*)workspace;
        const int64_t total = (int64_t)kDies * num_out;
        int64_t zb = ceil_div(total, kBlock * 4);
        if (zb > 4096) zb = 4096;
        GS_LAUNCH("spmm_zero", s,
                  spmm_zero_kernel<<<dim3((unsigned)zb), dim3(kBlock), 0, s>>>(
                      copies, total));
        GS_LAUNCH("spmm_coo_sum", s,
                  spmm_coo_sum_kernel<<<grid, dim3(kBlock), 0, s>>>(
                      a, b, edge_map, nnz, kind, op, ufeat, efeat, copies,
                      u_target, num_out, no_view()));
        GS_LAUNCH("spmm_fold", s,
                  spmm_fold_kernel<<<dim3((unsigned)ceil_div(num_out, kBlock)),
                                     dim3(kBlock), 0, s>>>(copies, num_out, out));
        return GS_OK;
      }
      GS_LAUNCH("spmm_coo_sum", s,
                spmm_coo_sum_kernel<<<grid, dim3(kBlock), 0, s>>>(
                    a, b, edge_map, nnz, kind, op, ufeat, efeat, out, u_target,
                    (int64_t)0, no_view()));
    } else {
      // four tiles per work-group once there are work-groups to spare
      const int rounds = nnz >= ((int64_t)kSumTile * kCscRounds) * 8192 ? kCscRounds : 1;
      GS_LAUNCH("spmm_csc_sum", s,
                spmm_csc_sum_kernel<<<dim3((unsigned)ceil_div(nnz, (int64_t)kSumTile * rounds)),
                                      dim3(kBlock), 0, s>>>(
                    a, b, edge_map, num_major, nnz, kind, op, ufeat, efeat, out, rounds));
    }
    return GS_OK;
  }
  if (format == GS_FMT_COO) {
    const int64_t total = nnz * out_len;
    GS_LAUNCH("spmm_coo", s,
              spmm_coo_kernel<<<dim3((unsigned)ceil_div(total, kBlock)),
                                dim3(kBlock), 0, s>>>(
                  a, b, edge_map, nnz, kind, op, reduce, ufeat, efeat, out,
                  u_target, ufeat_len, efeat_len, out_len, u_off, e_off));
    if (reduce != kReduceSum && (arg_u || arg_e))
      GS_LAUNCH("spmm_coo_arg", s,
                spmm_coo_arg_kernel<<<dim3((unsigned)ceil_div(total, kBlock)),
                                      dim3(kBlock), 0, s>>>(
                    a, b, edge_map, nnz, op, ufeat, efeat, out, arg_u, arg_e,
                    u_target, ufeat_len, efeat_len, out_len, u_off, e_off));
    return GS_OK;
  }
  if (scalar) {
    const int64_t avg = nnz / (num_major > 0 ? num_major : 1);
#define GS_SPMM_SCALAR(G)                                                      \
  GS_LAUNCH("spmm_csc_scalar", s,                                              \
            spmm_csc_scalar_kernel<G><<<dim3((unsigned)ceil_div(num_major * G, kBlock)), \
                                        dim3(kBlock), 0, s>>>(                 \
                a, b, edge_map, num_major, kind, op, reduce, ufeat, efeat, out, \
                arg_u, arg_e))
    if (avg <= 8)
      GS_SPMM_SCALAR(4);
    else if (avg <= 64)
      GS_SPMM_SCALAR(16);
    else
      GS_SPMM_SCALAR(64);
#undef GS_SPMM_SCALAR
    return GS_OK;
  }
  GS_LAUNCH("spmm_csc", s,
            spmm_csc_kernel<<<dim3((unsigned)ceil_div(num_major * out_len, kBlock)),
                              dim3(kBlock), 0, s>>>(
                a, b, edge_map, num_major, kind, op, reduce, ufeat, efeat, out,
                arg_u, arg_e, ufeat_len, efeat_len, out_len, u_off, e_off));
  return GS_OK;
}

}  // namespace gs

extern "C" {

int gs_sddmm(int format, const int64_t* a, const int64_t* b, int64_t num_major,
             int64_t nnz, const int64_t* edge_map, int op, int dtype,
             const void* lhs, const void* rhs, void* out, int lhs_target,
             int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
             int64_t reduce_size, const int64_t* lhs_off, const int64_t* rhs_off,
             gs_stream_t stream) {
  using namespace gs;
  int rc = check_view(format, a, b, num_major, nnz, "sddmm");
  if (rc != GS_OK) return rc;
  GS_REQUIRE(op >= kOpAdd && op <= kOpDot, "sddmm: unknown operator %d", op);
  GS_REQUIRE(dtype == GS_F32 || dtype == GS_F64, "sddmm: unknown dtype %d", dtype);
  GS_REQUIRE(lhs_target >= 0 && lhs_target <= 2 && rhs_target >= 0 && rhs_target <= 2,
             "sddmm: targets must be 0 (u), 1 (e) or 2 (v)");
  GS_REQUIRE(out_len >= 0 && reduce_size >= 1, "sddmm: bad feature sizes");
  if (nnz == 0 || out_len == 0) return GS_OK;
  GS_REQUIRE(out && (lhs || op == kOpCopyRhs) && (rhs || op == kOpCopyLhs),
             "sddmm: null operand");
  hipStream_t s = as_stream(stream);
  const EdgeView g{format == GS_FMT_COMPRESSED, a, b, num_major, edge_map};
#define GS_SDDMM_LAUNCH(T, ITEMS)                                                         \
  GS_LAUNCH("sddmm", s,                                                                   \
            (sddmm_kernel<T, ITEMS>)<<<dim3((unsigned)ceil_div(nnz * out_len, kBlock * ITEMS)), \
                                     dim3(kBlock), 0, s>>>(                               \
                g, nnz, op, (const T*)lhs, (const T*)rhs, (T*)out, lhs_target, rhs_target, \
                lhs_len, rhs_len, out_len, reduce_size, lhs_off, rhs_off))
  if (g.compressed) {
    if (dtype == GS_F32) GS_SDDMM_LAUNCH(float, kEdgeItems);
    else GS_SDDMM_LAUNCH(double, kEdgeItems);
  } else {
    if (dtype == GS_F32) GS_SDDMM_LAUNCH(float, 1);
    else GS_SDDMM_LAUNCH(double, 1);
  }
#undef GS_SDDMM_LAUNCH
  return GS_OK;
}

int gs_fused_u_op_v(int format, const int64_t* a, const int64_t* b,
                    int64_t num_major, int64_t nnz, const int64_t* edge_map,
                    int op, int dtype,
                    const void* lhs1, const void* rhs1, void* out1,
                    const void* lhs2, const void* rhs2, void* out2,
                    int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                    int64_t reduce_size, const int64_t* lhs_off,
                    const int64_t* rhs_off, gs_stream_t stream) {
  using namespace gs;
  int rc = check_view(format, a, b, num_major, nnz, "fused_u_op_v");
  if (rc != GS_OK) return rc;
  GS_REQUIRE((op >= kOpAdd && op <= kOpDiv) || op == kOpDot,
             "fused_u_op_v: operator %d needs both operands", op);
  GS_REQUIRE(dtype == GS_F32 || dtype == GS_F64, "fused_u_op_v: unknown dtype %d", dtype);
  if (nnz == 0 || out_len == 0) return GS_OK;
  GS_REQUIRE(lhs1 && rhs1 && out1 && lhs2 && rhs2 && out2, "fused_u_op_v: null operand");
  hipStream_t s = as_stream(stream);
  const EdgeView g{format == GS_FMT_COMPRESSED, a, b, num_major, edge_map};
#define GS_UOPV_LAUNCH(T, ITEMS)                                                          \
  GS_LAUNCH("fused_u_op_v", s,                                                            \
            (fused_u_op_v_kernel<T, ITEMS>)<<<dim3((unsigned)ceil_div(nnz * out_len,      \
                                                                      kBlock * ITEMS)),   \
                                            dim3(kBlock), 0, s>>>(                        \
                g, nnz, op, (const T*)lhs1, (const T*)rhs1, (T*)out1, (const T*)lhs2,     \
                (const T*)rhs2, (T*)out2, lhs_len, rhs_len, out_len, reduce_size, lhs_off, \
                rhs_off))
  if (g.compressed) {
    if (dtype == GS_F32) GS_UOPV_LAUNCH(float, kEdgeItems);
    else GS_UOPV_LAUNCH(double, kEdgeItems);
  } else {
    if (dtype == GS_F32) GS_UOPV_LAUNCH(float, 1);
    else GS_UOPV_LAUNCH(double, 1);
  }
#undef GS_UOPV_LAUNCH
  return GS_OK;
}

size_t gs_spmm_workspace_bytes(int format, int64_t nnz, int64_t num_out) {
  const gs::RowRangePlan plan = gs::row_range_plan(format, nnz, num_out);
  if (plan.total > 0) return plan.total;
  return gs::private_bytes(format, nnz, num_out);
}

int gs_spmm(int format, const int64_t* a, const int64_t* b, int64_t num_major,
            int64_t nnz, const int64_t* edge_map, int op, int reduce,
            const float* ufeat, const float* efeat, float* out, int64_t* arg_u,
            int64_t* arg_e, int u_target, int64_t ufeat_len, int64_t efeat_len,
            int64_t out_len, const int64_t* u_off, const int64_t* e_off,
            int64_t num_out, void* workspace, size_t workspace_bytes,
            gs_stream_t stream) {
  using namespace gs;
  int rc = check_view(format, a, b, num_major, nnz, "spmm");
  if (rc != GS_OK) return rc;
  GS_REQUIRE((op >= kOpAdd && op <= kOpCopyRhs), "spmm: unknown operator %d", op);
  GS_REQUIRE(reduce >= kReduceSum && reduce <= kReduceMin, "spmm: unknown reducer %d", reduce);
  GS_REQUIRE(u_target == 0 || u_target == 2, "spmm: u_target must be 0 or 2");
  if (nnz == 0 || out_len == 0) return GS_OK;
  GS_REQUIRE(out && (ufeat || op == kOpCopyRhs) && (efeat || op == kOpCopyLhs),
             "spmm: null operand");
  return spmm_launch(format, a, b, num_major, nnz, edge_map, 0, op, reduce,
                     op == kOpCopyRhs ? nullptr : ufeat,
                     op == kOpCopyLhs ? nullptr : efeat, out, arg_u, arg_e,
                     u_target, ufeat_len, efeat_len, out_len, u_off, e_off,
                     num_out, workspace, workspace_bytes, as_stream(stream));
}

int gs_e_square_sum(int format, const int64_t* a, const int64_t* b,
                    int64_t num_major, int64_t nnz, const int64_t* edge_map,
                    const float* efeat, float* out, int u_target,
                    int64_t feat_len, int64_t num_out, void* workspace,
                    size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  int rc = check_view(format, a, b, num_major, nnz, "e_square_sum");
  if (rc != GS_OK) return rc;
  GS_REQUIRE(u_target == 0 || u_target == 2, "e_square_sum: u_target must be 0 or 2");
  if (nnz == 0 || feat_len == 0) return GS_OK;
  GS_REQUIRE(efeat && out, "e_square_sum: null operand");
  return spmm_launch(format, a, b, num_major, nnz, edge_map, 1, kOpCopyRhs,
                     kReduceSum, nullptr, efeat, out, nullptr, nullptr, u_target,
                     0, feat_len, feat_len, nullptr, nullptr, num_out, workspace,
                     workspace_bytes, as_stream(stream));
}

size_t gs_sliced_e_square_sum_workspace_bytes(int64_t slice_nnz, int64_t num_out) {
  if (slice_nnz < 0 || num_out < 0) return 0;
  return gs::row_range_plan(GS_FMT_COO, slice_nnz, num_out).total;
}

int gs_sliced_e_square_sum(const int64_t* indptr, const int64_t* indices,
                           const int32_t* indices32, const int64_t* cols,
                           int64_t num_cols_picked, const int64_t* sub_indptr,
                           int64_t slice_nnz, const int64_t* edge_map, const float* efeat,
                           float* out,
                           int64_t num_out, void* workspace, size_t workspace_bytes,
                           gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_cols_picked >= 0 && slice_nnz >= 0 && num_out >= 0,
             "sliced_e_square_sum: negative size");
  if (slice_nnz == 0) return GS_OK;
  GS_REQUIRE(indptr && indices && cols && sub_indptr && efeat && out,
             "sliced_e_square_sum: null pointer");
  hipStream_t s = as_stream(stream);
  const SliceView view{sub_indptr, cols, indptr, nullptr, num_cols_picked};
  const RowRangePlan plan = row_range_plan(GS_FMT_COO, slice_nnz, num_out);
  if (plan.total > 0 && workspace != nullptr && workspace_bytes >= plan.total)
    return row_range_sum(plan, indices, indices32, nullptr, edge_map, slice_nnz, num_out, 1,
                         kOpCopyRhs, nullptr, efeat, out, workspace, s, view);
  // short slices: combined per tile in LDS, one atomic per (tile, row present);
  // ids outside [0, num_out) cannot occur for a slice of a checked matrix
  GS_LAUNCH("spmm_coo_sum", s,
            spmm_coo_sum_kernel<<<dim3((unsigned)ceil_div(slice_nnz, (int64_t)kSumTile)),
                                  dim3(kBlock), 0, s>>>(indices, indices, edge_map, slice_nnz, 1,
                                                        kOpCopyRhs, nullptr, efeat, out, 2,
                                                        (int64_t)0, view));
  return GS_OK;
}

int gs_e_div_u_sum(int format, const int64_t* a, const int64_t* b,
                   int64_t num_major, int64_t nnz, const int64_t* edge_map,
                   const float* ufeat, const float* efeat, float* out,
                   int u_target, int64_t feat_len, int64_t num_out,
                   void* workspace, size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  int rc = check_view(format, a, b, num_major, nnz, "e_div_u_sum");
  if (rc != GS_OK) return rc;
  GS_REQUIRE(u_target == 0 || u_target == 2, "e_div_u_sum: u_target must be 0 or 2");
  if (nnz == 0 || feat_len == 0) return GS_OK;
  GS_REQUIRE(ufeat && efeat && out, "e_div_u_sum: null operand");
  return spmm_launch(format, a, b, num_major, nnz, edge_map, 2, kOpDiv,
                     kReduceSum, ufeat, efeat, out, nullptr, nullptr, u_target,
                     feat_len, feat_len, feat_len, nullptr, nullptr, num_out,
                     workspace, workspace_bytes, as_stream(stream));
}

}  // extern "C"
