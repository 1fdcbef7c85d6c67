// gs_oracle.cpp -- CPU restatement of gSampler's sampling hot path.
//
// TEST INFRASTRUCTURE ONLY.  This file is the correctness oracle and the timed
// host baseline.  Nothing in the shipped package may link, load or call it:
// only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.
//
// Every function restates what the cited reference kernel computes (paths are
// relative to the gSampler source tree), written for clarity, parallel over
// columns / batches / walks with OpenMP.  Exported with a `_cpu` suffix and
// the same argument meaning as include/gsampler_hip.h, minus stream and
// workspace.
//
// Random numbers.  The reference draws from curand streams whose layout
// depends on the CUDA launch geometry (src/cuda/sampling.cu:25-26,56), so its
// exact picks cannot be restated on a CPU.  The convention here (shared with
// the HIP kernels, implemented independently in both) makes every pick a pure
// function of (seed, call_id, position, draw):
//   key     = seed + call_id * 0x9E3779B97F4A7C15  (mod 2^64), split lo/hi
//   counter = (lo32(draw), hi32(draw), lo32(pos), hi32(pos))
//   (w0,w1,w2,w3) = Philox4x32-10(counter, key)
//   r64 = w1:w0,  bounded(n) = floor(r64 * n / 2^64)
// Pinned by the Random123 known-answer vectors (tests/test_oracle_philox.py).
//
// Parity status of each function is listed in oracle/README.md.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <unordered_map>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#define GS_ALGO_AUTO 0
#define GS_ALGO_RESERVOIR 1
#define GS_ALGO_FLOYD 2

namespace {

// ---------------------------------------------------------------- Philox
struct U4 {
  uint32_t v[4];
};

inline U4 philox4x32_10(U4 ctr, uint32_t k0, uint32_t k1) {
  const uint64_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = M0 * ctr.v[0];
    uint64_t p1 = M1 * ctr.v[2];
    U4 n;
    n.v[0] = (uint32_t)(p1 >> 32) ^ ctr.v[1] ^ k0;
    n.v[1] = (uint32_t)p1;
    n.v[2] = (uint32_t)(p0 >> 32) ^ ctr.v[3] ^ k1;
    n.v[3] = (uint32_t)p0;
    ctr = n;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return ctr;
}

struct Stream {
  uint32_t k0, k1;
  Stream(uint64_t seed, uint64_t call_id) {
    uint64_t k = seed + call_id * 0x9E3779B97F4A7C15ull;
    k0 = (uint32_t)k;
    k1 = (uint32_t)(k >> 32);
  }
  U4 words(uint64_t pos, uint64_t draw) const {
    U4 c;
    c.v[0] = (uint32_t)draw;
    c.v[1] = (uint32_t)(draw >> 32);
    c.v[2] = (uint32_t)pos;
    c.v[3] = (uint32_t)(pos >> 32);
    return philox4x32_10(c, k0, k1);
  }
  uint64_t r64(uint64_t pos, uint64_t draw) const {
    U4 w = words(pos, draw);
    return ((uint64_t)w.v[1] << 32) | w.v[0];
  }
  // integer in [0, n)
  uint64_t bounded(uint64_t pos, uint64_t draw, uint64_t n) const {
    return (uint64_t)(((unsigned __int128)r64(pos, draw) * n) >> 64);
  }
};

inline int64_t col_degree(const int64_t* indptr, int64_t num_cols, int64_t c) {
  if (c < 0 || c >= num_cols) return 0;
  return indptr[c + 1] - indptr[c];
}

}  // namespace

extern "C" {

// Known-answer hook for the Philox block function.
void gs_philox4x32_10_cpu(const uint32_t* ctr, const uint32_t* key,
                          uint32_t* out) {
  U4 c = {{ctr[0], ctr[1], ctr[2], ctr[3]}};
  U4 r = philox4x32_10(c, key[0], key[1]);
  for (int i = 0; i < 4; ++i) out[i] = r.v[i];
}

// The four words drawn for (seed, call_id, pos, draw).
void gs_stream_words_cpu(uint64_t seed, uint64_t call_id, uint64_t pos,
                         uint64_t draw, uint32_t* out) {
  U4 r = Stream(seed, call_id).words(pos, draw);
  for (int i = 0; i < 4; ++i) out[i] = r.v[i];
}

int gs_num_threads_cpu(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

// -------------------------------------------------------------------------
// Exclusive scan (cub_exclusiveSum, src/cuda/utils.h:18-28).
void gs_exclusive_scan_i64_cpu(const int64_t* in, int64_t* out, int64_t n) {
  int64_t acc = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t v = in[i];
    out[i] = acc;
    acc += v;
  }
}

// -------------------------------------------------------------------------
// Per-column counts + prefix.  src/cuda/slicing.cu:133-141 (slice),
// src/cuda/sampling.cu:112-124 and src/cuda/fusion/slice_sampling.cu:111-124
// (sample): replace -> deg == 0 ? 0 : K ; else min(deg, K).
void gs_csc_col_count_cpu(const int64_t* indptr, int64_t num_cols,
                          const int64_t* column_ids, int64_t num_items,
                          int64_t fanout, int replace, int64_t* sub_indptr) {
  int64_t acc = 0;
  for (int64_t i = 0; i < num_items; ++i) {
    int64_t c = column_ids ? column_ids[i] : i;
    int64_t deg = col_degree(indptr, num_cols, c);
    int64_t cnt;
    if (fanout < 0)
      cnt = deg;
    else if (replace)
      cnt = deg == 0 ? 0 : fanout;
    else
      cnt = std::min(deg, fanout);
    sub_indptr[i] = acc;
    acc += cnt;
  }
  sub_indptr[num_items] = acc;
}

// -------------------------------------------------------------------------
// Column slice, src/cuda/slicing.cu:101-119 (_GetSubIndicesKernel) and the
// batched form src/cuda/batch/slicing.cu:12-38 (row id + batch * stride).
void gs_csc_col_slice_fill_cpu(const int64_t* indptr, int64_t num_cols,
                               const int64_t* indices,
                               const int64_t* column_ids, int64_t num_items,
                               const int64_t* sub_indptr, int64_t /*nnz*/,
                               const int64_t* batch_ptr, int64_t num_batches,
                               int64_t encode_stride, int64_t* out_coo_col,
                               int64_t* out_indices, int64_t* out_select) {
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < num_items; ++i) {
    int64_t c = column_ids ? column_ids[i] : i;
    int64_t deg = col_degree(indptr, num_cols, c);
    if (deg == 0) continue;
    int64_t in_start = indptr[c];
    int64_t out_start = sub_indptr[i];
    int64_t add = 0;
    if (batch_ptr && encode_stride > 0) {
      int64_t b = std::upper_bound(batch_ptr, batch_ptr + num_batches + 1, i) -
                  batch_ptr - 1;
      add = b * encode_stride;
    }
    for (int64_t k = 0; k < deg; ++k) {
      out_indices[out_start + k] = indices[in_start + k] + add;
      out_select[out_start + k] = in_start + k;
      if (out_coo_col) out_coo_col[out_start + k] = i;
    }
  }
}

// -------------------------------------------------------------------------
// Uniform per-column sampling, src/cuda/sampling.cu:18-101 and the fused form
// src/cuda/fusion/slice_sampling.cu:14-96.
//  * replace: slot j takes position r(j) mod deg            (:34-45)
//  * deg <= K: copy the column in order                      (:64-73)
//  * reservoir: slot[j] = j; for idx in [K, deg):
//      num = r(idx) mod (idx+1); if num < K: slot[num] = max(slot[num], idx)
//                                                            (:75-88)
//    The reference's `curand() % n` is replaced by the (less biased)
//    multiply-shift bounded(); the result depends only on idx -> r(idx).
//  * Floyd (not in the reference; same distribution over K-subsets, O(K)
//    draws instead of O(deg)): for i in [0,K): j = deg-K+i,
//      t = r(i) bounded to [0, j]; pick t unless already picked, then pick j.
void gs_csc_col_sample_uniform_fill_cpu(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const int64_t* column_ids, int64_t num_items, int64_t fanout, int replace,
    int algo, uint64_t seed, uint64_t call_id, const int64_t* sub_indptr,
    int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select) {
  Stream rng(seed, call_id);
  if (algo == GS_ALGO_AUTO)
    algo = fanout <= 64 ? GS_ALGO_FLOYD : GS_ALGO_RESERVOIR;
#pragma omp parallel
  {
    std::vector<int64_t> slot((size_t)std::max<int64_t>(fanout, 1));
#pragma omp for schedule(dynamic, 256)
    for (int64_t i = 0; i < num_items; ++i) {
      int64_t c = column_ids ? column_ids[i] : i;
      int64_t deg = col_degree(indptr, num_cols, c);
      if (deg == 0) continue;
      int64_t in_start = indptr[c];
      int64_t out_start = sub_indptr[i];
      int64_t cnt = sub_indptr[i + 1] - out_start;
      if (replace) {
        for (int64_t j = 0; j < cnt; ++j)
          slot[j] = (int64_t)rng.bounded((uint64_t)i, (uint64_t)j, (uint64_t)deg);
      } else if (deg <= fanout) {
        for (int64_t j = 0; j < cnt; ++j) slot[j] = j;
      } else if (algo == GS_ALGO_RESERVOIR) {
        for (int64_t j = 0; j < fanout; ++j) slot[j] = j;
        for (int64_t idx = fanout; idx < deg; ++idx) {
          int64_t num = (int64_t)rng.bounded((uint64_t)i, (uint64_t)idx,
                                             (uint64_t)idx + 1);
          if (num < fanout) slot[num] = std::max(slot[num], idx);
        }
      } else {  // Floyd
        for (int64_t k = 0; k < fanout; ++k) {
          int64_t j = deg - fanout + k;
          int64_t t = (int64_t)rng.bounded((uint64_t)i, (uint64_t)k,
                                           (uint64_t)j + 1);
          bool seen = false;
          for (int64_t m = 0; m < k; ++m)
            if (slot[m] == t) {
              seen = true;
              break;
            }
          slot[k] = seen ? j : t;
        }
      }
      for (int64_t j = 0; j < cnt; ++j) {
        int64_t p = in_start + slot[j];
        out_indices[out_start + j] = indices ? indices[p] : p;
        out_select[out_start + j] = p;
        if (out_coo_col) out_coo_col[out_start + j] = i;
      }
    }
  }
}

// -------------------------------------------------------------------------
// Unique (first-occurrence order) + relabel.
//  single batch : Unique / Relabel, src/cuda/unique_reindex.cu:81-172 -- the
//    table keeps the minimum index per key (:25 AtomicMin), an element is kept
//    iff it holds that minimum (:113), its rank is the prefix count (:138-139).
//  super-batch  : src/cuda/batch/batch_relabel.cu:92-377 -- one table per
//    batch, keys of batch b are seeds_b ++ rows_b (:138-161), ranks are
//    batch-local, unique_ptr[b] = uniques before batch b (:437-438).
// out_col[e] = rank of seeds[edge_col[e]] (the reference relabels
// coo_col = col_seeds[coo.col], src/batch_graph.cc:230, src/graph.cc:582).
static void batch_bounds(const int64_t* ptr, int64_t total, int64_t nb,
                         int64_t b, int64_t* lo, int64_t* hi) {
  if (ptr) {
    *lo = ptr[b];
    *hi = ptr[b + 1];
  } else {
    *lo = 0;
    *hi = total;
    (void)nb;
  }
}

// Pass 1 (count): unique_ptr.  Pass 2 (fill): outputs.  Both recompute the
// per-batch map; the oracle favours obviousness over speed.
static void unique_batch(const int64_t* seeds, int64_t s_lo, int64_t s_hi,
                         const int64_t* rows, int64_t r_lo, int64_t r_hi,
                         std::unordered_map<int64_t, int64_t>* rank,
                         std::vector<int64_t>* uniq) {
  rank->clear();
  uniq->clear();
  rank->reserve((size_t)((s_hi - s_lo) + (r_hi - r_lo)));
  for (int64_t i = s_lo; i < s_hi; ++i)
    if (rank->emplace(seeds[i], (int64_t)uniq->size()).second)
      uniq->push_back(seeds[i]);
  for (int64_t i = r_lo; i < r_hi; ++i)
    if (rank->emplace(rows[i], (int64_t)uniq->size()).second)
      uniq->push_back(rows[i]);
}

void gs_unique_count_cpu(const int64_t* seeds, const int64_t* seeds_ptr,
                         int64_t num_seeds, const int64_t* rows,
                         const int64_t* rows_ptr, int64_t num_rows_keys,
                         int64_t num_batches, int64_t* unique_ptr) {
  std::vector<int64_t> counts((size_t)num_batches);
#pragma omp parallel
  {
    std::unordered_map<int64_t, int64_t> rank;
    std::vector<int64_t> uniq;
#pragma omp for schedule(dynamic, 1)
    for (int64_t b = 0; b < num_batches; ++b) {
      int64_t s_lo, s_hi, r_lo, r_hi;
      batch_bounds(seeds_ptr, num_seeds, num_batches, b, &s_lo, &s_hi);
      batch_bounds(rows_ptr, num_rows_keys, num_batches, b, &r_lo, &r_hi);
      unique_batch(seeds, s_lo, s_hi, rows, r_lo, r_hi, &rank, &uniq);
      counts[(size_t)b] = (int64_t)uniq.size();
    }
  }
  int64_t acc = 0;
  for (int64_t b = 0; b < num_batches; ++b) {
    unique_ptr[b] = acc;
    acc += counts[(size_t)b];
  }
  unique_ptr[num_batches] = acc;
}

void gs_unique_fill_cpu(const int64_t* seeds, const int64_t* seeds_ptr,
                        int64_t num_seeds, const int64_t* rows,
                        const int64_t* rows_ptr, int64_t num_rows_keys,
                        int64_t num_batches, const int64_t* unique_ptr,
                        int64_t* out_unique) {
#pragma omp parallel
  {
    std::unordered_map<int64_t, int64_t> rank;
    std::vector<int64_t> uniq;
#pragma omp for schedule(dynamic, 1)
    for (int64_t b = 0; b < num_batches; ++b) {
      int64_t s_lo, s_hi, r_lo, r_hi;
      batch_bounds(seeds_ptr, num_seeds, num_batches, b, &s_lo, &s_hi);
      batch_bounds(rows_ptr, num_rows_keys, num_batches, b, &r_lo, &r_hi);
      unique_batch(seeds, s_lo, s_hi, rows, r_lo, r_hi, &rank, &uniq);
      std::copy(uniq.begin(), uniq.end(), out_unique + unique_ptr[b]);
    }
  }
}

void gs_unique_relabel_cpu(const int64_t* seeds, const int64_t* seeds_ptr,
                           int64_t num_seeds, const int64_t* rows,
                           const int64_t* rows_ptr, int64_t num_rows_keys,
                           int64_t num_batches, const int64_t* edge_col,
                           int64_t* out_row, int64_t* out_col) {
#pragma omp parallel
  {
    std::unordered_map<int64_t, int64_t> rank;
    std::vector<int64_t> uniq;
#pragma omp for schedule(dynamic, 1)
    for (int64_t b = 0; b < num_batches; ++b) {
      int64_t s_lo, s_hi, r_lo, r_hi;
      batch_bounds(seeds_ptr, num_seeds, num_batches, b, &s_lo, &s_hi);
      batch_bounds(rows_ptr, num_rows_keys, num_batches, b, &r_lo, &r_hi);
      unique_batch(seeds, s_lo, s_hi, rows, r_lo, r_hi, &rank, &uniq);
      for (int64_t e = r_lo; e < r_hi; ++e) {
        if (out_row) out_row[e] = rank[rows[e]];
        if (out_col) out_col[e] = rank[seeds[edge_col[e]]];
      }
    }
  }
}

// -------------------------------------------------------------------------
// Format conversion, src/cuda/format_transform.cu.
//  CSC -> COO (:24-46): col[e] = UpperBound(indptr, e) - 1.
//  COO -> CSC (:109-142), after a sort by column:
//    indptr[c + 1] = UpperBound(sorted_cols, c)  <=>  indptr[c] = #entries < c.
void gs_csc2coo_cpu(const int64_t* indptr, int64_t num_cols, int64_t nnz,
                    int64_t* out_col) {
  for (int64_t c = 0; c < num_cols; ++c)
    for (int64_t e = indptr[c]; e < indptr[c + 1] && e < nnz; ++e) out_col[e] = c;
}

void gs_sorted_to_indptr_cpu(const int64_t* sorted_ids, int64_t nnz,
                             int64_t num_cols, int64_t* out_indptr) {
  for (int64_t c = 0; c <= num_cols; ++c)
    out_indptr[c] = std::lower_bound(sorted_ids, sorted_ids + nnz, c) - sorted_ids;
}

// -------------------------------------------------------------------------
// Super-batch bookkeeping.
//  decode: mask = id / size, orig = id - mask * size
//    (src/cuda/batch/encoding_decoding.cu:99-113).
//  split indptr: out[offset[b] + b + j] = indptr[offset[b] + j] - indptr[offset[b]]
//    for j in [0, offset[b+1] - offset[b]]  (src/cuda/batch/batch_split.cu:53-72).
void gs_decode_batch_ids_cpu(const int64_t* encoded, int64_t n, int64_t stride,
                             int64_t* out_orig, int64_t* out_batch) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t b = encoded[i] / stride;
    if (out_batch) out_batch[i] = b;
    if (out_orig) out_orig[i] = encoded[i] - b * stride;
  }
}

void gs_split_indptr_cpu(const int64_t* indptr, const int64_t* offset,
                         int64_t num_batches, int64_t /*out_len*/, int64_t* out) {
  for (int64_t b = 0; b < num_batches; ++b) {
    int64_t lo = offset[b], hi = offset[b + 1];
    for (int64_t j = 0; j <= hi - lo; ++j)
      out[lo - offset[0] + b + j] = indptr[lo + j] - indptr[lo];
  }
}

// -------------------------------------------------------------------------
// Edge-wise compute operators (DGL-derived in the reference).
//  endpoints: COO src = row[e], dst = col[e] (src/cuda/sddmm.cu:37-38);
//  compressed src = indices[e], dst = UpperBound(indptr, e) - 1 (:134-135);
//  eid = edge_map ? edge_map[e] : e (:39,136).
//  SDDMM  out[eid*len + f] = op(lhs[sel_l*lhs_len + off_l[f]*red], rhs[...])  (:40-57)
//  SpMM   COO: out[dst] (+)= op(u[src], e[eid]) with src/dst swapped when
//         u_target != 0 (src/cuda/spmm.cu:39-56); compressed: per segment
//         accumulate from 0, then out += acc (:122-141).  Max / Min start from
//         0 as well because the accumulator / output start at 0.
//  e^2 sum (src/cuda/fusion/fused_csc_e_square_sum.cu:49-54), e/u sum
//  (fused_csc_e_div_u_sum.cu:43: BinaryOp::Call(eoff, uoff)).
}  // extern "C"

namespace {
template <typename T>
T apply_op(int op, const T* l, const T* r, int64_t red) {
  switch (op) {
    case 0: return l[0] + r[0];
    case 1: return l[0] - r[0];
    case 2: return l[0] * r[0];
    case 3: return l[0] / r[0];
    case 4: return l[0];
    case 5: return r[0];
    default: {
      T acc = 0;
      for (int64_t k = 0; k < red; ++k) acc += l[k] * r[k];
      return acc;
    }
  }
}

struct View {
  int format;
  const int64_t *a, *b;
  int64_t num_major;
  const int64_t* edge_map;
  void endpoints(int64_t e, int64_t* src, int64_t* dst, int64_t* eid) const {
    if (format == 2) {
      *src = b[e];
      *dst = (std::upper_bound(a, a + num_major + 1, e) - a) - 1;
    } else {
      *src = a[e];
      *dst = b[e];
    }
    *eid = edge_map ? edge_map[e] : e;
  }
};

template <typename T>
void sddmm_impl(const View& g, int64_t nnz, int op, const T* lhs, const T* rhs,
                T* out, int lt, int rt, int64_t lhs_len, int64_t rhs_len,
                int64_t out_len, int64_t red, const int64_t* lo,
                const int64_t* ro) {
  for (int64_t e = 0; e < nnz; ++e) {
    int64_t src, dst, eid;
    g.endpoints(e, &src, &dst, &eid);
    int64_t ls = lt == 0 ? src : (lt == 1 ? eid : dst);
    int64_t rs = rt == 0 ? src : (rt == 1 ? eid : dst);
    for (int64_t f = 0; f < out_len; ++f) {
      const T* l = op == 5 ? nullptr : lhs + ls * lhs_len + (lo ? lo[f] : f) * red;
      const T* r = op == 4 ? nullptr : rhs + rs * rhs_len + (ro ? ro[f] : f) * red;
      out[eid * out_len + f] = apply_op<T>(op, l, r, red);
    }
  }
}

float edge_value(int kind, int op, const float* u, const float* e) {
  if (kind == 1) return e[0] * e[0];
  if (kind == 2) return e[0] / u[0];
  return apply_op<float>(op, u, e, 1);
}

void spmm_impl(const View& g, int64_t nnz, int kind, int op, int reduce,
               const float* ufeat, const float* efeat, float* out,
               int64_t* arg_u, int64_t* arg_e, int u_target, int64_t ulen,
               int64_t elen, int64_t out_len, const int64_t* uo,
               const int64_t* eo) {
  auto better = [&](float v, float cur) {
    return reduce == 1 ? v > cur : v < cur;
  };
  if (g.format == 2) {
    for (int64_t c = 0; c < g.num_major; ++c)
      for (int64_t f = 0; f < out_len; ++f) {
        float acc = 0.f;
        double sum = 0.0;
        int64_t bu = 0, be = 0;
        for (int64_t i = g.a[c]; i < g.a[c + 1]; ++i) {
          int64_t eid = g.edge_map ? g.edge_map[i] : i, cid = g.b[i];
          float v = edge_value(kind, op,
                               ufeat ? ufeat + cid * ulen + (uo ? uo[f] : f) : nullptr,
                               efeat ? efeat + eid * elen + (eo ? eo[f] : f) : nullptr);
          if (reduce == 0)
            sum += (double)v;
          else if (better(v, acc)) {
            acc = v;
            bu = cid;
            be = eid;
          }
        }
        if (reduce == 0) acc = (float)sum;
        out[c * out_len + f] += acc;
        if (reduce != 0) {
          if (arg_u) arg_u[c * out_len + f] = bu;
          if (arg_e) arg_e[c * out_len + f] = be;
        }
      }
    return;
  }
  // Sums are taken in double and rounded once (per-edge values stay float32,
  // as on the device): the reference adds with float atomics in whatever order
  // the hardware takes them, so no float32 sum is "the" result, and a yardstick
  // that carries a rounding error of its own per term would only blur the
  // comparison for long rows.
  std::vector<double> sums;
  if (reduce == 0) {
    int64_t n_out = 0;
    for (int64_t e = 0; e < nnz; ++e)
      n_out = std::max(n_out, (u_target == 0 ? g.b[e] : g.a[e]) + 1);
    sums.assign((size_t)(n_out * out_len), 0.0);
  }
  for (int64_t e = 0; e < nnz; ++e) {
    int64_t src = u_target == 0 ? g.a[e] : g.b[e];
    int64_t dst = u_target == 0 ? g.b[e] : g.a[e];
    int64_t eid = g.edge_map ? g.edge_map[e] : e;
    for (int64_t f = 0; f < out_len; ++f) {
      float v = edge_value(kind, op,
                           ufeat ? ufeat + src * ulen + (uo ? uo[f] : f) : nullptr,
                           efeat ? efeat + eid * elen + (eo ? eo[f] : f) : nullptr);
      float& o = out[dst * out_len + f];
      if (reduce == 0)
        sums[(size_t)(dst * out_len + f)] += (double)v;
      else if (better(v, o)) {
        o = v;
        if (arg_u) arg_u[dst * out_len + f] = src;
        if (arg_e) arg_e[dst * out_len + f] = eid;
      }
    }
  }
  for (size_t i = 0; i < sums.size(); ++i) out[i] += (float)sums[i];
}
}  // namespace

extern "C" {

void gs_sddmm_cpu(int format, const int64_t* a, const int64_t* b,
                  int64_t num_major, int64_t nnz, const int64_t* edge_map,
                  int op, int dtype, const void* lhs, const void* rhs, void* out,
                  int lhs_target, int rhs_target, int64_t lhs_len,
                  int64_t rhs_len, int64_t out_len, int64_t reduce_size,
                  const int64_t* lhs_off, const int64_t* rhs_off) {
  View g{format, a, b, num_major, edge_map};
  if (dtype == 0)
    sddmm_impl<float>(g, nnz, op, (const float*)lhs, (const float*)rhs,
                      (float*)out, lhs_target, rhs_target, lhs_len, rhs_len,
                      out_len, reduce_size, lhs_off, rhs_off);
  else
    sddmm_impl<double>(g, nnz, op, (const double*)lhs, (const double*)rhs,
                       (double*)out, lhs_target, rhs_target, lhs_len, rhs_len,
                       out_len, reduce_size, lhs_off, rhs_off);
}

void gs_fused_u_op_v_cpu(int format, const int64_t* a, const int64_t* b,
                         int64_t num_major, int64_t nnz, int op, int dtype,
                         const void* lhs1, const void* rhs1, void* out1,
                         const void* lhs2, const void* rhs2, void* out2,
                         int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                         int64_t reduce_size, const int64_t* lhs_off,
                         const int64_t* rhs_off) {
  gs_sddmm_cpu(format, a, b, num_major, nnz, nullptr, op, dtype, lhs1, rhs1, out1,
               0, 2, lhs_len, rhs_len, out_len, reduce_size, lhs_off, rhs_off);
  gs_sddmm_cpu(format, a, b, num_major, nnz, nullptr, op, dtype, lhs2, rhs2, out2,
               0, 2, lhs_len, rhs_len, out_len, reduce_size, lhs_off, rhs_off);
}

void gs_spmm_cpu(int format, const int64_t* a, const int64_t* b,
                 int64_t num_major, int64_t nnz, const int64_t* edge_map, int op,
                 int reduce, const float* ufeat, const float* efeat, float* out,
                 int64_t* arg_u, int64_t* arg_e, int u_target, int64_t ufeat_len,
                 int64_t efeat_len, int64_t out_len, const int64_t* u_off,
                 const int64_t* e_off) {
  View g{format, a, b, num_major, edge_map};
  spmm_impl(g, nnz, 0, op, reduce, op == 5 ? nullptr : ufeat,
            op == 4 ? nullptr : efeat, out, arg_u, arg_e, u_target, ufeat_len,
            efeat_len, out_len, u_off, e_off);
}

void gs_e_square_sum_cpu(int format, const int64_t* a, const int64_t* b,
                         int64_t num_major, int64_t nnz, const int64_t* edge_map,
                         const float* efeat, float* out, int u_target,
                         int64_t feat_len) {
  View g{format, a, b, num_major, edge_map};
  spmm_impl(g, nnz, 1, 5, 0, nullptr, efeat, out, nullptr, nullptr, u_target, 0,
            feat_len, feat_len, nullptr, nullptr);
}

void gs_e_div_u_sum_cpu(int format, const int64_t* a, const int64_t* b,
                        int64_t num_major, int64_t nnz, const int64_t* edge_map,
                        const float* ufeat, const float* efeat, float* out,
                        int u_target, int64_t feat_len) {
  View g{format, a, b, num_major, edge_map};
  spmm_impl(g, nnz, 2, 3, 0, ufeat, efeat, out, nullptr, nullptr, u_target,
            feat_len, feat_len, feat_len, nullptr, nullptr);
}

}  // extern "C"

// -------------------------------------------------------------------------
// Slicing across the compressed axis and COO slicing.
//  src/cuda/slicing.cu:185-229 (_OnIndicesSlicinigQueryKernel): every edge whose
//  row id is in the picked set is kept, its row becomes the value stored for it
//  in the set's hash map, edge order is preserved, every column is kept
//  (:283-293 compaction by nonzero(mask)).  src/cuda/slicing.cu:312-371: the
//  coordinate form keeps (relabelled id, other id, position).
//  The reference stores the position of whichever duplicate wrote last
//  (:56 `vptr[pos] = value`, racy); this restatement keeps the smallest.
extern "C" void gs_minor_slice_cpu(const int64_t* ids, int64_t nnz,
                                   const int64_t* picked, int64_t num_picked,
                                   const int64_t* indptr, int64_t num_major,
                                   const int64_t* edge_major, int64_t* out_indptr,
                                   int64_t* out_total, int64_t* out_major,
                                   int64_t* out_minor, int64_t* out_select) {
  std::unordered_map<int64_t, int64_t> where;
  for (int64_t i = 0; i < num_picked; ++i) where.emplace(picked[i], i);
  int64_t kept = 0, c = 0;
  if (out_indptr) out_indptr[0] = 0;
  for (int64_t e = 0; e < nnz; ++e) {
    if (indptr)
      while (c < num_major && indptr[c + 1] <= e) {
        ++c;
        if (out_indptr) out_indptr[c] = kept;
      }
    auto it = where.find(ids[e]);
    if (it == where.end()) continue;
    if (out_minor) {
      out_minor[kept] = it->second;
      out_select[kept] = e;
      if (out_major) out_major[kept] = edge_major ? edge_major[e] : c;
    }
    ++kept;
  }
  if (out_indptr)
    for (int64_t k = c + 1; k <= num_major; ++k) out_indptr[k] = kept;
  if (out_total) *out_total = kept;
}

// -------------------------------------------------------------------------
// Weighted sampling.
//
// Without replacement the reference uses Efraimidis-Spirakis keys u^(1/w) and
// keeps the K largest (src/cuda/sampling_probs.cu:55-75 per column,
// src/cuda/list_sampling_probs.cu:51-80 for lists: sort all keys descending,
// first K in sorted order).  Ranking by u^(1/w) descending is ranking by
// (-log2 u) / w ascending; that form is used here because it can be computed
// with correctly rounded double operations only (+, -, *, fma; quotients by
// det_div below), hence identically on the CPU and the GPU:
//   v = (r64 >> 12) + 1 in [1, 2^52],  u = v / 2^52,
//   -log2 u = (52 - e) - log2(m),  v = m * 2^e,  m in (sqrt(1/2), sqrt(2)],
//   log2(m) = s * P(s^2),  s = (m - 1) / (m + 1),  P = 11-term atanh series.
// Items with w <= 0 (or NaN) get key +inf: they are taken last, in index order
// (the list form of the reference gives them key -1, :63-66).  Ties break
// towards the smaller index.  Output order is ascending key, which is the
// reference's descending u^(1/w) order.
//
// With replacement the reference inverts a per-column fp32 CDF
// (src/cuda/sampling_probs.cu:150-174, src/cuda/list_sampling_probs.cu:28-48).
// A floating-point prefix sum depends on the summation order, so weights are
// first quantised to integers q = floor(w * scale), scale = det_div(2^31, wmax)
// (exact max, one rounded product per item); integer prefix sums are
// order-independent.  pick = min(upper_bound(cdf, t), n - 1), t = bounded(total)
// (t = 0 when every weight is <= 0, which selects the last item as the
// reference's all-zero CDF does).
namespace {

const double kLogC[11] = {0x1.71547652b82fep+1, 0x1.ec709dc3a03fep-1,
                          0x1.2776c50ef9bfep-1, 0x1.a61762a7adedap-2,
                          0x1.484b13d7c02a9p-2, 0x1.0c9a84994022dp-2,
                          0x1.c68f568d31761p-3, 0x1.89f3b1694cffep-3,
                          0x1.5b9ac9b743f0dp-3, 0x1.3703c1f4d0ffep-3,
                          0x1.1964ec6fc9491p-3};

// x / y (y > 0, finite, normal) from fused multiply-adds only, so that the
// quotient is the same on every IEEE machine: reciprocal estimate by integer
// subtraction on the bit pattern, six Newton steps r += r * (1 - y r), then
// q = x r corrected once by the residual x - y q.
double det_div(double x, double y) {
  int64_t yb;
  std::memcpy(&yb, &y, 8);
  int64_t rb = 0x7FDE623822FC16E6ll - yb;
  double r;
  std::memcpy(&r, &rb, 8);
  for (int i = 0; i < 6; ++i) r = std::fma(r, std::fma(-y, r, 1.0), r);
  double q = x * r;
  return std::fma(std::fma(-y, q, x), r, q);
}

double neg_log2_unit(uint64_t r64) {
  uint64_t v = (r64 >> 12) + 1;
  int e = 63 - __builtin_clzll(v);
  double m = std::ldexp((double)v, -e);
  if (m > 0x1.6a09e667f3bcdp+0) {
    m *= 0.5;
    e += 1;
  }
  double s = det_div(m - 1.0, m + 1.0);
  double s2 = s * s;
  double p = kLogC[10];
  for (int k = 9; k >= 0; --k) p = std::fma(p, s2, kLogC[k]);
  return std::fma(-s, p, (double)(52 - e));  // (52 - e) - log2(m), one rounding
}

double weighted_key(const Stream& rng, uint64_t pos, uint64_t draw, float w) {
  if (!(w > 0.0f)) return std::numeric_limits<double>::infinity();
  return det_div(neg_log2_unit(rng.r64(pos, draw)), (double)w);
}

struct KeyIdx {
  double key;
  int64_t idx;
  bool operator<(const KeyIdx& o) const {
    return key < o.key || (key == o.key && idx < o.idx);
  }
};

// Integer CDF of n weights into cdf[n]; returns the total.
uint64_t integer_cdf(const float* w, int64_t n, uint64_t* cdf) {
  float wmax = 0.0f;
  for (int64_t i = 0; i < n; ++i)
    if (w[i] > wmax) wmax = w[i];
  uint64_t acc = 0;
  if (wmax > 0.0f) {
    double scale = det_div(2147483648.0, (double)wmax);
    for (int64_t i = 0; i < n; ++i) {
      uint64_t q = w[i] > 0.0f ? (uint64_t)((double)w[i] * scale) : 0;
      acc += q;
      cdf[i] = acc;
    }
  } else {
    for (int64_t i = 0; i < n; ++i) cdf[i] = 0;
  }
  return acc;
}

int64_t cdf_pick(const uint64_t* cdf, int64_t n, uint64_t total, const Stream& rng,
                 uint64_t pos, uint64_t draw) {
  uint64_t t = total > 0 ? rng.bounded(pos, draw, total) : 0;
  int64_t item = std::upper_bound(cdf, cdf + n, t) - cdf;
  return std::min(item, n - 1);
}

}  // namespace

extern "C" {

// Known-answer hooks for the key arithmetic.
double gs_neg_log2_unit_cpu(uint64_t r64) { return neg_log2_unit(r64); }
double gs_weighted_key_cpu(uint64_t seed, uint64_t call_id, uint64_t pos,
                           uint64_t draw, float w) {
  return weighted_key(Stream(seed, call_id), pos, draw, w);
}

// Weighted per-column sampling, src/cuda/sampling_probs.cu:25-188.  probs are
// aligned with `indices`.  deg <= fanout (no replace): whole column in order,
// zero-weight edges included (:94-106).
void gs_csc_col_sample_weighted_fill_cpu(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const float* probs, const int64_t* column_ids, int64_t num_items,
    int64_t fanout, int replace, uint64_t seed, uint64_t call_id,
    const int64_t* sub_indptr, int64_t* out_coo_col, int64_t* out_indices,
    int64_t* out_select) {
  Stream rng(seed, call_id);
#pragma omp parallel
  {
    std::vector<KeyIdx> keys;
    std::vector<uint64_t> cdf;
#pragma omp for schedule(dynamic, 64)
    for (int64_t i = 0; i < num_items; ++i) {
      int64_t c = column_ids ? column_ids[i] : i;
      int64_t deg = col_degree(indptr, num_cols, c);
      if (deg == 0) continue;
      int64_t in_start = indptr[c], out_start = sub_indptr[i];
      int64_t cnt = sub_indptr[i + 1] - out_start;
      auto emit = [&](int64_t j, int64_t off) {
        out_indices[out_start + j] = indices ? indices[in_start + off] : in_start + off;
        out_select[out_start + j] = in_start + off;
        if (out_coo_col) out_coo_col[out_start + j] = i;
      };
      if (replace) {
        cdf.resize((size_t)deg);
        uint64_t total = integer_cdf(probs + in_start, deg, cdf.data());
        for (int64_t j = 0; j < cnt; ++j)
          emit(j, cdf_pick(cdf.data(), deg, total, rng, (uint64_t)i, (uint64_t)j));
      } else if (deg <= fanout) {
        for (int64_t j = 0; j < cnt; ++j) emit(j, j);
      } else {
        keys.resize((size_t)deg);
        for (int64_t j = 0; j < deg; ++j)
          keys[(size_t)j] = {weighted_key(rng, (uint64_t)i, (uint64_t)j, probs[in_start + j]), j};
        std::partial_sort(keys.begin(), keys.begin() + fanout, keys.end());
        for (int64_t j = 0; j < cnt; ++j) emit(j, keys[(size_t)j].idx);
      }
    }
  }
}

// Collective (list) sampling, weighted.  range == NULL: one list of n items.
// Otherwise range[num_segments + 1] delimits segments; per segment
// min(K, n_b) picks; indices are global positions
// (src/cuda/batch/list_sampling_probs.cu:30-100).  out_range[b] = picks before
// segment b.  Returns the number of picks.  n <= K without replacement: all
// items in order (src/cuda/list_sampling_probs.cu:16-19).
int64_t gs_list_sample_weighted_cpu(const float* probs, int64_t n, int64_t num_picks,
                                    int replace, const int64_t* range,
                                    int64_t num_segments, uint64_t seed,
                                    uint64_t call_id, int64_t* out_index,
                                    int64_t* out_range) {
  Stream rng(seed, call_id);
  int64_t total_out = 0;
  const int64_t nseg = range ? num_segments : 1;
  std::vector<KeyIdx> keys;
  std::vector<uint64_t> cdf;
  for (int64_t b = 0; b < nseg; ++b) {
    int64_t lo = range ? range[b] : 0, hi = range ? range[b + 1] : n;
    int64_t nb = hi - lo;
    if (out_range) out_range[b] = total_out;
    if (replace) {
      if (nb == 0) continue;
      cdf.resize((size_t)nb);
      uint64_t total = integer_cdf(probs + lo, nb, cdf.data());
      for (int64_t k = 0; k < num_picks; ++k)
        if (out_index)
          out_index[total_out + k] =
              lo + cdf_pick(cdf.data(), nb, total, rng, (uint64_t)b, (uint64_t)k);
      total_out += num_picks;
    } else if (nb <= num_picks) {
      if (out_index)
        for (int64_t k = 0; k < nb; ++k) out_index[total_out + k] = lo + k;
      total_out += nb;
    } else {
      keys.resize((size_t)nb);
      for (int64_t j = 0; j < nb; ++j)
        keys[(size_t)j] = {weighted_key(rng, (uint64_t)(lo + j), 0, probs[lo + j]), lo + j};
      std::stable_sort(keys.begin(), keys.end());
      if (out_index)
        for (int64_t k = 0; k < num_picks; ++k) out_index[total_out + k] = keys[(size_t)k].idx;
      total_out += num_picks;
    }
  }
  if (out_range) out_range[nseg] = total_out;
  return total_out;
}

}  // extern "C"

// Uniform collective sampling, src/cuda/list_sampling.cu:21-68: the per-column
// sampler on one virtual column 0..n-1 (stream position 0).
extern "C" int64_t gs_list_sample_uniform_cpu(int64_t n, int64_t num_picks,
                                              int replace, int algo, uint64_t seed,
                                              uint64_t call_id, int64_t* out_index) {
  int64_t indptr[2] = {0, n};
  int64_t sub[2];
  gs_csc_col_count_cpu(indptr, 1, nullptr, 1, num_picks, replace, sub);
  if (out_index && sub[1] > 0) {
    std::vector<int64_t> sel((size_t)sub[1]);
    gs_csc_col_sample_uniform_fill_cpu(indptr, 1, nullptr, nullptr, 1, num_picks,
                                       replace, algo, seed, call_id, sub, nullptr,
                                       out_index, sel.data());
  }
  return sub[1];
}

// -------------------------------------------------------------------------
// Walks.  Trace layout out[step * N + walk] (src/cuda/fusion/random_walk.cu:34).
//  random walk (:30-46): curr == -1 or deg == 0 -> -1, else a uniform row id of
//  column curr; stream pos = walk, draw = step.
//  node2vec (src/cuda/fusion/node2vec.cu:90-135), per step with deg > 1, per
//  attempt (stream draw = step << 32 | attempt, one Philox block: w2 -> u,
//  w1:w0 -> candidate):
//    y = (int)floor(u * max(p, q));  reject if y >= max(max(p, q), 1);
//    candidate = uniform row id of column curr;
//    accept if y < min(p, q, 1);
//    else h = p if candidate == previous, q if candidate is a row id of column
//    `previous` (sorted, binary search), 1 otherwise;  accept if y < h.
//  deg == 1 takes the only neighbour.  The reference starts with previous =
//  thread id (:89); here there is no previous node before the first step.  Its
//  candidate index floor(u * deg) can reach deg when u == 1; bounded() cannot.
//  After 2^16 attempts the last candidate is taken (never reached in practice;
//  it bounds the loop).
namespace {
bool sorted_contains(const int64_t* ptr, int64_t n, int64_t target) {
  return std::binary_search(ptr, ptr + n, target);
}
}  // namespace

extern "C" {

void gs_random_walk_cpu(const int64_t* indptr, const int64_t* indices,
                        int64_t num_cols, const int64_t* seeds, int64_t num_seeds,
                        int64_t walk_length, uint64_t seed, uint64_t call_id,
                        int64_t* out) {
  Stream rng(seed, call_id);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < num_seeds; ++i) {
    int64_t curr = seeds[i];
    out[i] = curr;
    for (int64_t step = 1; step <= walk_length; ++step) {
      int64_t pick = -1;
      if (curr >= 0 && curr < num_cols) {
        int64_t deg = indptr[curr + 1] - indptr[curr];
        if (deg > 0)
          pick = indices[indptr[curr] +
                         (int64_t)rng.bounded((uint64_t)i, (uint64_t)step, (uint64_t)deg)];
      }
      curr = pick;
      out[step * num_seeds + i] = pick;
    }
  }
}

void gs_node2vec_cpu(const int64_t* indptr, const int64_t* indices,
                     int64_t num_cols, const int64_t* seeds, int64_t num_seeds,
                     int64_t walk_length, double p, double q, uint64_t seed,
                     uint64_t call_id, int64_t* out) {
  Stream rng(seed, call_id);
  const double max_scale = std::max(p, q);
  const double reject_from = std::max(max_scale, 1.0);
  const double accept_below = std::min(std::min(p, q), 1.0);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < num_seeds; ++i) {
    int64_t curr = seeds[i], last = -1;
    out[i] = curr;
    for (int64_t step = 1; step <= walk_length; ++step) {
      int64_t pick = -1;
      if (curr >= 0 && curr < num_cols) {
        int64_t start = indptr[curr], deg = indptr[curr + 1] - start;
        if (deg == 1) {
          pick = indices[start];
        } else if (deg > 1) {
          for (uint32_t attempt = 0;; ++attempt) {
            U4 w = rng.words((uint64_t)i, ((uint64_t)step << 32) | attempt);
            double u = (double)((w.v[2] >> 8) + 1u) * 0x1p-24;
            int y = (int)std::floor(u * max_scale);
            uint64_t r = ((uint64_t)w.v[1] << 32) | w.v[0];
            int64_t cand =
                indices[start + (int64_t)(((unsigned __int128)r * (uint64_t)deg) >> 64)];
            pick = cand;
            if (attempt + 1 >= (1u << 16)) break;
            if ((double)y >= reject_from) continue;
            if ((double)y < accept_below) break;
            double h = 1.0;
            if (cand == last)
              h = p;
            else if (last >= 0 && last < num_cols &&
                     sorted_contains(indices + indptr[last],
                                     indptr[last + 1] - indptr[last], cand))
              h = q;
            if ((double)y < h) break;
          }
        }
      }
      last = curr;
      curr = pick;
      out[step * num_seeds + i] = pick;
    }
  }
}

// Sort of the row ids inside every column, src/cuda/sort_indices.cu:11-37.
void gs_segment_sort_i64_cpu(const int64_t* indptr, int64_t num_segments,
                             const int64_t* keys_in, int64_t* keys_out) {
  for (int64_t c = 0; c < num_segments; ++c) {
    std::copy(keys_in + indptr[c], keys_in + indptr[c + 1], keys_out + indptr[c]);
    std::sort(keys_out + indptr[c], keys_out + indptr[c + 1]);
  }
}

}  // extern "C"

// -------------------------------------------------------------------------
// Weighted sampling through a persistent CDF (no counterpart in the
// reference, whose A-Res kernel reads every weight of a column on every call,
// src/cuda/sampling_probs.cu:25-110; the distribution is the same: successive
// weighted sampling without replacement, which is what A-Res produces).
//  cdf[0] = row_bits, cdf[e + 1] = share(e) << row_bits | indices[e], where
//  share(e) = floor(G(e) * 2^cb / T) for G(e) < T and 2^cb - 1 for G(e) = T > 0
//  (0 when T = 0); G = inclusive prefix sums inside the column of the weights
//  quantised to 31 bits against the column's maximum exactly as integer_cdf()
//  does, T = the column's total, cb = min(62, 64 - row_bits); row_bits = the
//  bits that ids below num_rows need, or 0 (no ids packed) when there are no
//  indices or they need more than 32 bits.
//  Without replacement, deg > fanout: draw d = 0, 1, ... takes r uniform in the
//  mass that is left, walks the intervals already taken in ascending order
//  (r >= start ? r += len) and picks the item whose interval holds r -- the
//  textbook form of successive sampling.  Output in draw order; when the
//  positive mass runs out, zero-weight items follow in index order.
//  With replacement: slot j picks the item holding a uniform point of the
//  total; a column without positive weights gives its last item.
//  Streams: pos = column position, draw = slot.
extern "C" void gs_weight_cdf_build_cpu(const int64_t* indptr, int64_t num_cols,
                                        const int64_t* indices, int64_t num_rows,
                                        const float* probs, int64_t nnz,
                                        int64_t* cdf) {
  int row_bits = 0;
  if (indices) {
    row_bits = 1;
    while (row_bits < 63 && (int64_t(1) << row_bits) < num_rows) ++row_bits;
    if (row_bits > 32) row_bits = 0;
  }
  const int cb = std::min(62, 64 - row_bits);
  const uint64_t full = (uint64_t(1) << cb) - 1;
  uint64_t* out = (uint64_t*)cdf;
  out[0] = (uint64_t)row_bits;
  (void)nnz;
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t c = 0; c < num_cols; ++c) {
    const int64_t lo = indptr[c], hi = indptr[c + 1];
    float wmax = 0.0f;
    for (int64_t e = lo; e < hi; ++e)
      if (probs[e] > wmax) wmax = probs[e];
    const double scale = wmax > 0.0f ? det_div(2147483648.0, (double)wmax) : 0.0;
    auto q = [&](int64_t e) -> uint64_t {
      return wmax > 0.0f && probs[e] > 0.0f ? (uint64_t)((double)probs[e] * scale) : 0;
    };
    uint64_t total = 0;
    for (int64_t e = lo; e < hi; ++e) total += q(e);
    uint64_t g = 0;
    for (int64_t e = lo; e < hi; ++e) {
      g += q(e);
      uint64_t share = 0;
      if (total > 0)
        share = g == total ? full
                           : (uint64_t)(((unsigned __int128)g << cb) / (unsigned __int128)total);
      const uint64_t row =
          row_bits ? ((uint64_t)indices[e] & (~uint64_t(0) >> (64 - row_bits))) : 0;
      out[e + 1] = (share << row_bits) | row;
    }
  }
}

extern "C" void gs_csc_col_sample_weighted_cdf_fill_cpu(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const int64_t* cdf, const int64_t* column_ids, int64_t num_items,
    int64_t fanout, int replace, uint64_t seed, uint64_t call_id,
    const int64_t* sub_indptr, int64_t* out_coo_col, int64_t* out_indices,
    int64_t* out_select) {
  Stream rng(seed, call_id);
  const uint64_t* packed = (const uint64_t*)cdf;
  const int row_bits = (int)packed[0];
  const uint64_t row_mask = row_bits ? (~uint64_t(0) >> (64 - row_bits)) : 0;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < num_items; ++i) {
    const int64_t c = column_ids ? column_ids[i] : i;
    const int64_t deg = col_degree(indptr, num_cols, c);
    if (deg == 0) continue;
    const int64_t in_start = indptr[c], out_start = sub_indptr[i];
    const uint64_t* col = packed + 1 + in_start;  // entry of item j at col[j]
    // start(j): the share at which item j begins, 0 <= j <= deg
    std::vector<uint64_t> start((size_t)deg + 1, 0);
    for (int64_t j = 0; j < deg; ++j) start[(size_t)j + 1] = col[j] >> row_bits;
    auto emit = [&](int64_t j, int64_t off) {
      int64_t row = in_start + off;
      if (row_bits) row = (int64_t)(col[off] & row_mask);
      else if (indices) row = indices[in_start + off];
      out_indices[out_start + j] = row;
      out_select[out_start + j] = in_start + off;
      if (out_coo_col) out_coo_col[out_start + j] = i;
    };
    const uint64_t total = start[(size_t)deg];
    // item whose interval [start(j), start(j + 1)) holds the point x
    auto locate = [&](uint64_t x) {
      return (int64_t)(std::upper_bound(start.begin(), start.end(), x) - start.begin()) - 1;
    };
    if (replace) {
      for (int64_t j = 0; j < fanout; ++j)
        emit(j, total > 0 ? locate(rng.bounded((uint64_t)i, (uint64_t)j, total)) : deg - 1);
      continue;
    }
    if (deg <= fanout) {
      for (int64_t j = 0; j < deg; ++j) emit(j, j);
      continue;
    }
    // Draw d takes a uniform point r of the mass that is left, walks the
    // intervals already taken in ascending order (r >= start ? r += len) and
    // picks the item whose interval holds r: no draw repeats an item.
    std::vector<std::pair<uint64_t, uint64_t>> taken_iv;  // (start, len), ascending
    uint64_t removed = 0;
    int64_t taken = 0;
    for (; taken < fanout && removed < total; ++taken) {
      uint64_t r = rng.bounded((uint64_t)i, (uint64_t)taken, total - removed);
      size_t at = 0;
      for (; at < taken_iv.size() && r >= taken_iv[at].first; ++at) r += taken_iv[at].second;
      const int64_t off = locate(r);
      emit(taken, off);
      const uint64_t len = start[(size_t)off + 1] - start[(size_t)off];
      taken_iv.insert(taken_iv.begin() + (std::ptrdiff_t)at, {start[(size_t)off], len});
      removed += len;
    }
    for (int64_t off = 0; taken < fanout && off < deg; ++off)
      if (start[(size_t)off + 1] == start[(size_t)off]) emit(taken++, off);
  }
}

// -------------------------------------------------------------------------
// Row gather, out[i, :] = table[ids[i], :] over rows of row_bytes bytes:
// IndexSelectSingleKernel of src/cuda/index_select_uvm.cu:9-19 generalised
// from scalars to rows (what dgl.utils.gather_pinned_tensor_rows does for
// python/gs/matrix_api/matrix.py:19-23).  An id outside [0, num_rows) gives a
// row of zero bytes and is counted.
extern "C" void gs_gather_rows_cpu(const void* table, int64_t num_rows,
                                   int64_t row_bytes, const int64_t* ids, int64_t n,
                                   void* out, int64_t* bad_count) {
  int64_t bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
  for (int64_t i = 0; i < n; ++i) {
    char* dst = (char*)out + i * row_bytes;
    if (ids[i] >= 0 && ids[i] < num_rows)
      std::memcpy(dst, (const char*)table + ids[i] * row_bytes, (size_t)row_bytes);
    else {
      std::memset(dst, 0, (size_t)row_bytes);
      ++bad;
    }
  }
  if (bad_count) *bad_count = bad;
}

// Stable sort of edge positions by their id on the axis to compress (the
// first half of COO2CSCCUDA, src/cuda/format_transform.cu:65-84,121-142).
extern "C" void gs_coo_sort_cpu(const int64_t* major, int64_t nnz, int64_t* sorted_major,
                                int64_t* perm) {
  for (int64_t e = 0; e < nnz; ++e) perm[e] = e;
  std::stable_sort(perm, perm + nnz,
                   [major](int64_t a, int64_t b) { return major[a] < major[b]; });
  for (int64_t e = 0; e < nnz; ++e) sorted_major[e] = major[perm[e]];
}
