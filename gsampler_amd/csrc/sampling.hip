// sampling.hip -- uniform per-column sampling, optionally fused with the
// column slice (the GraphSAGE kernel).
//
// Work mapping: a slice of one wavefront owns one requested column, so that a
// wavefront keeps several independent columns -- and their dependent seed ->
// indptr -> indices load chains -- in flight at once.  With one lane per
// output slot (fanout <= 64, Floyd's rule or sampling with replacement) the
// slice is exactly `fanout` lanes; otherwise it is a power-of-two group that
// strides over the slots.  Exchange inside a slice uses wavefront shuffles
// only, so divergent columns never meet at a block barrier.
#include "common.h"

namespace gs {

// Reads a value that other lanes may have updated with an atomic, bypassing
// the per-CU vector cache.
__device__ __forceinline__ int64_t load_coherent(const int64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One column by a group of G lanes, any fanout: slots are strided over the
// lanes.  The path of the reservoir algorithm and of fanouts above 64.
template <int G, typename IdxT>
__device__ __forceinline__ void sample_column_generic(
    int lane, int64_t item, int64_t col_label, int64_t in_start, int64_t deg, int64_t out_start,
    const IdxT* __restrict__ indices, int64_t fanout, int replace,
    PhiloxKey key, int64_t* __restrict__ out_coo_col,
    int64_t* __restrict__ out_indices, int64_t* __restrict__ out_select) {
  const uint64_t pos = (uint64_t)item;
  if (replace) {
    // slot j takes a uniform position of the column
    for (int64_t j = lane; j < fanout; j += G) {
      int64_t p = in_start + (int64_t)philox_bounded(key, pos, (uint64_t)j,
                                                      (uint64_t)deg);
      out_indices[out_start + j] = indices ? (int64_t)indices[p] : p;
      out_select[out_start + j] = p;
      if (out_coo_col) out_coo_col[out_start + j] = col_label;
    }
    return;
  }
  if (deg <= fanout) {
    // the whole column, original order
    for (int64_t j = lane; j < deg; j += G) {
      int64_t p = in_start + j;
      out_indices[out_start + j] = indices ? (int64_t)indices[p] : p;
      out_select[out_start + j] = p;
      if (out_coo_col) out_coo_col[out_start + j] = col_label;
    }
    return;
  }
  // Reservoir (Algorithm R in max-form): slot[j] = j, then every idx in
  // [fanout, deg) draws num in [0, idx]; if num < fanout the slot keeps the
  // largest idx that hit it.  The slots live in out_select until the final
  // gather.  Order-independent, so lanes take idx values strided by G.
  for (int64_t jj = lane; jj < fanout; jj += G) out_select[out_start + jj] = jj;
  // (the slots are shared among lanes of this wavefront only; a fence for the
  // whole device would make the die write its L2 back)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  for (int64_t idx = fanout + lane; idx < deg; idx += G) {
    int64_t num = (int64_t)philox_bounded(key, pos, (uint64_t)idx,
                                          (uint64_t)idx + 1);
    if (num < fanout)
      atomicMax((long long*)(out_select + out_start + num), (long long)idx);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
  __builtin_amdgcn_wave_barrier();
  for (int64_t jj = lane; jj < fanout; jj += G) {
    int64_t p = in_start + load_coherent(out_select + out_start + jj);
    out_indices[out_start + jj] = indices ? (int64_t)indices[p] : p;
    out_select[out_start + jj] = p;
    if (out_coo_col) out_coo_col[out_start + jj] = col_label;
  }
}

// Floyd's subset sampling, one lane per output slot: slot i of a column is lane
// gbase + i of the wavefront (K <= 64 slots).  Slot i draws t_i in [0, j_i],
// j_i = deg - K + i, and keeps t_i unless an earlier slot already holds it, in
// which case it keeps j_i.  "Already held" <=> some earlier slot drew the same
// t, or t_i equals the j_m of an earlier slot m that fell back to j_m; m is
// then unique (m = t_i - (deg - K)), so the fall-back flags form a chain that
// is settled by visiting slots in increasing order.  Returns the slot's offset
// inside the column.
__device__ __forceinline__ int64_t floyd_slot_packed(int lane, int gbase, int K, int64_t deg,
                                                     PhiloxKey key, uint64_t pos) {
  const int64_t base = deg - K;
  const int64_t j = base + lane;
  const int64_t t = (int64_t)philox_bounded(key, pos, (uint64_t)lane, (uint64_t)j + 1);
  bool dup = false;
  for (int m = 0; m < K; ++m) {
    const int64_t tm = __shfl(t, gbase + m, kWave);
    dup |= (m < lane) & (tm == t);
  }
  const int64_t mi = t - base;  // slot whose j equals my t, if in [0, lane)
  for (int m = 0; m < K; ++m) {
    const int dm = __shfl((int)dup, gbase + m, kWave);
    if (mi == m && m < lane) dup |= (dm != 0);
  }
  return dup ? j : t;
}

// One lane per output slot, a column on exactly `fanout` consecutive lanes: a
// wavefront holds 64 / fanout columns (twelve at fanout 5, where power-of-two
// groups would hold eight).  Lanes past the last whole slice idle.  On a
// 124M-edge power-law graph the kernel moves about 6 TB/s through the memory
// fabric, nearly all of it the 128-byte lines behind 4- or 8-byte picks;
// giving a slice several columns to pipeline measured 3 % to 20 % slower.
// kProbe (0 in every operator) switches parts of the kernel off for the
// measurement that prices them (gs_probe_sample_uniform): 1 a multiplicative hash
// instead of Philox, 2 no exchange among a column's lanes (repeats are kept),
// 4 no read of the column pointer (every column `probe_degree` long, starting at
// id * probe_degree), 8 no read of the row ids, 16 only the row id is stored,
// 32 nothing is stored.
constexpr int kProbeHash = 1, kProbeNoExchange = 2, kProbeNoIndptr = 4, kProbeNoIndices = 8,
              kProbeOneStore = 16, kProbeNoStore = 32;
template <typename IdxT, int kProbe = 0>
__global__ __launch_bounds__(kBlock) void sample_uniform_packed_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const IdxT* __restrict__ indices, const int64_t* __restrict__ column_ids,
    int64_t num_items, int fanout, int cols_per_wave, int replace, PhiloxKey key,
    const int64_t* __restrict__ sub_indptr, int64_t* __restrict__ out_coo_col,
    int64_t* __restrict__ out_indices, int64_t* __restrict__ out_select,
    ColumnLabels labels, const int64_t* __restrict__ col_span, int64_t probe_degree = 0) {
  const int wave_lane = threadIdx.x & (kWave - 1);
  const int group = wave_lane / fanout;
  const int lane = wave_lane - group * fanout;
  // die x (work-groups x, x + 8, ...) takes the x-th eighth of the columns in order
  const int64_t per_die = gridDim.x / 8;
  const int64_t block = (int64_t)(blockIdx.x % 8) * per_die + blockIdx.x / 8;
  const int64_t wave = (block * kBlock + threadIdx.x) / kWave;
  const int64_t item = wave * cols_per_wave + group;
  if (group >= cols_per_wave || item >= num_items) return;  // whole groups leave together
  // (asked for here, so that its loads travel with the ones below)
  const int64_t col_label = out_coo_col ? labels.of_near(item, wave * cols_per_wave) : item;
  int64_t in_start;
  int64_t deg;
  if (kProbe & kProbeNoIndptr) {
    deg = probe_degree;
    in_start = (column_ids ? column_ids[item] : item) * probe_degree;
  } else {
    deg = column_span(col_span, column_ids, indptr, num_cols, item, &in_start);
  }
  if (deg == 0) return;
  const int64_t out_start = (kProbe & kProbeNoIndptr) ? item * fanout : sub_indptr[item];
  int64_t p = -1;
  if (replace) {
    p = in_start + (int64_t)philox_bounded(key, (uint64_t)item, (uint64_t)lane, (uint64_t)deg);
  } else if (deg <= fanout) {
    if (lane < deg) p = in_start + lane;  // whole column, in order
  } else if (kProbe & (kProbeHash | kProbeNoExchange)) {
    const int64_t j = deg - fanout + lane;
    uint64_t r;
    if (kProbe & kProbeHash) {
      r = ((uint64_t)item * 64 + (uint64_t)lane + key.k0) * 0x9E3779B97F4A7C15ull;
      r ^= r >> 31;
      r = __umul64hi(r * 0xBF58476D1CE4E5B9ull, (uint64_t)j + 1);
    } else {
      r = philox_bounded(key, (uint64_t)item, (uint64_t)lane, (uint64_t)j + 1);
    }
    p = in_start + (int64_t)r;
    if (!(kProbe & kProbeNoExchange)) {  // the exchange of floyd_slot_packed on these draws
      const int gbase = group * fanout;
      const int64_t t = (int64_t)r, base = deg - fanout;
      bool dup = false;
      for (int m = 0; m < fanout; ++m) {
        const int64_t tm = __shfl(t, gbase + m, kWave);
        dup |= (m < lane) & (tm == t);
      }
      const int64_t mi = t - base;
      for (int m = 0; m < fanout; ++m) {
        const int dm = __shfl((int)dup, gbase + m, kWave);
        if (mi == m && m < lane) dup |= (dm != 0);
      }
      p = in_start + (dup ? j : t);
    }
  } else {
    p = in_start + floyd_slot_packed(lane, group * fanout, fanout, deg, key, (uint64_t)item);
  }
  if (p < 0) return;
  const int64_t v = (indices && !(kProbe & kProbeNoIndices)) ? (int64_t)indices[p] : p;
  if (kProbe & kProbeNoStore) {
    // keep the pick (and the row id behind it) live without a store that happens
    if (v == -7777) out_indices[0] = p;  // ids are not negative; the compiler cannot know
    return;
  }
  out_indices[out_start + lane] = v;
  if (kProbe & kProbeOneStore) return;
  out_select[out_start + lane] = p;
  if (out_coo_col) out_coo_col[out_start + lane] = col_label;
}

// Any fanout, any algorithm: a group of G lanes (a power of two) owns a column
// and strides over its slots.  The path of the reservoir algorithm and of
// fanouts above 64.
template <int G, typename IdxT>
__global__ __launch_bounds__(kBlock) void sample_uniform_strided_kernel(
    const int64_t* __restrict__ indptr, int64_t num_cols,
    const IdxT* __restrict__ indices, const int64_t* __restrict__ column_ids,
    int64_t num_items, int64_t fanout, int replace, PhiloxKey key,
    const int64_t* __restrict__ sub_indptr, int64_t* __restrict__ out_coo_col,
    int64_t* __restrict__ out_indices, int64_t* __restrict__ out_select, ColumnLabels labels,
    const int64_t* __restrict__ col_span) {
  const int lane = threadIdx.x & (G - 1);
  const int64_t item = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / G;
  if (item >= num_items) return;  // whole groups leave together
  int64_t in_start;
  const int64_t deg = column_span(col_span, column_ids, indptr, num_cols, item, &in_start);
  if (deg == 0) return;
  sample_column_generic<G, IdxT>(lane, item, out_coo_col ? labels.of(item) : item, in_start, deg,
                                 sub_indptr[item], indices, fanout, replace, key, out_coo_col,
                                 out_indices, out_select);
}

template <int G, typename IdxT>
static int launch_sample_strided(const int64_t* indptr, int64_t num_cols, const IdxT* indices,
                                 const int64_t* column_ids, int64_t num_items, int64_t fanout,
                                 int replace, PhiloxKey key, const int64_t* sub_indptr,
                                 int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
                                 ColumnLabels labels, const int64_t* col_span,
                                 hipStream_t stream) {
  const int64_t blocks = ceil_div(num_items * G, kBlock);
  GS_LAUNCH("sample_uniform", stream,
            (sample_uniform_strided_kernel<G, IdxT>)<<<dim3((unsigned)blocks), dim3(kBlock), 0,
                                                      stream>>>(
                indptr, num_cols, indices, column_ids, num_items, fanout, replace, key,
                sub_indptr, out_coo_col, out_indices, out_select, labels, col_span));
  return GS_OK;
}

}  // namespace gs

namespace gs {
template <typename IdxT>
static int sample_uniform_fill(const int64_t* indptr, int64_t num_cols, const IdxT* indices,
                               const int64_t* column_ids, int64_t num_items, int64_t fanout,
                               int replace, int algo, uint64_t seed, uint64_t call_id,
                               const int64_t* sub_indptr, const int64_t* col_span,
                               int64_t* out_coo_col, int64_t* out_indices,
                               int64_t* out_select, const int64_t* col_batch_ptr,
                               int64_t num_col_batches, gs_stream_t stream) {
  GS_REQUIRE(num_items >= 0 && num_cols >= 0, "sample_uniform: negative size");
  GS_REQUIRE(col_batch_ptr == nullptr || num_col_batches >= 1,
             "sample_uniform: col_batch_ptr given but num_col_batches = %lld",
             (long long)num_col_batches);
  const ColumnLabels labels{col_batch_ptr, num_col_batches};
  GS_REQUIRE(fanout >= 0, "sample_uniform: negative fanout %lld",
             (long long)fanout);
  GS_REQUIRE(algo == GS_ALGO_AUTO || algo == GS_ALGO_RESERVOIR ||
                 algo == GS_ALGO_FLOYD,
             "sample_uniform: unknown algorithm %d", algo);
  GS_REQUIRE(!(algo == GS_ALGO_FLOYD && fanout > 64),
             "sample_uniform: Floyd sampling needs fanout <= 64, got %lld",
             (long long)fanout);
  if (num_items == 0 || fanout == 0) return GS_OK;
  GS_REQUIRE(indptr && sub_indptr && out_indices && out_select,
             "sample_uniform: null pointer");
  GS_REQUIRE(column_ids != nullptr || num_items <= num_cols,
             "sample_uniform: %lld items but the matrix has %lld columns",
             (long long)num_items, (long long)num_cols);
  if (algo == GS_ALGO_AUTO)
    algo = fanout <= 64 ? GS_ALGO_FLOYD : GS_ALGO_RESERVOIR;
  const PhiloxKey key = make_key(seed, call_id);
  hipStream_t s = as_stream(stream);
  if (fanout <= kWave && (replace || algo == GS_ALGO_FLOYD)) {
    const int cols_per_wave = kWave / (int)fanout;
    const int64_t waves = ceil_div(num_items, cols_per_wave);
    GS_LAUNCH("sample_uniform", s,
              sample_uniform_packed_kernel<IdxT><<<dim3((unsigned)(ceil_div(ceil_div(waves * kWave, kBlock), 8) * 8)),
                                                   dim3(kBlock), 0, s>>>(
                  indptr, num_cols, indices, column_ids, num_items, (int)fanout, cols_per_wave,
                  replace, key, sub_indptr, out_coo_col, out_indices, out_select, labels,
                  col_span));
    return GS_OK;
  }
#define GS_SAMPLE_ARGS                                                          \
  indptr, num_cols, indices, column_ids, num_items, fanout, replace, key, sub_indptr, \
      out_coo_col, out_indices, out_select, labels, col_span, s
  if (fanout <= 8) return launch_sample_strided<8, IdxT>(GS_SAMPLE_ARGS);
  if (fanout <= 16) return launch_sample_strided<16, IdxT>(GS_SAMPLE_ARGS);
  if (fanout <= 32) return launch_sample_strided<32, IdxT>(GS_SAMPLE_ARGS);
  return launch_sample_strided<64, IdxT>(GS_SAMPLE_ARGS);
#undef GS_SAMPLE_ARGS
}
}  // namespace gs

extern "C" int gs_csc_col_sample_uniform_fill(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const int64_t* column_ids, int64_t num_items, int64_t fanout, int replace,
    int algo, uint64_t seed, uint64_t call_id, const int64_t* sub_indptr,
    const int64_t* col_span, int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    const int64_t* col_batch_ptr, int64_t num_col_batches, gs_stream_t stream) {
  return gs::sample_uniform_fill<int64_t>(indptr, num_cols, indices, column_ids, num_items,
                                          fanout, replace, algo, seed, call_id, sub_indptr,
                                          col_span, out_coo_col, out_indices, out_select, col_batch_ptr,
                                          num_col_batches, stream);
}

extern "C" int gs_csc_col_sample_uniform_fill_i32(
    const int64_t* indptr, int64_t num_cols, const int32_t* indices32,
    const int64_t* column_ids, int64_t num_items, int64_t fanout, int replace,
    int algo, uint64_t seed, uint64_t call_id, const int64_t* sub_indptr,
    const int64_t* col_span, int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    const int64_t* col_batch_ptr, int64_t num_col_batches, gs_stream_t stream) {
  GS_REQUIRE(indices32 != nullptr, "sample_uniform_i32: null indices");
  return gs::sample_uniform_fill<int32_t>(indptr, num_cols, indices32, column_ids, num_items,
                                          fanout, replace, algo, seed, call_id, sub_indptr,
                                          col_span, out_coo_col, out_indices, out_select, col_batch_ptr,
                                          num_col_batches, stream);
}

// One launch of the packed sampler with parts switched off (`variant` = a sum of
// the kProbe* bits above); int32 row ids, fanout <= 64, without replacement.
// With kProbeNoIndptr the columns are taken to be probe_degree long and the
// outputs need num_items * fanout entries.  Measurement only: the picks of a
// variant are not those of the operator.
extern "C" int gs_probe_sample_uniform(
    const int64_t* indptr, int64_t num_cols, const int32_t* indices32,
    const int64_t* column_ids, int64_t num_items, int64_t fanout, int variant,
    int64_t probe_degree, uint64_t seed, uint64_t call_id, const int64_t* sub_indptr,
    const int64_t* col_span, int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(num_items > 0 && fanout >= 1 && fanout <= kWave, "probe_sample_uniform: bad size");
  GS_REQUIRE(indptr && indices32 && column_ids && sub_indptr && out_indices && out_select,
             "probe_sample_uniform: null pointer");
  GS_REQUIRE(!(variant & kProbeNoIndptr) || probe_degree > fanout,
             "probe_sample_uniform: probe_degree must exceed the fanout");
  const PhiloxKey key = make_key(seed, call_id);
  hipStream_t s = as_stream(stream);
  const int cols_per_wave = kWave / (int)fanout;
  const int64_t waves = ceil_div(num_items, cols_per_wave);
  const dim3 grid((unsigned)(ceil_div(ceil_div(waves * kWave, kBlock), 8) * 8));
#define GS_PROBE_CASE(V)                                                                      \
  case V:                                                                                     \
    GS_LAUNCH("probe_sample_uniform", s,                                                      \
              (sample_uniform_packed_kernel<int32_t, V>)<<<grid, dim3(kBlock), 0, s>>>(       \
                  indptr, num_cols, indices32, column_ids, num_items, (int)fanout,            \
                  cols_per_wave, 0, key, sub_indptr, out_coo_col, out_indices, out_select,    \
                  ColumnLabels{nullptr, 0}, col_span, probe_degree));                         \
    return GS_OK;
  switch (variant) {
    GS_PROBE_CASE(0)
    GS_PROBE_CASE(kProbeHash)
    GS_PROBE_CASE(kProbeNoExchange)
    GS_PROBE_CASE(kProbeNoIndptr)
    GS_PROBE_CASE(kProbeNoIndices)
    GS_PROBE_CASE(kProbeNoIndices | kProbeOneStore)
    GS_PROBE_CASE(kProbeOneStore)
    GS_PROBE_CASE(kProbeNoStore)
    GS_PROBE_CASE(kProbeNoIndices | kProbeNoStore)
    default:
      break;
  }
#undef GS_PROBE_CASE
  set_error("probe_sample_uniform: variant %d is not built", variant);
  return GS_ERR_INVALID;
}

// ---------------------------------------------------------------------------
// Uniform collective (list) sampling: K of the positions 0..n-1.  It is the
// per-column sampler applied to one virtual column whose row ids are the
// positions themselves (stream position 0), so it produces exactly what
// gs_csc_col_sample_uniform_fill would for that column; the reservoir form is
// spread over the whole grid because a list can be far longer than a column.
namespace gs {

__global__ __launch_bounds__(kBlock) void list_uniform_kernel(
    int64_t n, int64_t num_picks, int mode, PhiloxKey key,
    int64_t* __restrict__ out) {
  // mode 0: with replacement; 1: identity (n <= picks); 2: reservoir slot init
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num_picks) return;
  out[j] = mode == 0 ? (int64_t)philox_bounded(key, 0, (uint64_t)j, (uint64_t)n) : j;
}

__global__ __launch_bounds__(kBlock) void list_reservoir_kernel(
    int64_t n, int64_t num_picks, PhiloxKey key, int64_t* out) {
  const int64_t idx = num_picks + (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= n) return;
  const int64_t num = (int64_t)philox_bounded(key, 0, (uint64_t)idx, (uint64_t)idx + 1);
  if (num < num_picks) atomicMax((long long*)(out + num), (long long)idx);
}

// One wavefront, one lane per slot (num_picks <= 64): the Floyd rule of
// sample_uniform_kernel on the virtual column.
__global__ void list_floyd_kernel(int64_t n, int num_picks, PhiloxKey key,
                                  int64_t* __restrict__ out) {
  const int lane = threadIdx.x;
  const int K = num_picks;
  const int64_t base = n - K;
  const int64_t j = base + lane;
  int64_t t = -1;
  if (lane < K) t = (int64_t)philox_bounded(key, 0, (uint64_t)lane, (uint64_t)j + 1);
  bool dup = false;
  for (int m = 0; m < K; ++m) {
    const int64_t tm = __shfl(t, m, kWave);
    dup |= (m < lane) & (tm == t);
  }
  const int64_t mi = t - base;
  for (int m = 0; m < K; ++m) {
    const int dm = __shfl((int)dup, m, kWave);
    if (mi == m && m < lane) dup |= (dm != 0);
  }
  if (lane < K) out[lane] = dup ? j : t;
}

}  // namespace gs

extern "C" int gs_list_sample_uniform(int64_t n, int64_t num_picks, int replace,
                                      int algo, uint64_t seed, uint64_t call_id,
                                      int64_t* out_index, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0 && num_picks >= 0, "list_sample_uniform: negative size");
  GS_REQUIRE(algo == GS_ALGO_AUTO || algo == GS_ALGO_RESERVOIR || algo == GS_ALGO_FLOYD,
             "list_sample_uniform: unknown algorithm %d", algo);
  const int64_t count = replace ? (n > 0 ? num_picks : 0) : (n < num_picks ? n : num_picks);
  if (count == 0) return GS_OK;
  GS_REQUIRE(out_index, "list_sample_uniform: null output");
  const PhiloxKey key = make_key(seed, call_id);
  hipStream_t s = as_stream(stream);
  const unsigned blocks = (unsigned)ceil_div(count, kBlock);
  if (replace || n <= num_picks) {
    GS_LAUNCH("list_uniform", s,
              list_uniform_kernel<<<dim3(blocks), dim3(kBlock), 0, s>>>(
                  n, count, replace ? 0 : 1, key, out_index));
    return GS_OK;
  }
  if (algo == GS_ALGO_AUTO) algo = num_picks <= 64 ? GS_ALGO_FLOYD : GS_ALGO_RESERVOIR;
  GS_REQUIRE(!(algo == GS_ALGO_FLOYD && num_picks > 64),
             "list_sample_uniform: Floyd sampling needs num_picks <= 64");
  if (algo == GS_ALGO_FLOYD) {
    GS_LAUNCH("list_floyd", s,
              list_floyd_kernel<<<dim3(1), dim3(kWave), 0, s>>>(n, (int)num_picks,
                                                                key, out_index));
    return GS_OK;
  }
  GS_LAUNCH("list_uniform", s,
            list_uniform_kernel<<<dim3(blocks), dim3(kBlock), 0, s>>>(
                n, num_picks, 2, key, out_index));
  GS_LAUNCH("list_reservoir", s,
            list_reservoir_kernel<<<dim3((unsigned)ceil_div(n - num_picks, kBlock)),
                                    dim3(kBlock), 0, s>>>(n, num_picks, key,
                                                          out_index));
  return GS_OK;
}
