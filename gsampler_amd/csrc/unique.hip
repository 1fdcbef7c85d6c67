// unique.hip -- unique in first-occurrence order + relabel, for one batch or a
// whole super-batch in one set of launches.
//
// Keys of batch b are seeds_b ++ rows_b.  All batches are laid out back to
// back in one "flat" key space of N = num_seeds + num_rows_keys positions;
// flat_ptr[b] is where batch b starts.  Batch b owns the open-addressing table
// slots [2 * flat_ptr[b], 2 * flat_ptr[b+1])  (load factor <= 1/2, linear
// probing so that a probe sequence stays inside one 128-byte line most of the
// time).  A slot is one 64-bit word  key << 32 | value  so that insertion with
// "smallest position wins" is a single 64-bit atomicMin on the slot:
//   pass 1  insert   value = position of the key inside its batch (min wins)
//   pass 2  flag     key is a first occurrence  <=>  slot value == own position;
//                    one ballot bit per key + one count per block
//   scan of the block counts, unique_ptr from the flags
//   pass 3  fill     first occurrences write out_unique and replace the slot
//                    value by their batch-local rank
//   pass 4  relabel  one lookup per edge row; columns come from the per-seed
//                    rank array written in pass 3
#include "common.h"
#include "hashtable.h"
#include "scan.h"

namespace gs {

constexpr int kWordsPerBlock = kBlock / kWave;

struct UniqueWs {
  int64_t* flat_ptr;      // [B + 1]
  uint64_t* table;        // [2 N]
  uint64_t* flags;        // [nblocks * kWordsPerBlock]
  int64_t* block_off;     // [nblocks + 1]
  int64_t* seed_rank;     // [S]
  void* scan_ws;
  size_t scan_ws_bytes;
  size_t total;
};

static UniqueWs carve_unique(void* ws, int64_t S, int64_t E, int64_t B) {
  const int64_t N = S + E;
  const int64_t nblocks = ceil_div(N > 0 ? N : 1, kBlock);
  Carver c(ws);
  UniqueWs w;
  w.flat_ptr = c.take<int64_t>((size_t)B + 1);
  w.table = c.take<uint64_t>((size_t)(2 * N + 2));
  w.flags = c.take<uint64_t>((size_t)nblocks * kWordsPerBlock);
  w.block_off = c.take<int64_t>((size_t)nblocks + 1);
  w.seed_rank = c.take<int64_t>((size_t)(S > 0 ? S : 1));
  w.scan_ws_bytes = scan_workspace_bytes(nblocks + 1);
  w.scan_ws = c.take<char>(w.scan_ws_bytes);
  w.total = c.total();
  return w;
}

// Where a flat position lives: batch, position inside the batch, key.
struct FlatItem {
  int64_t batch, local, seed_index;  // seed_index = -1 for row keys
  uint64_t key;
  uint64_t table_base, cap;
};

__device__ __forceinline__ FlatItem locate(
    int64_t p, const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr) {
  FlatItem it;
  it.batch = B == 1 ? 0 : segment_of(flat_ptr, B, p);
  const int64_t fb = flat_ptr[it.batch];
  it.local = p - fb;
  const int64_t s_lo = seeds_ptr ? seeds_ptr[it.batch] : 0;
  const int64_t s_hi = seeds_ptr ? seeds_ptr[it.batch + 1] : S;
  const int64_t ns = s_hi - s_lo;
  if (it.local < ns) {
    it.seed_index = s_lo + it.local;
    it.key = (uint64_t)seeds[it.seed_index];
  } else {
    const int64_t r_lo = rows_ptr ? rows_ptr[it.batch] : 0;
    it.seed_index = -1;
    it.key = (uint64_t)rows[r_lo + it.local - ns];
  }
  it.table_base = 2 * (uint64_t)fb;
  it.cap = 2 * (uint64_t)(flat_ptr[it.batch + 1] - fb);
  return it;
}

__global__ void unique_flat_ptr_kernel(const int64_t* seeds_ptr, int64_t S,
                                       const int64_t* rows_ptr, int64_t E,
                                       int64_t B, int64_t* flat_ptr) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > B) return;
  const int64_t s = seeds_ptr ? seeds_ptr[b] : (b == 0 ? 0 : S);
  const int64_t r = rows_ptr ? rows_ptr[b] : (b == 0 ? 0 : E);
  flat_ptr[b] = s + r;
}

__global__ __launch_bounds__(kBlock) void unique_insert_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t N, uint64_t* table) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= N) return;
  const FlatItem it = locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr);
  table_insert_min(table + it.table_base, it.cap, it.key, (uint64_t)it.local);
}

// Keys looked up here were all inserted, so the slot always exists; slot 0
// stands in if a caller passed inconsistent pointer arrays.
__device__ __forceinline__ uint64_t find_slot(const uint64_t* tab, uint64_t cap,
                                              uint64_t key) {
  const uint64_t slot = table_find(tab, cap, key);
  return slot < cap ? slot : 0;
}

__global__ __launch_bounds__(kBlock) void unique_flag_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t N,
    const uint64_t* __restrict__ table, uint64_t* __restrict__ flags,
    int64_t* __restrict__ block_count) {
  __shared__ int wave_count[kWordsPerBlock];
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  bool first = false;
  if (p < N) {
    const FlatItem it =
        locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr);
    const uint64_t* tab = table + it.table_base;
    const uint64_t cur = tab[find_slot(tab, it.cap, it.key)];
    first = (uint32_t)cur == (uint32_t)it.local;
  }
  const uint64_t word = __ballot(first);
  const int wave = threadIdx.x / kWave;
  if (lane_id() == 0) {
    flags[(int64_t)blockIdx.x * kWordsPerBlock + wave] = word;
    wave_count[wave] = __popcll(word);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kWordsPerBlock; ++w) total += wave_count[w];
    block_count[blockIdx.x] = total;
    if (blockIdx.x == gridDim.x - 1) block_count[gridDim.x] = 0;
  }
}

// Number of first occurrences at flat positions < p.
__device__ __forceinline__ int64_t rank_before(
    int64_t p, const uint64_t* __restrict__ flags,
    const int64_t* __restrict__ block_off) {
  const int64_t blk = p / kBlock;
  int64_t r = block_off[blk];
  const int in_blk = (int)(p - blk * kBlock);
  const int full = in_blk / kWave, rem = in_blk % kWave;
  for (int w = 0; w < full; ++w)
    r += __popcll(flags[blk * kWordsPerBlock + w]);
  if (rem)
    r += __popcll(flags[blk * kWordsPerBlock + full] & ((1ull << rem) - 1));
  return r;
}

__global__ void unique_ptr_kernel(const int64_t* __restrict__ flat_ptr,
                                  int64_t B, const uint64_t* __restrict__ flags,
                                  const int64_t* __restrict__ block_off,
                                  int64_t* __restrict__ unique_ptr) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b > B) return;
  unique_ptr[b] = rank_before(flat_ptr[b], flags, block_off);
}

__global__ __launch_bounds__(kBlock) void unique_fill_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t N, uint64_t* table,
    const uint64_t* __restrict__ flags, const int64_t* __restrict__ block_off,
    const int64_t* __restrict__ unique_ptr, int64_t* __restrict__ out_unique,
    int64_t* __restrict__ seed_rank) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= N) return;
  const FlatItem it = locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr);
  const bool first = (flags[p / kWave] >> (p % kWave)) & 1ull;
  if (first) {
    const int64_t grank = rank_before(p, flags, block_off);
    const int64_t lrank = grank - unique_ptr[it.batch];
    out_unique[grank] = (int64_t)it.key;
    uint64_t* tab = table + it.table_base;
    // Only the value half changes; concurrent probes compare the key half.
    tab[find_slot(tab, it.cap, it.key)] = (it.key << 32) | (uint64_t)lrank;
    if (it.seed_index >= 0) seed_rank[it.seed_index] = lrank;
  } else if (it.seed_index >= 0) {
    seed_rank[it.seed_index] = -1;  // repeated seed: resolved by lookup later
  }
}

__global__ __launch_bounds__(kBlock) void unique_relabel_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t E,
    const uint64_t* __restrict__ table, const int64_t* __restrict__ seed_rank,
    const int64_t* __restrict__ edge_col, int64_t* __restrict__ out_row,
    int64_t* __restrict__ out_col) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= E) return;
  const int64_t b = (B == 1 || rows_ptr == nullptr) ? 0 : segment_of(rows_ptr, B, e);
  const int64_t fb = flat_ptr[b];
  const uint64_t* tab = table + 2 * (uint64_t)fb;
  const uint64_t cap = 2 * (uint64_t)(flat_ptr[b + 1] - fb);
  if (out_row) {
    const uint64_t key = (uint64_t)rows[e];
    out_row[e] = (int64_t)(uint32_t)tab[find_slot(tab, cap, key)];
  }
  if (out_col) {
    const int64_t c = edge_col[e];
    int64_t r = seed_rank[c];
    if (r < 0) r = (int64_t)(uint32_t)tab[find_slot(tab, cap, (uint64_t)seeds[c])];
    out_col[e] = r;
  }
}

static int check_unique_args(const int64_t* seeds, const int64_t* seeds_ptr,
                             int64_t S, const int64_t* rows,
                             const int64_t* rows_ptr, int64_t E, int64_t B) {
  GS_REQUIRE(S >= 0 && E >= 0, "unique: negative size");
  GS_REQUIRE(B >= 1, "unique: num_batches must be >= 1, got %lld", (long long)B);
  GS_REQUIRE(S == 0 || seeds, "unique: null seeds");
  GS_REQUIRE(E == 0 || rows, "unique: null rows");
  GS_REQUIRE((seeds_ptr == nullptr) == (rows_ptr == nullptr),
             "unique: seeds_ptr and rows_ptr must both be given or both be null");
  GS_REQUIRE(seeds_ptr != nullptr || B == 1,
             "unique: %lld batches need seeds_ptr / rows_ptr", (long long)B);
  return GS_OK;
}

}  // namespace gs

extern "C" {

size_t gs_unique_workspace_bytes(int64_t num_seeds, int64_t num_rows_keys,
                                 int64_t num_batches) {
  if (num_seeds < 0 || num_rows_keys < 0 || num_batches < 1) return 0;
  return gs::carve_unique(nullptr, num_seeds, num_rows_keys, num_batches).total;
}

int gs_unique_count(const int64_t* seeds, const int64_t* seeds_ptr,
                    int64_t num_seeds, const int64_t* rows,
                    const int64_t* rows_ptr, int64_t num_rows_keys,
                    int64_t num_batches, int64_t* unique_ptr, void* workspace,
                    size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  GS_REQUIRE(unique_ptr, "unique_count: null unique_ptr");
  UniqueWs w = carve_unique(workspace, S, E, B);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("unique workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  const int64_t N = S + E;
  if (N == 0) {
    GS_LAUNCH("unique_clear", s,
              table_fill_kernel<><<<dim3((unsigned)ceil_div(B + 1, kBlock)),
                                    dim3(kBlock), 0, s>>>((uint64_t*)unique_ptr,
                                                          B + 1, 0ull));
    return GS_OK;
  }
  const int64_t nblocks = ceil_div(N, kBlock);
  GS_LAUNCH("unique_flat_ptr", s,
            unique_flat_ptr_kernel<<<dim3((unsigned)ceil_div(B + 1, kBlock)),
                                     dim3(kBlock), 0, s>>>(seeds_ptr, S, rows_ptr,
                                                           E, B, w.flat_ptr));
  {
    const int64_t slots = 2 * N;
    int64_t blocks = ceil_div(slots, kBlock * 8);
    GS_LAUNCH("unique_clear", s,
              table_fill_kernel<><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(
                  w.table, slots, kEmptySlot));
  }
  GS_LAUNCH("unique_insert", s,
            unique_insert_kernel<<<dim3((unsigned)nblocks), dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.table));
  GS_LAUNCH("unique_flag", s,
            unique_flag_kernel<<<dim3((unsigned)nblocks), dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.table,
                w.flags, w.block_off));
  rc = exclusive_scan_i64(w.block_off, w.block_off, nblocks + 1, w.scan_ws,
                          w.scan_ws_bytes, s);
  if (rc != GS_OK) return rc;
  GS_LAUNCH("unique_ptr", s,
            unique_ptr_kernel<<<dim3((unsigned)ceil_div(B + 1, kBlock)),
                                dim3(kBlock), 0, s>>>(w.flat_ptr, B, w.flags,
                                                      w.block_off, unique_ptr));
  return GS_OK;
}

int gs_unique_fill(const int64_t* seeds, const int64_t* seeds_ptr,
                   int64_t num_seeds, const int64_t* rows,
                   const int64_t* rows_ptr, int64_t num_rows_keys,
                   int64_t num_batches, const int64_t* unique_ptr,
                   int64_t* out_unique, void* workspace, size_t workspace_bytes,
                   gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  GS_REQUIRE(unique_ptr, "unique_fill: null unique_ptr");
  UniqueWs w = carve_unique(workspace, S, E, B);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("unique workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  const int64_t N = S + E;
  if (N == 0) return GS_OK;
  GS_REQUIRE(out_unique, "unique_fill: null out_unique");
  hipStream_t s = as_stream(stream);
  const int64_t nblocks = ceil_div(N, kBlock);
  GS_LAUNCH("unique_fill", s,
            unique_fill_kernel<<<dim3((unsigned)nblocks), dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.table,
                w.flags, w.block_off, unique_ptr, out_unique, w.seed_rank));
  return GS_OK;
}

int gs_unique_relabel(const int64_t* seeds, const int64_t* seeds_ptr,
                      int64_t num_seeds, const int64_t* rows,
                      const int64_t* rows_ptr, int64_t num_rows_keys,
                      int64_t num_batches, const int64_t* edge_col,
                      int64_t* out_row, int64_t* out_col, void* workspace,
                      size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  GS_REQUIRE(out_col == nullptr || edge_col != nullptr,
             "unique_relabel: out_col needs edge_col");
  UniqueWs w = carve_unique(workspace, S, E, B);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("unique workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  if (E > 0 && (out_row || out_col)) {
    GS_LAUNCH("unique_relabel", s,
              unique_relabel_kernel<<<dim3((unsigned)ceil_div(E, kBlock)),
                                      dim3(kBlock), 0, s>>>(
                  w.flat_ptr, B, seeds, rows, rows_ptr, E, w.table, w.seed_rank,
                  edge_col, out_row, out_col));
  }
  return GS_OK;
}

}  // extern "C"
