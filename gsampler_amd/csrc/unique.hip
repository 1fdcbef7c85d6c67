// unique.hip -- unique in first-occurrence order + relabel, for one batch or a
// whole super-batch in one set of launches.
//
// Keys of batch b are seeds_b ++ rows_b.  All batches are laid out back to
// back in one "flat" key space of N = num_seeds + num_rows_keys positions;
// flat_ptr[b] is where batch b starts.  Batch b owns the open-addressing table
// slots of its own (two per key: load factor <= 1/2, linear probing so that a
// probe run stays inside one 128-byte line most of the time).  A slot is one
// 64-bit word  key << 32 | value  so that insertion with "smallest position
// wins" is a single 64-bit atomicMin on the slot.  Every random table access
// costs a 128-byte line from HBM, so the passes are arranged to touch the table
// as rarely as possible:
//   pass 1  insert   value = position of the key inside its batch (min wins);
//                    a key that loses on arrival can never be a first
//                    occurrence, so each key also leaves a "may be first" bit
//   pass 2  flag     only "may be first" keys look the table up again:
//                    first occurrence <=> slot value == own position;
//                    one ballot bit per key + one count per tile
//   scan of the tile counts, unique_ptr from the flags
//   pass 3  fill     streaming, no table access: first occurrences write
//                    out_unique and their batch-local rank into rank[position]
//   pass 4  relabel  one lookup per edge row gives the first position of its
//                    key, rank[] (a per-batch array that stays in L2) gives the
//                    label; column labels are rank[] of the seed positions
#include "common.h"
#include "hashtable.h"
#include "scan.h"

#include <cstdlib>

namespace gs {

constexpr int kWordsPerBlock = kBlock / kWave;
constexpr int kXcds = 8;  // accelerator dies of an MI355X, each with its own L2

// Table slots per key in percent (GS_TABLE_PERCENT, default below) and whether
// blocks are laid out per die (GS_XCD_REMAP).  Read once.
struct UniqueTuning {
  int64_t percent;
  int remap;
};
static UniqueTuning tuning() {
  static const UniqueTuning t = [] {
    UniqueTuning r{200, 1};
    if (const char* e = getenv("GS_TABLE_PERCENT")) r.percent = atoll(e);
    if (const char* e = getenv("GS_XCD_REMAP")) r.remap = atoi(e);
    if (r.percent < 110) r.percent = 110;
    return r;
  }();
  return t;
}

// Slot range of a batch whose keys occupy flat positions [lo, hi): base and
// capacity grow with the key count at `percent` slots per 100 keys; the + batch
// term absorbs the rounding so that ranges never overlap.
__host__ __device__ inline uint64_t table_base_of(int64_t lo, int64_t batch,
                                                  int64_t percent) {
  return (uint64_t)(lo * percent / 100 + batch);
}
__host__ __device__ inline uint64_t table_cap_of(int64_t n, int64_t percent) {
  return (uint64_t)(n * percent / 100 + 1);
}

// Work-group index -> tile of the flat key space.  Consecutive work-groups go
// to consecutive dies, so die x is given the x-th eighth of the tiles, in
// order: at any moment each die walks one batch (its keys are contiguous in
// the flat space) and that batch's table stays in the die's own L2 instead of
// being pulled into all eight.
__device__ __forceinline__ int64_t tile_of_block(int64_t num_tiles, int remap) {
  if (!remap) return blockIdx.x;
  const int64_t per = (num_tiles + kXcds - 1) / kXcds;
  return (int64_t)(blockIdx.x % kXcds) * per + blockIdx.x / kXcds;
}
static int64_t grid_for_tiles(int64_t num_tiles, int remap) {
  return remap ? ceil_div(num_tiles, kXcds) * kXcds : num_tiles;
}

struct UniqueWs {
  int64_t* flat_ptr;      // [B + 1]
  uint64_t* table;        // [percent/100 * N + B + 2]
  uint64_t* maybe;        // [tiles * kWordsPerBlock]  "may be first" bits
  uint64_t* flags;        // [tiles * kWordsPerBlock]  first-occurrence bits
  int64_t* block_off;     // [tiles + 1]
  int32_t* rank;          // [N] batch-local rank of a first occurrence, else -1
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
  w.table = c.take<uint64_t>((size_t)(N * tuning().percent / 100 + B + 2));
  w.maybe = c.take<uint64_t>((size_t)nblocks * kWordsPerBlock);
  w.flags = c.take<uint64_t>((size_t)nblocks * kWordsPerBlock);
  w.block_off = c.take<int64_t>((size_t)nblocks + 1);
  w.rank = c.take<int32_t>((size_t)(N > 0 ? N : 1));
  w.scan_ws_bytes = scan_workspace_bytes(nblocks + 1);
  w.scan_ws = c.take<char>(w.scan_ws_bytes);
  w.total = c.total();
  return w;
}

// Where a flat position lives: batch, position inside the batch, key.
struct FlatItem {
  int64_t batch, local;
  uint64_t key;
  uint64_t table_base, cap;
};

__device__ __forceinline__ FlatItem locate(
    int64_t p, const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t percent) {
  FlatItem it;
  it.batch = B == 1 ? 0 : segment_of(flat_ptr, B, p);
  const int64_t fb = flat_ptr[it.batch];
  it.local = p - fb;
  const int64_t s_lo = seeds_ptr ? seeds_ptr[it.batch] : 0;
  const int64_t s_hi = seeds_ptr ? seeds_ptr[it.batch + 1] : S;
  const int64_t ns = s_hi - s_lo;
  if (it.local < ns) {
    it.key = (uint64_t)seeds[s_lo + it.local];
  } else {
    const int64_t r_lo = rows_ptr ? rows_ptr[it.batch] : 0;
    it.key = (uint64_t)rows[r_lo + it.local - ns];
  }
  it.table_base = table_base_of(fb, it.batch, percent);
  it.cap = table_cap_of(flat_ptr[it.batch + 1] - fb, percent);
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
    const int64_t* __restrict__ rows_ptr, int64_t N, uint64_t* table,
    uint64_t* __restrict__ maybe, int64_t percent, int remap) {
  const int64_t num_tiles = ceil_div_dev(N, kBlock);
  const int64_t tile = tile_of_block(num_tiles, remap);
  if (tile >= num_tiles) return;  // uniform per work-group
  const int64_t p = tile * kBlock + threadIdx.x;
  bool may_be_first = false;
  if (p < N) {
    const FlatItem it =
        locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, percent);
    may_be_first = table_insert_min(table + it.table_base, it.cap, it.key,
                                    (uint64_t)it.local);
  }
  const uint64_t word = __ballot(may_be_first);
  if (lane_id() == 0) maybe[tile * kWordsPerBlock + threadIdx.x / kWave] = word;
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
    const uint64_t* __restrict__ table, const uint64_t* __restrict__ maybe,
    uint64_t* __restrict__ flags, int64_t* __restrict__ block_count,
    int64_t percent, int remap) {
  __shared__ int wave_count[kWordsPerBlock];
  const int64_t num_tiles = ceil_div_dev(N, kBlock);
  const int64_t tile = tile_of_block(num_tiles, remap);
  if (tile >= num_tiles) return;  // uniform per work-group
  const int64_t p = tile * kBlock + threadIdx.x;
  const int wave = threadIdx.x / kWave;
  bool first = false;
  if (p < N && ((maybe[tile * kWordsPerBlock + wave] >> lane_id()) & 1ull)) {
    const FlatItem it =
        locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, percent);
    const uint64_t* tab = table + it.table_base;
    const uint64_t cur = tab[find_slot(tab, it.cap, it.key)];
    first = (uint32_t)cur == (uint32_t)it.local;
  }
  const uint64_t word = __ballot(first);
  if (lane_id() == 0) {
    flags[tile * kWordsPerBlock + wave] = word;
    wave_count[wave] = __popcll(word);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kWordsPerBlock; ++w) total += wave_count[w];
    block_count[tile] = total;
    if (tile == num_tiles - 1) block_count[num_tiles] = 0;
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

// Streaming: every position writes its rank (or -1); first occurrences also
// write their key to the frontier.
__global__ __launch_bounds__(kBlock) void unique_fill_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ seeds_ptr,
    int64_t S, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t N,
    const uint64_t* __restrict__ flags, const int64_t* __restrict__ block_off,
    const int64_t* __restrict__ unique_ptr, int64_t* __restrict__ out_unique,
    int32_t* __restrict__ rank, int64_t percent) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= N) return;
  int32_t r = -1;
  if ((flags[p / kWave] >> (p % kWave)) & 1ull) {
    const FlatItem it =
        locate(p, flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, percent);
    const int64_t grank = rank_before(p, flags, block_off);
    out_unique[grank] = (int64_t)it.key;
    r = (int32_t)(grank - unique_ptr[it.batch]);
  }
  rank[p] = r;
}

__global__ __launch_bounds__(kBlock) void unique_relabel_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ rows,
    const int64_t* __restrict__ rows_ptr, int64_t E,
    const uint64_t* __restrict__ table, const int32_t* __restrict__ rank,
    const int64_t* __restrict__ edge_col, int64_t* __restrict__ out_row,
    int64_t* __restrict__ out_col, int64_t percent, int remap) {
  const int64_t tile = tile_of_block(ceil_div_dev(E, kBlock), remap);
  const int64_t e = tile * kBlock + threadIdx.x;
  if (e >= E) return;
  const int64_t b = (B == 1 || rows_ptr == nullptr) ? 0 : segment_of(rows_ptr, B, e);
  const int64_t fb = flat_ptr[b];
  const uint64_t* tab = table + table_base_of(fb, b, percent);
  const uint64_t cap = table_cap_of(flat_ptr[b + 1] - fb, percent);
  // first position of a key inside the batch -> its rank
  auto label_of = [&](uint64_t key) -> int64_t {
    const uint32_t first_local = (uint32_t)tab[find_slot(tab, cap, key)];
    return (int64_t)rank[fb + first_local];
  };
  if (out_row) out_row[e] = label_of((uint64_t)rows[e]);
  if (out_col) {
    // seed c of batch b sits at flat position c + rows_ptr[b]
    const int64_t c = edge_col[e];
    int64_t r = rank[c + (rows_ptr ? rows_ptr[b] : 0)];
    if (r < 0) r = label_of((uint64_t)seeds[c]);  // a repeated seed
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
  const UniqueTuning tn = tuning();
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
    const int64_t slots = N * tuning().percent / 100 + B + 2;
    int64_t blocks = ceil_div(slots, kBlock * 8);
    GS_LAUNCH("unique_clear", s,
              table_fill_kernel<><<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(
                  w.table, slots, kEmptySlot));
  }
  GS_LAUNCH("unique_insert", s,
            unique_insert_kernel<<<dim3((unsigned)grid_for_tiles(nblocks, tn.remap)),
                                   dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.table,
                w.maybe, tn.percent, tn.remap));
  GS_LAUNCH("unique_flag", s,
            unique_flag_kernel<<<dim3((unsigned)grid_for_tiles(nblocks, tn.remap)),
                                 dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.table,
                w.maybe, w.flags, w.block_off, tn.percent, tn.remap));
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
  const UniqueTuning tn = tuning();
  const int64_t nblocks = ceil_div(N, kBlock);
  GS_LAUNCH("unique_fill", s,
            unique_fill_kernel<<<dim3((unsigned)nblocks), dim3(kBlock), 0, s>>>(
                w.flat_ptr, B, seeds, seeds_ptr, S, rows, rows_ptr, N, w.flags,
                w.block_off, unique_ptr, out_unique, w.rank, tn.percent));
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
  const UniqueTuning tn = tuning();
  if (E > 0 && (out_row || out_col)) {
    GS_LAUNCH("unique_relabel", s,
              unique_relabel_kernel<<<dim3((unsigned)grid_for_tiles(ceil_div(E, kBlock), tn.remap)),
                                      dim3(kBlock), 0, s>>>(
                  w.flat_ptr, B, seeds, rows, rows_ptr, E, w.table, w.rank,
                  edge_col, out_row, out_col, tn.percent, tn.remap));
  }
  return GS_OK;
}

}  // extern "C"
