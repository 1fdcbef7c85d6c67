// unique.hip -- unique in first-occurrence order + relabel, for one batch or a
// whole super-batch in one set of launches.
//
// Keys of batch b are seeds_b ++ rows_b.  All batches are laid out back to
// back in one "flat" key space of N = num_seeds + num_rows_keys positions;
// flat_ptr[b] is where batch b starts.
//
// A hash table over all keys of a batch does not fit in a die's L2, and every
// random access to it costs a whole line from HBM.  So the keys of a batch are
// first partitioned by hash into buckets of about 1500 entries (streaming
// reads and writes only), and each bucket is then deduplicated by one
// work-group in an LDS table:
//   plan     per-batch record (where its keys, tiles, buckets and bucket regions
//            start), the batch of every tile, bucket, group of positions and
//            tile of edges (so that a work-group finds its work with two
//            dependent loads instead of a binary search); zero the counters
//   scatter  per tile: order the tile by bucket in LDS, reserve a run in every
//            bucket with one atomic on the bucket's cursor, write
//            key << 32 | local.  A bucket owns a region of fixed capacity (as
//            many entries as the batch has keys, at most kBucketCap, five times
//            the average bucket), so where a run goes is known without
//            counting the keys per bucket first: the keys are read once here,
//            not twice.  What does not fit a region (a key that repeats more
//            than kBucketCap times in one batch) goes to the batch's overflow
//            list together with its bucket
//   dedup    per bucket: LDS table with "smallest position wins" (64-bit
//            atomicMin on the packed entry), then every entry writes the first
//            position of its key into first[position]
//   flag     streaming, one work-group per group of 4096 positions: position is
//            a first occurrence <=> first[p] == local(p); per 64 positions one
//            rank word (the ballot + the first occurrences of the group before
//            it), per group one count
//   offsets  one work-group: group counts -> group offsets; unique_ptr
//   fill     streaming: first occurrences write out_unique
//   relabel  label of a position = rank of its first occurrence = group offset
//            + rank word of that position: two gathers in tables of N/4 bytes
//            (80 KB per batch of 330 K keys), which a die's L2 holds
// The result does not depend on the order in which entries land in a bucket, so
// the atomics above leave it deterministic.  A bucket with more entries than the
// LDS table is sure to hold (a hub that repeats thousands of times, a batch too
// large for kMaxBuckets buckets) is deduplicated by the same work-group in a
// table in global memory that is private to the bucket; a bucket whose region
// ran over first collects its entries from the batch's overflow list.
//
// A packed entry is  low 32 bits of the key << 32 | position.  While every key
// of a call is below 2^32 - 1 those bits are the key.  The partition pass notes
// when one is not (an id of a very large graph, an id encoded as
// id + batch * num_rows): the upper half is then only a fingerprint, and the
// dedup pass confirms every fingerprint match by comparing the two keys
// themselves, read back through their positions.
#include "common.h"
#include "hashtable.h"
#include "scan.h"

namespace gs {

constexpr int kXcds = 8;  // accelerator dies of an MI355X, each with its own L2

constexpr int kPartItems = 16;                    // keys per thread and tile
constexpr int kPartTile = kBlock * kPartItems;    // keys per partition tile
constexpr int kMaxBuckets = 2048;                 // buckets per batch (LDS bins)
constexpr int kLdsSlots = 4096;                   // dedup table, 32 KB of LDS
constexpr int kLdsMaxEntries = kLdsSlots * 3 / 4; // bucket sizes the LDS table takes
constexpr int64_t kBucketCap = 8192;              // entries a bucket's region holds at most
static_assert(kBucketCap >= kLdsMaxEntries, "the short dedup path reads a bucket from its region alone");

// Average entries per bucket and whether work-groups are laid out per die: the
// best of a sweep on 21M keys in 64 batches (bucket sizes 512..3072, with and
// without the per-die layout).
struct UniqueTuning {
  int64_t bucket_keys;
  int remap;
};
static UniqueTuning tuning() { return UniqueTuning{1536, 1}; }

// Work-group index -> unit of work (tile or bucket).  Consecutive work-groups
// go to consecutive dies, so die x is given the x-th eighth of the units, in
// order: at any moment each die walks one batch, and what that batch touches
// (its open bucket lines, its first[] and rank[] ranges) stays in the die's own
// L2 instead of being pulled into all eight.
__device__ __forceinline__ int64_t unit_of_block(int64_t num_units, int remap) {
  if (!remap) return blockIdx.x;
  const int64_t per = (num_units + kXcds - 1) / kXcds;
  return (int64_t)(blockIdx.x % kXcds) * per + blockIdx.x / kXcds;
}
static int64_t grid_for_units(int64_t num_units, int remap) {
  return remap ? ceil_div(num_units, kXcds) * kXcds : num_units;
}

// What a work-group needs to know about a batch, in one aligned record.
struct alignas(16) BatchInfo {
  int64_t fb;        // first flat position
  int64_t n;         // keys (seeds + rows)
  int64_t s_lo, ns;  // its seeds: seeds[s_lo .. s_lo + ns)
  int64_t r_lo;      // its rows start at rows[r_lo]
  int64_t tile0;     // first partition tile
  int64_t bucket0;   // first bucket
  int64_t buckets;   // number of buckets
  int64_t region0;   // first entry of its first bucket's region
  int64_t cap;       // entries per bucket region: min(n, kBucketCap)
};

constexpr int kRelabelItems = 4;
constexpr int kRelabelTile = kBlock * kRelabelItems;

// First occurrences are counted per group of kGroup consecutive flat positions
// (one work-group of the flag pass).  A rank word covers 64 positions: which of
// them are first occurrences, and how many first occurrences the group has
// before the word.
constexpr int kGroupWords = 64;
constexpr int kGroup = kGroupWords * kWave;
constexpr int kWordsPerWave = kGroupWords / (kBlock / kWave);
struct alignas(16) RankWord {
  uint64_t bits;
  uint32_t before;
  uint32_t unused;
};

struct UniqueWs {
  BatchInfo* batch;       // [B]
  int64_t* flat_ptr;      // [B + 1] first flat position of a batch
  int64_t* tile_ptr;      // [B + 1] first partition tile of a batch
  int64_t* bucket_ptr;    // [B + 1] first bucket of a batch
  int64_t* region_ptr;    // [B + 1] first region entry of a batch
  int32_t* tile_batch;    // [max_tiles] batch of a tile, -1 past the last one
  int32_t* bucket_batch;  // [max_buckets] batch of a bucket, -1 past the last one
  int64_t* bucket_base;   // [max_buckets] first entry of a bucket's region
  int32_t* bucket_cap;    // [max_buckets] capacity of a bucket's region
  int32_t* group_batch;   // [groups + 1] batch of the first position of a group
  int32_t* etile_batch;   // [edge tiles + 1] batch of the first edge of a tile
  int64_t* bucket_cur;    // [max_buckets + 1] entries sent to a bucket
  int64_t* ovf_cur;       // [B + 1] entries on a batch's overflow list
  unsigned long long* pool_cur;  // [1] entries handed out from the spill pool
  int* wide_keys;         // [1] set when some key does not fit the upper half of an entry
  uint64_t* packed;       // [region_entries] key << 32 | local, one region per bucket
  uint64_t* ovf_entry;    // [N] entries that found their region full, per batch at flat_ptr[b]
  int32_t* ovf_bucket;    // [N] and their buckets
  uint32_t* first;        // [N] local position of the first occurrence
  uint64_t* spill;        // [3 N + max_buckets + 1] pool: tables of oversize buckets, collected overflow
  RankWord* words;        // [groups * kGroupWords]
  int64_t* group_cnt;     // [groups] first occurrences per group
  int64_t* group_off;     // [groups + 1] first occurrences before a group
  int64_t* unique_ptr;    // [B + 1] copy of the caller's unique_ptr for the relabel pass
  int64_t max_tiles, max_buckets, groups, etiles, region_entries, pool_entries;
  size_t total;
};

static UniqueWs carve_unique(void* ws, int64_t S, int64_t E, int64_t B) {
  const int64_t N = S + E;
  const int64_t n1 = N > 0 ? N : 1;
  Carver c(ws);
  UniqueWs w;
  // sum over batches of ceil(n_b / x) <= N / x + B
  w.max_tiles = N / kPartTile + B;
  w.max_buckets = N / tuning().bucket_keys + B;
  w.groups = ceil_div(n1, kGroup);
  w.etiles = ceil_div(E > 0 ? E : 1, kRelabelTile);
  // A batch of n keys has ceil(n / bucket_keys) regions of min(n, kBucketCap)
  // entries: at most n (kBucketCap / bucket_keys + 1) entries when n <= kBucketCap,
  // at most n kBucketCap / bucket_keys + kBucketCap otherwise, and there are at
  // most N / kBucketCap batches of the second kind.
  w.region_entries = n1 * (kBucketCap / tuning().bucket_keys + 2) + kBucketCap;
  w.pool_entries = 3 * n1 + w.max_buckets + 1;
  w.batch = c.take<BatchInfo>((size_t)B);
  w.flat_ptr = c.take<int64_t>((size_t)B + 1);
  w.tile_ptr = c.take<int64_t>((size_t)B + 1);
  w.bucket_ptr = c.take<int64_t>((size_t)B + 1);
  w.region_ptr = c.take<int64_t>((size_t)B + 1);
  w.tile_batch = c.take<int32_t>((size_t)w.max_tiles);
  w.bucket_batch = c.take<int32_t>((size_t)w.max_buckets);
  w.bucket_base = c.take<int64_t>((size_t)w.max_buckets);
  w.bucket_cap = c.take<int32_t>((size_t)w.max_buckets);
  w.group_batch = c.take<int32_t>((size_t)w.groups + 1);
  w.etile_batch = c.take<int32_t>((size_t)w.etiles + 1);
  w.bucket_cur = c.take<int64_t>((size_t)w.max_buckets + 1);
  w.ovf_cur = c.take<int64_t>((size_t)B + 1);
  w.pool_cur = c.take<unsigned long long>(1);
  w.wide_keys = c.take<int>(1);
  w.packed = c.take<uint64_t>((size_t)w.region_entries);
  w.ovf_entry = c.take<uint64_t>((size_t)n1);
  w.ovf_bucket = c.take<int32_t>((size_t)n1);
  w.first = c.take<uint32_t>((size_t)n1);
  w.spill = c.take<uint64_t>((size_t)w.pool_entries);
  w.words = c.take<RankWord>((size_t)w.groups * kGroupWords);
  w.group_cnt = c.take<int64_t>((size_t)w.groups);
  w.group_off = c.take<int64_t>((size_t)w.groups + 1);
  w.unique_ptr = c.take<int64_t>((size_t)B + 1);
  w.total = c.total();
  return w;
}

// The caller's view of the keys.
struct Keys {
  const int64_t* seeds;
  const int64_t* seeds_ptr;  // null: one batch
  int64_t S;
  const int64_t* rows;
  const int64_t* rows_ptr;   // null: one batch
  int64_t E;
  int64_t B;
};

__device__ __forceinline__ int64_t seeds_lo(const Keys& k, int64_t b) {
  return k.seeds_ptr ? k.seeds_ptr[b] : (b == 0 ? 0 : k.S);
}
__device__ __forceinline__ int64_t rows_lo(const Keys& k, int64_t b) {
  return k.rows_ptr ? k.rows_ptr[b] : (b == 0 ? 0 : k.E);
}

// Key at position `local` of batch b (whose seeds are [s_lo, s_lo + ns)).
__device__ __forceinline__ uint64_t key_at(const Keys& k, int64_t s_lo,
                                           int64_t ns, int64_t r_lo,
                                           int64_t local) {
  return (uint64_t)(local < ns ? k.seeds[s_lo + local] : k.rows[r_lo + local - ns]);
}

// Bucket of a key among the `buckets` of its batch: the high bits of the hash.
__device__ __forceinline__ uint32_t bucket_of(uint64_t key, uint32_t buckets) {
  return (uint32_t)(((uint64_t)hash32(key) * buckets) >> 32);
}
// Home slot inside a bucket's table: bits the bucket choice did not use.
__device__ __forceinline__ uint32_t slot_hash(uint64_t key) {
  return (uint32_t)((key * 0xC2B2AE3D27D4EB4Full) >> 29);
}

// ---------------------------------------------------------------- plan
// The walk over the batches: where the keys, tiles and buckets of every batch
// start.  Run by one whole work-group; the three offset arrays may live in LDS
// or in global memory, `batch` (the records) may be null.
__device__ __forceinline__ void walk_batches(const Keys& k, int64_t bucket_keys,
                                             BatchInfo* batch, int64_t* flat_ptr,
                                             int64_t* tile_ptr, int64_t* bucket_ptr,
                                             int64_t* region_ptr, int64_t* smem) {
  int64_t tile_carry = 0, bucket_carry = 0, region_carry = 0;
  for (int64_t base = 0; base <= k.B; base += kBlock) {
    const int64_t b = base + threadIdx.x;
    BatchInfo info{};
    int64_t tiles = 0;
    if (b <= k.B) {
      info.s_lo = seeds_lo(k, b);
      info.r_lo = rows_lo(k, b);
      info.fb = info.s_lo + info.r_lo;
      flat_ptr[b] = info.fb;
      if (b < k.B) {
        info.ns = seeds_lo(k, b + 1) - info.s_lo;
        info.n = info.ns + rows_lo(k, b + 1) - info.r_lo;
        tiles = ceil_div_dev(info.n, kPartTile);
        info.buckets = ceil_div_dev(info.n, bucket_keys);
        if (info.buckets > kMaxBuckets) info.buckets = kMaxBuckets;
        info.cap = info.n < kBucketCap ? info.n : kBucketCap;
      }
    }
    int64_t total;
    info.tile0 = tile_carry + block_exclusive_sum(tiles, smem, &total);
    tile_carry += total;
    __syncthreads();
    info.bucket0 = bucket_carry + block_exclusive_sum(info.buckets, smem, &total);
    bucket_carry += total;
    __syncthreads();
    info.region0 = region_carry + block_exclusive_sum(info.buckets * info.cap, smem, &total);
    region_carry += total;
    __syncthreads();
    if (b <= k.B) {
      tile_ptr[b] = info.tile0;
      bucket_ptr[b] = info.bucket0;
      region_ptr[b] = info.region0;
    }
    if (batch && b < k.B) batch[b] = info;
  }
}

// Unit i of the list (tiles, buckets, groups of positions, tiles of edges):
// which batch it belongs to.  One search per unit here instead of one at the
// start of every work-group later.
struct UnitTables {
  int64_t max_tiles, max_buckets, groups, etiles;
  int32_t *tile_batch, *bucket_batch, *group_batch, *etile_batch;
  int64_t* bucket_base;
  int32_t* bucket_cap;
  __host__ __device__ int64_t units() const {
    return max_tiles + max_buckets + groups + 1 + etiles + 1;
  }
};
__device__ __forceinline__ void assign_unit(int64_t i, const Keys& k, int64_t N,
                                            const int64_t* flat_ptr,
                                            const int64_t* tile_ptr,
                                            const int64_t* bucket_ptr,
                                            const int64_t* region_ptr,
                                            const UnitTables& u) {
  const int64_t B = k.B;
  if (i < u.max_tiles) {
    u.tile_batch[i] = i < tile_ptr[B] ? (int32_t)segment_of(tile_ptr, B, i) : -1;
    return;
  }
  i -= u.max_tiles;
  if (i < u.max_buckets) {
    int32_t b = -1;
    int64_t base = 0, cap = 0;
    if (i < bucket_ptr[B]) {
      b = (int32_t)segment_of(bucket_ptr, B, i);
      const int64_t n = flat_ptr[b + 1] - flat_ptr[b];
      cap = n < kBucketCap ? n : kBucketCap;
      base = region_ptr[b] + (i - bucket_ptr[b]) * cap;
    }
    u.bucket_batch[i] = b;
    u.bucket_base[i] = base;
    u.bucket_cap[i] = (int32_t)cap;
    return;
  }
  i -= u.max_buckets;
  if (i <= u.groups) {
    int64_t p = i * kGroup;
    if (p > N - 1) p = N - 1;
    u.group_batch[i] = (int32_t)segment_of(flat_ptr, B, p);
    return;
  }
  i -= u.groups + 1;
  if (i <= u.etiles) {
    int64_t e = i * kRelabelTile;
    if (e > k.E - 1) e = k.E - 1;
    u.etile_batch[i] =
        (k.rows_ptr && k.E > 0) ? (int32_t)segment_of(k.rows_ptr, B, e) : 0;
  }
}

__device__ __forceinline__ void zero_counters(int64_t* bucket_cur, int64_t max_buckets,
                                              int64_t* ovf_cur, int64_t num_batches,
                                              unsigned long long* pool_cur, int* wide_keys) {
  const int64_t i0 = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = i0; i <= max_buckets; i += stride) bucket_cur[i] = 0;
  for (int64_t i = i0; i <= num_batches; i += stride) ovf_cur[i] = 0;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *wide_keys = 0;
    *pool_cur = 0ull;
  }
}

// Up to kPlanMaxBatches batches: every work-group walks the batches into LDS
// (a few block scans) and then assigns its units from there; work-group 0 also
// leaves the records and offset arrays in global memory.
constexpr int kPlanMaxBatches = 1024;
__global__ __launch_bounds__(kBlock) void unique_plan_kernel(
    Keys k, int64_t N, int64_t bucket_keys, BatchInfo* __restrict__ batch,
    int64_t* __restrict__ flat_ptr, int64_t* __restrict__ tile_ptr,
    int64_t* __restrict__ bucket_ptr, int64_t* __restrict__ region_ptr,
    int64_t* __restrict__ bucket_cur, int64_t* __restrict__ ovf_cur,
    unsigned long long* __restrict__ pool_cur, int* __restrict__ wide_keys, UnitTables u) {
  __shared__ int64_t l_flat[kPlanMaxBatches + 1];
  __shared__ int64_t l_tile[kPlanMaxBatches + 1];
  __shared__ int64_t l_bucket[kPlanMaxBatches + 1];
  __shared__ int64_t l_region[kPlanMaxBatches + 1];
  __shared__ int64_t smem[kBlock / kWave + 1];
  zero_counters(bucket_cur, u.max_buckets, ovf_cur, k.B, pool_cur, wide_keys);
  walk_batches(k, bucket_keys, blockIdx.x == 0 ? batch : nullptr, l_flat, l_tile,
               l_bucket, l_region, smem);
  __syncthreads();
  if (blockIdx.x == 0)
    for (int64_t b = threadIdx.x; b <= k.B; b += kBlock) {
      flat_ptr[b] = l_flat[b];
      tile_ptr[b] = l_tile[b];
      bucket_ptr[b] = l_bucket[b];
      region_ptr[b] = l_region[b];
    }
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < u.units()) assign_unit(i, k, N, l_flat, l_tile, l_bucket, l_region, u);
}

// More batches than that: the walk by one work-group into global memory ...
__global__ __launch_bounds__(kBlock) void unique_prep_kernel(
    Keys k, int64_t bucket_keys, BatchInfo* __restrict__ batch,
    int64_t* __restrict__ flat_ptr, int64_t* __restrict__ tile_ptr,
    int64_t* __restrict__ bucket_ptr, int64_t* __restrict__ region_ptr,
    int64_t* __restrict__ bucket_cur, int64_t max_buckets, int64_t* __restrict__ ovf_cur,
    unsigned long long* __restrict__ pool_cur, int* __restrict__ wide_keys) {
  __shared__ int64_t smem[kBlock / kWave + 1];
  zero_counters(bucket_cur, max_buckets, ovf_cur, k.B, pool_cur, wide_keys);
  if (blockIdx.x != 0) return;
  walk_batches(k, bucket_keys, batch, flat_ptr, tile_ptr, bucket_ptr, region_ptr, smem);
}

// ... and the units from there in a launch of their own.
__global__ __launch_bounds__(kBlock) void unique_units_kernel(
    Keys k, int64_t N, const int64_t* __restrict__ flat_ptr,
    const int64_t* __restrict__ tile_ptr, const int64_t* __restrict__ bucket_ptr,
    const int64_t* __restrict__ region_ptr, UnitTables u) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < u.units()) assign_unit(i, k, N, flat_ptr, tile_ptr, bucket_ptr, region_ptr, u);
}

// One partition tile: which batch, which keys.
struct TileInfo {
  BatchInfo b;
  int64_t begin, end;  // local positions [begin, end)
};

__device__ __forceinline__ bool tile_info(int64_t tile,
                                          const int32_t* __restrict__ tile_batch,
                                          const BatchInfo* __restrict__ batch,
                                          TileInfo* t) {
  const int32_t b = tile_batch[tile];
  if (b < 0) return false;
  t->b = batch[b];
  t->begin = (tile - t->b.tile0) * kPartTile;
  t->end = t->begin + kPartTile < t->b.n ? t->begin + kPartTile : t->b.n;
  return true;
}

__device__ __forceinline__ uint64_t key_at(const Keys& k, const BatchInfo& b,
                                           int64_t local) {
  return key_at(k, b.s_lo, b.ns, b.r_lo, local);
}

// Upper half of a packed entry: the low 32 bits of the key, kept clear of the
// pattern of the empty slot (for keys below 2^32 - 1 this is the key itself).
__device__ __forceinline__ uint32_t key_tag(uint64_t key) {
  const uint32_t t = (uint32_t)key;
  return t == 0xFFFFFFFFu ? 0xFFFFFFFEu : t;
}

// ---------------------------------------------------------------- scatter
// Bucket j of a batch owns entries [region0 + j cap, region0 + (j + 1) cap) of
// `packed`.  A tile that brings c entries to a bucket takes the next c places at
// the bucket's cursor; places past the region's capacity are on the batch's
// overflow list instead (the cursor still counts them, which is how the dedup
// pass knows).  The tile is first ordered by bucket in LDS so that every run
// leaves as one contiguous write instead of one line per entry.
// 48 KB of LDS per work-group lets three share a compute unit: with 512 threads
// each they fill three quarters of its wavefront slots (256 threads: 11 % slower
// on 21 M keys; 1024, two work-groups per unit: 45 % slower).
constexpr int kScatterThreads = 512;
constexpr int kScatterItems = kPartTile / kScatterThreads;
__global__ __launch_bounds__(kScatterThreads) void unique_scatter_kernel(
    Keys k, const int32_t* __restrict__ tile_batch,
    const BatchInfo* __restrict__ batch, int64_t* bucket_cur, int64_t* ovf_cur,
    uint64_t* __restrict__ packed, uint64_t* __restrict__ ovf_entry,
    int32_t* __restrict__ ovf_bucket, uint32_t* __restrict__ first, int64_t max_tiles,
    int remap, int* wide_keys) {
  __shared__ uint32_t hist[kMaxBuckets];   // counts, then offsets inside the tile
  __shared__ uint32_t run_at[kMaxBuckets]; // where the tile's run starts in the bucket
  __shared__ uint64_t stage[kPartTile];
  __shared__ uint32_t scan_smem[kScatterThreads / kWave + 1];
  const int64_t tile = unit_of_block(max_tiles, remap);
  if (tile >= max_tiles) return;
  TileInfo t;
  if (!tile_info(tile, tile_batch, batch, &t)) return;  // uniform per work-group
  const uint32_t buckets = (uint32_t)t.b.buckets;
  uint64_t* out = packed + t.b.region0;
  if (buckets == 1) {  // the bucket is the batch, in order
    if (tile == t.b.tile0 && threadIdx.x == 0) bucket_cur[t.b.bucket0] = t.b.n;
    bool wide = false;
    for (int64_t l = t.begin + threadIdx.x; l < t.end; l += kScatterThreads) {
      const uint64_t full = key_at(k, t.b, l);
      wide |= full > kMaxPackedKey;  // negative ids land here too
      out[l] = ((uint64_t)key_tag(full) << 32) | (uint64_t)l;
      first[t.b.fb + l] = (uint32_t)l;
    }
    if (wide) *wide_keys = 1;  // every writer stores the same value
    return;
  }
  uint64_t full[kScatterItems];
  uint32_t key[kScatterItems], place[kScatterItems];
#pragma unroll
  for (int i = 0; i < kScatterItems; ++i) {
    // All loads in flight before anything else: a position past the end reads
    // the tile's last key instead of branching around the load (the compiler
    // otherwise moves the first use of the key into that branch and waits
    // there, one load at a time).
    const int64_t l = t.begin + i * kScatterThreads + threadIdx.x;
    full[i] = key_at(k, t.b, l < t.end ? l : t.end - 1);
  }
  constexpr int kBins = kMaxBuckets / kScatterThreads;
#pragma unroll
  for (int r = 0; r < kBins; ++r) {
    const uint32_t bin = threadIdx.x + r * kScatterThreads;
    if (bin < buckets) hist[bin] = 0;
  }
  __syncthreads();
  bool wide = false;
#pragma unroll
  for (int i = 0; i < kScatterItems; ++i) {
    const int64_t l = t.begin + i * kScatterThreads + threadIdx.x;
    wide |= full[i] > kMaxPackedKey;
    key[i] = key_tag(full[i]);
    // every position starts as its own first occurrence; the dedup pass only
    // writes the positions that are not (half as many scattered stores)
    if (l < t.end) first[t.b.fb + l] = (uint32_t)l;
  }
  if (wide) *wide_keys = 1;
#pragma unroll
  for (int i = 0; i < kScatterItems; ++i)
    if (t.begin + i * kScatterThreads + threadIdx.x < t.end)
      place[i] = atomicAdd(&hist[bucket_of(key[i], buckets)], 1u);
  __syncthreads();
  const uint32_t count = (uint32_t)(t.end - t.begin);
  {
    const uint32_t bin0 = threadIdx.x * kBins;
    uint32_t c[kBins], sum = 0;
#pragma unroll
    for (int j = 0; j < kBins; ++j) {
      c[j] = bin0 + j < buckets ? hist[bin0 + j] : 0u;
      sum += c[j];
    }
    uint32_t total;
    uint32_t run = block_exclusive_sum<uint32_t, kScatterThreads>(sum, scan_smem, &total);
#pragma unroll
    for (int j = 0; j < kBins; ++j) {
      if (bin0 + j < buckets) hist[bin0 + j] = run;
      run += c[j];
    }
  }
  __syncthreads();
  // One bin per thread and round; all reservations are sent off before the tile
  // is ordered in LDS, and their answers (a trip to the L2 and back) are only
  // looked at after that.
  const uint32_t cap = (uint32_t)t.b.cap;
  uint32_t taken[kBins], mine[kBins];
#pragma unroll
  for (int r = 0; r < kBins; ++r) {
    const uint32_t bin = threadIdx.x + r * kScatterThreads;
    taken[r] = mine[r] = 0;
    if (bin < buckets) {
      mine[r] = (bin + 1 < buckets ? hist[bin + 1] : count) - hist[bin];
      if (mine[r])
        taken[r] = (uint32_t)atomicAdd((unsigned long long*)&bucket_cur[t.b.bucket0 + bin],
                                       (unsigned long long)mine[r]);
    }
  }
#pragma unroll
  for (int i = 0; i < kScatterItems; ++i) {
    const int64_t l = t.begin + i * kScatterThreads + threadIdx.x;
    if (l < t.end)
      stage[hist[bucket_of(key[i], buckets)] + place[i]] =
          ((uint64_t)key[i] << 32) | (uint64_t)l;
  }
#pragma unroll
  for (int r = 0; r < kBins; ++r) {
    const uint32_t bin = threadIdx.x + r * kScatterThreads;
    if (bin < buckets) run_at[bin] = taken[r];
  }
  __syncthreads();
  for (uint32_t j = threadIdx.x; j < count; j += kScatterThreads) {
    const uint64_t e = stage[j];
    const uint32_t bk = bucket_of(e >> 32, buckets);
    const uint32_t at = run_at[bk] + (j - hist[bk]);
    if (at < cap) out[(uint64_t)bk * cap + at] = e;
  }
  // The part of a run that found the region full: the thread that reserved the
  // run moves it to the batch's overflow list.
#pragma unroll
  for (int r = 0; r < kBins; ++r) {
    if (taken[r] + mine[r] <= cap) continue;
    const uint32_t bin = threadIdx.x + r * kScatterThreads;
    const uint32_t fits = taken[r] < cap ? cap - taken[r] : 0u;
    const uint32_t over = mine[r] - fits;
    const int64_t at = t.b.fb + (int64_t)atomicAdd((unsigned long long*)&ovf_cur[tile_batch[tile]],
                                                   (unsigned long long)over);
    for (uint32_t i = 0; i < over; ++i) {
      ovf_entry[at + i] = stage[hist[bin] + fits + i];
      ovf_bucket[at + i] = (int32_t)bin;
    }
  }
}

// ---------------------------------------------------------------- dedup
// Whether two entries with the same upper half stand for the same key: always
// when every key of the call fits that half; otherwise the keys themselves are
// read back through the entries' positions and compared.
template <bool kWide>
struct SameKey {
  const Keys* k;
  const BatchInfo* b;
  __device__ __forceinline__ bool operator()(uint64_t a, uint64_t c) const {
    if (!kWide) return true;
    return key_at(*k, *b, (int64_t)(uint32_t)a) == key_at(*k, *b, (int64_t)(uint32_t)c);
  }
};

template <typename Same>
__device__ __forceinline__ void lds_insert_min(uint64_t* tab, uint32_t mask,
                                               uint64_t entry, const Same& same) {
  const uint64_t tag = entry >> 32;
  uint32_t slot = slot_hash(tag) & mask;
  for (;;) {
    uint64_t cur = tab[slot];
    if (cur == kEmptySlot) {
      cur = atomicCAS((unsigned long long*)&tab[slot],
                      (unsigned long long)kEmptySlot, (unsigned long long)entry);
      if (cur == kEmptySlot) return;
    }
    // a slot only ever holds positions of one key, so a stale read is as good
    if ((cur >> 32) == tag && same(cur, entry)) {
      if (cur > entry)
        atomicMin((unsigned long long*)&tab[slot], (unsigned long long)entry);
      return;
    }
    slot = (slot + 1) & mask;
  }
}

template <typename Same>
__device__ __forceinline__ uint32_t lds_first_of(const uint64_t* tab,
                                                 uint32_t mask, uint64_t entry,
                                                 const Same& same) {
  const uint64_t tag = entry >> 32;
  uint32_t slot = slot_hash(tag) & mask;
  for (;;) {
    const uint64_t cur = tab[slot];
    // (an empty slot is never met: every entry looked up was inserted, and no
    // tag equals the upper half of the empty pattern)
    if ((cur >> 32) == tag && same(cur, entry)) return (uint32_t)cur;
    slot = (slot + 1) & mask;
  }
}

// Table in global memory, used by one work-group inside one kernel: loads must
// not be served from the compute unit's own cache.
__device__ __forceinline__ uint64_t load_l2(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename Same>
__device__ __forceinline__ void spill_insert_min(uint64_t* tab, uint64_t cap,
                                                 uint64_t entry, const Same& same) {
  const uint64_t tag = entry >> 32;
  uint64_t slot = ((uint64_t)slot_hash(tag) * cap) >> 32;
  for (uint64_t probes = 0; probes < cap; ++probes) {
    uint64_t cur = load_l2(tab + slot);
    if (cur == kEmptySlot) {
      cur = atomicCAS((unsigned long long*)(tab + slot),
                      (unsigned long long)kEmptySlot, (unsigned long long)entry);
      if (cur == kEmptySlot) return;
    }
    if ((cur >> 32) == tag && same(cur, entry)) {
      if (cur > entry)
        atomicMin((unsigned long long*)(tab + slot), (unsigned long long)entry);
      return;
    }
    if (++slot == cap) slot = 0;
  }
}

template <typename Same>
__device__ __forceinline__ uint32_t spill_first_of(const uint64_t* tab,
                                                   uint64_t cap, uint64_t entry,
                                                   const Same& same) {
  const uint64_t tag = entry >> 32;
  uint64_t slot = ((uint64_t)slot_hash(tag) * cap) >> 32;
  for (uint64_t probes = 0; probes < cap; ++probes) {
    const uint64_t cur = load_l2(tab + slot);
    if (cur == kEmptySlot) break;
    if ((cur >> 32) == tag && same(cur, entry)) return (uint32_t)cur;
    if (++slot == cap) slot = 0;
  }
  return (uint32_t)entry;  // not reached: every entry looked up was inserted
}

// Same as lds_insert_min for a bucket that may hold more distinct keys than the
// table takes: counts the slots it claims and raises *overflow instead of
// filling the table up.
template <typename Same>
__device__ __forceinline__ void lds_insert_min_counted(uint64_t* tab,
                                                       uint32_t mask,
                                                       uint64_t entry,
                                                       const Same& same,
                                                       uint32_t* distinct,
                                                       volatile uint32_t* overflow) {
  const uint64_t tag = entry >> 32;
  uint32_t slot = slot_hash(tag) & mask;
  for (;;) {
    uint64_t cur = tab[slot];
    if (cur == kEmptySlot) {
      cur = atomicCAS((unsigned long long*)&tab[slot],
                      (unsigned long long)kEmptySlot, (unsigned long long)entry);
      if (cur == kEmptySlot) {
        if (atomicAdd(distinct, 1u) >= (uint32_t)kLdsMaxEntries) *overflow = 1u;
        return;
      }
    }
    if ((cur >> 32) == tag && same(cur, entry)) {
      if (cur > entry)
        atomicMin((unsigned long long*)&tab[slot], (unsigned long long)entry);
      return;
    }
    slot = (slot + 1) & mask;
  }
}

// The entries of a bucket: the first `fit` in its region, the rest (what the
// region had no room for) in a run of the spill pool.
struct BucketEntries {
  const uint64_t* region;
  const uint64_t* extra;
  int64_t fit;
  // (one load either way, so that a thread's loads of a round go out together;
  // the run of the pool was written by this work-group a moment ago and is
  // read past the compute unit's own cache)
  __device__ __forceinline__ uint64_t operator[](int64_t i) const {
    return load_l2(i < fit ? region + i : extra + (i - fit));
  }
};

template <int kThreads, bool kWide>
__device__ __forceinline__ void dedup_bucket(
    const Keys& k, const BatchInfo& info, int64_t n, const BucketEntries& entries,
    uint64_t* spill, unsigned long long* pool_cur, uint32_t* __restrict__ first,
    uint64_t* tab, uint32_t* distinct_ptr, uint32_t* overflow_ptr,
    unsigned long long* pool_at) {
  uint32_t& distinct = *distinct_ptr;
  uint32_t& overflow = *overflow_ptr;
  const SameKey<kWide> same{&k, &info};
  uint32_t* first_b = first + info.fb;
  // table of two slots per entry, a power of two, at most kLdsSlots
  uint32_t slots = 256;
  while (slots < kLdsSlots && (int64_t)slots < 2 * n) slots <<= 1;
  const uint32_t mask = slots - 1;
  for (uint32_t i = threadIdx.x; i < slots; i += kThreads) tab[i] = kEmptySlot;
  if (threadIdx.x == 0) distinct = overflow = 0;
  __syncthreads();
  constexpr int kKeep = kLdsMaxEntries / kThreads;
  if (n <= kLdsMaxEntries) {
    // sure to fit; the thread's entries stay in registers between the phases
    uint64_t mine[kKeep];
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
      const int64_t i = j * kThreads + threadIdx.x;
      mine[j] = i < n ? entries[i] : kEmptySlot;
    }
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
      if (mine[j] != kEmptySlot) lds_insert_min(tab, mask, mine[j], same);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
      if (mine[j] != kEmptySlot) {
        const uint32_t f = lds_first_of(tab, mask, mine[j], same);
        if (f != (uint32_t)mine[j]) first_b[(uint32_t)mine[j]] = f;
      }
    return;
  }
  // Many entries: fine for the LDS table while few of them are distinct (a hub
  // that repeats thousands of times), so try, and count.  Entries are read
  // kDeep at a time per thread so that a long bucket streams at memory speed;
  // the overflow flag is read before every insert, which bounds the slots
  // claimed after it rises to one per thread.
  constexpr int kDeep = 8;
  volatile uint32_t* over = &overflow;
  for (int64_t base = 0; base < n && !*over; base += (int64_t)kThreads * kDeep) {
    uint64_t e[kDeep];
#pragma unroll
    for (int j = 0; j < kDeep; ++j) {
      const int64_t i = base + j * kThreads + threadIdx.x;
      e[j] = i < n ? entries[i] : kEmptySlot;
    }
#pragma unroll
    for (int j = 0; j < kDeep; ++j)
      if (e[j] != kEmptySlot && !*over)
        lds_insert_min_counted(tab, mask, e[j], same, &distinct, over);
  }
  __syncthreads();
  if (!overflow) {
    for (int64_t base = 0; base < n; base += (int64_t)kThreads * kDeep) {
      uint64_t e[kDeep];
#pragma unroll
      for (int j = 0; j < kDeep; ++j) {
        const int64_t i = base + j * kThreads + threadIdx.x;
        e[j] = i < n ? entries[i] : kEmptySlot;
      }
#pragma unroll
      for (int j = 0; j < kDeep; ++j)
        if (e[j] != kEmptySlot) {
          const uint32_t f = lds_first_of(tab, mask, e[j], same);
          if (f != (uint32_t)e[j]) first_b[(uint32_t)e[j]] = f;
        }
    }
    return;
  }
  // too many distinct keys: a table of its own from the pool, two slots per entry
  const uint64_t cap = (uint64_t)(2 * n + 1);
  if (threadIdx.x == 0) *pool_at = atomicAdd(pool_cur, (unsigned long long)cap);
  __syncthreads();
  uint64_t* gt = spill + *pool_at;
  // The table is private to this work-group: the barrier orders its stores and
  // atomics for the work-group's own wavefronts.  (A fence for the whole device
  // makes the die write its L2 back, tens of microseconds each time.)
  for (uint64_t i = threadIdx.x; i < cap; i += kThreads) gt[i] = kEmptySlot;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += kThreads)
    spill_insert_min(gt, cap, entries[i], same);
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += kThreads) {
    const uint64_t e = entries[i];
    const uint32_t f = spill_first_of(gt, cap, e, same);
    if (f != (uint32_t)e) first_b[(uint32_t)e] = f;
  }
}

// One work-group per bucket.  A bucket that is sure to fit the LDS table, in a
// call whose keys all fit the upper half of an entry (nearly every bucket of
// nearly every call), takes the short path below: the pass is bound by the
// instructions of its probe loops, not by LDS or memory, so the table is split
// into 32-bit keys and 32-bit positions (32-bit compares and atomics, a 32-bit
// multiplicative hash), and an entry remembers the slot its key landed in, so
// that reading the first position back is one load and no second probe.
// Everything else (oversize buckets, wide keys) goes through dedup_bucket.
constexpr uint32_t kNoTag = 0xFFFFFFFFu;  // never a tag, see key_tag

template <int kThreads>
__global__ __launch_bounds__(kThreads) void unique_dedup_kernel(
    Keys k, const int* __restrict__ wide_keys,
    const int32_t* __restrict__ bucket_batch, const BatchInfo* __restrict__ batch,
    const int64_t* __restrict__ bucket_cur, const int64_t* __restrict__ bucket_base,
    const int32_t* __restrict__ bucket_cap, const int64_t* __restrict__ ovf_cur,
    const uint64_t* __restrict__ packed, const uint64_t* __restrict__ ovf_entry,
    const int32_t* __restrict__ ovf_bucket, uint64_t* spill, unsigned long long* pool_cur,
    uint32_t* __restrict__ first, int64_t max_buckets, int remap) {
  __shared__ uint64_t tab[kLdsSlots];
  __shared__ uint32_t distinct;
  __shared__ uint32_t overflow;
  __shared__ unsigned long long pool_at;
  const int64_t g = unit_of_block(max_buckets, remap);
  if (g >= max_buckets) return;
  // Everything the bucket needs to know is asked for at once, and its entries
  // right behind (two round trips to memory, not one per early exit): an unused
  // bucket has count 0, and entries are only read below that count.
  const int32_t b = bucket_batch[g];
  const int64_t lo = bucket_base[g], n = bucket_cur[g];
  const int64_t region_cap = bucket_cap[g];
  const bool wide = *wide_keys != 0;
  constexpr int kKeep = kLdsMaxEntries / kThreads;
  uint64_t mine[kKeep];
  // (a region holds every entry of a bucket this small: it has room for
  // kBucketCap entries, or for as many as the batch has keys)
  const bool small = n <= kLdsMaxEntries;
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    const int64_t i = j * kThreads + threadIdx.x;
    mine[j] = small && i < n ? packed[lo + i] : kEmptySlot;
  }
  if (b < 0 || n == 0) return;  // uniform per work-group
  const BatchInfo info = batch[b];
  if (wide || !small) {
    BucketEntries entries{packed + lo, nullptr, n < region_cap ? n : region_cap};
    if (n > region_cap) {
      // collect what the partition pass left on the batch's overflow list
      if (threadIdx.x == 0) {
        pool_at = atomicAdd(pool_cur, (unsigned long long)(n - region_cap));
        distinct = 0;
      }
      __syncthreads();
      uint64_t* extra = spill + pool_at;
      const int32_t bin = (int32_t)(g - info.bucket0);
      const int64_t listed = ovf_cur[b];
      // (several loads per thread in flight, one LDS atomic per wavefront)
      constexpr int kDeep = 8;
      for (int64_t base = 0; base < listed; base += (int64_t)kThreads * kDeep) {
        int32_t of[kDeep];
        uint64_t e[kDeep];
#pragma unroll
        for (int j = 0; j < kDeep; ++j) {
          const int64_t i = base + j * kThreads + threadIdx.x;
          of[j] = i < listed ? ovf_bucket[info.fb + i] : -1;
          e[j] = ovf_entry[info.fb + (i < listed ? i : listed - 1)];
        }
#pragma unroll
        for (int j = 0; j < kDeep; ++j) {
          const bool hit = of[j] == bin;
          const uint64_t peers = __ballot(hit);
          if (peers == 0) continue;
          uint32_t at = 0;
          if (lane_id() == 0) at = atomicAdd(&distinct, (uint32_t)__popcll(peers));
          at = __shfl(at, 0);
          if (hit) extra[at + __popcll(peers & ((1ull << lane_id()) - 1ull))] = e[j];
        }
      }
      __syncthreads();  // (read back by this work-group only: no wider fence)
      entries.extra = extra;
    }
    if (wide)
      dedup_bucket<kThreads, true>(k, info, n, entries, spill, pool_cur, first, tab,
                                   &distinct, &overflow, &pool_at);
    else
      dedup_bucket<kThreads, false>(k, info, n, entries, spill, pool_cur, first, tab,
                                    &distinct, &overflow, &pool_at);
    return;
  }
  uint32_t* tags = (uint32_t*)tab;          // [slots]
  uint32_t* mins = tags + kLdsSlots;        // [slots]
  uint32_t shift = 24;  // 32 - log2(slots): 256 slots to start with
  while (shift > 20 && (int64_t)(1u << (32 - shift)) < 2 * n) --shift;
  const uint32_t slots = 1u << (32 - shift), mask = slots - 1;
  for (uint32_t i = threadIdx.x; i < slots; i += kThreads) {
    tags[i] = kNoTag;
    mins[i] = 0xFFFFFFFFu;
  }
  __syncthreads();
  uint32_t at[kKeep];
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    if (mine[j] == kEmptySlot) continue;
    const uint32_t tag = (uint32_t)(mine[j] >> 32), pos = (uint32_t)mine[j];
    uint32_t slot = (tag * 0x85EBCA6Bu) >> shift;  // a multiplier unrelated to the one that chose the bucket
    for (;;) {
      uint32_t cur = tags[slot];
      if (cur == kNoTag) cur = atomicCAS(&tags[slot], kNoTag, tag);
      if (cur == kNoTag || cur == tag) break;
      slot = (slot + 1) & mask;
    }
    at[j] = slot;
    if (mins[slot] > pos) atomicMin(&mins[slot], pos);
  }
  __syncthreads();
  uint32_t* first_b = first + info.fb;
#pragma unroll
  for (int j = 0; j < kKeep; ++j) {
    if (mine[j] == kEmptySlot) continue;
    const uint32_t f = mins[at[j]];
    if (f != (uint32_t)mine[j]) first_b[(uint32_t)mine[j]] = f;
  }
}

// ---------------------------------------------------------------- flag
// A value that is the same in every lane, moved to scalar registers so that
// what is computed from it (the batch search) runs on the scalar unit.
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
  return wave_uniform_first(v);
}

// Batches that a run of consecutive items may touch: from the batch of its
// first item to the batch of the next run's first item.
struct BatchSpan {
  int64_t lo, hi;
};
__device__ __forceinline__ BatchSpan batch_span(
    const int32_t* __restrict__ unit_batch, int64_t unit) {
  return BatchSpan{unit_batch[unit], unit_batch[unit + 1]};
}
__device__ __forceinline__ int64_t batch_in_span(const int64_t* __restrict__ ptr,
                                                 const BatchSpan& s, int64_t x) {
  return s.lo == s.hi ? s.lo : s.lo + segment_of(ptr + s.lo, s.hi - s.lo + 1, x);
}

// One work-group per group of kGroup positions; a wave takes kWordsPerWave
// consecutive words, lane l the positions l, l + 64, ...: coalesced rows whose
// ballots are the words.
__global__ __launch_bounds__(kBlock) void unique_flag_kernel(
    const int64_t* __restrict__ flat_ptr, const int32_t* __restrict__ group_batch,
    int64_t N, const uint32_t* __restrict__ first, RankWord* __restrict__ words,
    int64_t* __restrict__ group_cnt) {
  __shared__ uint32_t wave_total[kBlock / kWave];
  const int64_t group = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int64_t word0 = group * kGroupWords + wave * kWordsPerWave;
  const int64_t p0 = word0 * kWave;
  const BatchSpan span = batch_span(group_batch, group);
  const int64_t fb_lo = flat_ptr[span.lo];
  uint32_t f[kWordsPerWave];
#pragma unroll
  for (int j = 0; j < kWordsPerWave; ++j) {
    const int64_t p = p0 + j * kWave + lane;
    f[j] = p < N ? first[p] : 0u;
  }
  uint64_t my_bits = 0;
  uint32_t my_before = 0, total = 0;
#pragma unroll
  for (int j = 0; j < kWordsPerWave; ++j) {
    const int64_t p = p0 + j * kWave + lane;
    bool is_first = false;
    if (p < N) {
      const int64_t fb =
          span.lo == span.hi ? fb_lo : flat_ptr[batch_in_span(flat_ptr, span, p)];
      is_first = (int64_t)f[j] == p - fb;
    }
    const uint64_t bits = __ballot(is_first);
    if (lane == j) {
      my_bits = bits;
      my_before = total;
    }
    total += (uint32_t)__popcll(bits);
  }
  if (lane == 0) wave_total[wave] = total;
  __syncthreads();
  uint32_t base = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kBlock / kWave; ++w) {
    const uint32_t t = wave_total[w];
    if (w < wave) base += t;
    all += t;
  }
  if (lane < kWordsPerWave && (word0 + lane) * kWave < N)
    words[word0 + lane] = RankWord{my_bits, base + my_before, 0u};
  if (threadIdx.x == 0) group_cnt[group] = (int64_t)all;
}

// Number of first occurrences at flat positions < p, for p < N.
__device__ __forceinline__ int64_t rank_of(int64_t p, const RankWord* __restrict__ words,
                                           const int64_t* __restrict__ group_off) {
  const RankWord w = words[p / kWave];
  const int bit = (int)(p % kWave);
  return group_off[p / kGroup] + w.before +
         __popcll(w.bits & ((1ull << bit) - 1ull));
}

// ---------------------------------------------------------------- offsets
// One work-group: group counts -> group offsets (group_off[groups] = number of
// unique keys), then where the unique keys of every batch start.  The offsets
// also go to unique_ptr_mirror when that is given (pinned host memory, so that
// the host has them without a copy of its own).
constexpr int kOffsetsThreads = 1024;
__global__ __launch_bounds__(kOffsetsThreads) void unique_offsets_kernel(
    const int64_t* __restrict__ flat_ptr, int64_t B, int64_t N, int64_t groups,
    const int64_t* __restrict__ group_cnt, int64_t* group_off,
    const RankWord* __restrict__ words, int64_t* __restrict__ unique_ptr,
    int64_t* __restrict__ unique_ptr_ws, int64_t* unique_ptr_mirror) {
  __shared__ int64_t smem[kOffsetsThreads / kWave + 1];
  int64_t carry = 0;
  constexpr int kPer = 8;
  for (int64_t base = 0; base < groups; base += kOffsetsThreads * kPer) {
    const int64_t i0 = base + (int64_t)threadIdx.x * kPer;
    int64_t v[kPer], sum = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      v[j] = i0 + j < groups ? group_cnt[i0 + j] : 0;
      sum += v[j];
    }
    int64_t total;
    int64_t run = carry + block_exclusive_sum<int64_t, kOffsetsThreads>(sum, smem, &total);
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      if (i0 + j < groups) group_off[i0 + j] = run;
      run += v[j];
    }
    carry += total;
  }
  if (threadIdx.x == 0) group_off[groups] = carry;
  __syncthreads();
  for (int64_t b = threadIdx.x; b <= B; b += kOffsetsThreads) {
    const int64_t p = flat_ptr[b];
    int64_t r = carry;
    if (p < N) {
      const RankWord w = words[p / kWave];
      // written above by other threads of this work-group: read past the
      // compute unit's own cache
      const int64_t off = __hip_atomic_load(group_off + p / kGroup, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
      r = off + w.before + __popcll(w.bits & ((1ull << (int)(p % kWave)) - 1ull));
    }
    unique_ptr[b] = r;
    unique_ptr_ws[b] = r;
    if (unique_ptr_mirror) unique_ptr_mirror[b] = r;
  }
}

// ---------------------------------------------------------------- fill
// Streaming: first occurrences write their key to the frontier.  A wave reads
// the keys of its kWordsPerWave rows of 64 positions in one go (whole rows:
// about half of the positions are first occurrences, so every line is needed
// anyway) and then stores the flagged ones.
struct FillArgs {
  const int64_t* flat_ptr;
  const int32_t* group_batch;
  int64_t N;
  int64_t* out_unique;
};

__device__ __forceinline__ void fill_group(
    int64_t group, const Keys& k, const int64_t* __restrict__ flat_ptr,
    const int32_t* __restrict__ group_batch, const BatchInfo* __restrict__ batch,
    int64_t N, const RankWord* __restrict__ words,
    const int64_t* __restrict__ group_off, int64_t* __restrict__ out_unique) {
  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int64_t word0 = group * kGroupWords + wave * kWordsPerWave;
  if (wave_uniform(word0 * kWave) >= N) return;
  const BatchSpan span = batch_span(group_batch, group);
  const bool one_batch = span.lo == span.hi;
  BatchInfo info = batch[span.lo];
  RankWord mine{0ull, 0u, 0u};  // lane j holds word j of this wave
  if (lane < kWordsPerWave && (word0 + lane) * kWave < N) mine = words[word0 + lane];
  int64_t* out = out_unique + group_off[group];
  uint64_t key[kWordsPerWave];
#pragma unroll
  for (int j = 0; j < kWordsPerWave; ++j) {
    const int64_t p = (word0 + j) * kWave + lane;
    key[j] = 0;
    if (p < N) {
      if (!one_batch) info = batch[batch_in_span(flat_ptr, span, p)];
      key[j] = key_at(k, info, p - info.fb);
    }
  }
#pragma unroll
  for (int j = 0; j < kWordsPerWave; ++j) {
    const uint64_t bits = __shfl((unsigned long long)mine.bits, j, kWave);
    const uint32_t before = __shfl(mine.before, j, kWave);
    if ((bits >> lane) & 1ull)
      out[before + __popcll(bits & ((1ull << lane) - 1ull))] = (int64_t)key[j];
  }
}

__global__ __launch_bounds__(kBlock) void unique_fill_kernel(
    Keys k, FillArgs f, const BatchInfo* __restrict__ batch,
    const RankWord* __restrict__ words, const int64_t* __restrict__ group_off) {
  fill_group(blockIdx.x, k, f.flat_ptr, f.group_batch, batch, f.N, words, group_off,
             f.out_unique);
}

// ---------------------------------------------------------------- relabel
// The largest c in [0, n) with ptr[c] <= x (ptr nondecreasing, ptr[0] <= x) when
// a good guess is at hand: the wavefront looks at the 64 entries around the
// guess first, one round trip, and searches the rest only when the answer is
// not among them.  Columns of a sampled matrix hold about the same number of
// edges, so the column of an edge is close to its share of the batch's columns.
__device__ __forceinline__ int64_t wave_segment_near(const int64_t* __restrict__ ptr, int64_t n,
                                                     int64_t x, int64_t guess) {
  int64_t w0 = guess - kWave / 2;
  if (w0 > n - kWave) w0 = n - kWave;
  if (w0 < 0) w0 = 0;
  const int64_t c = w0 + lane_id();
  const bool ok = c < n && ptr[c] <= x;
  const int hits = __popcll(__ballot(ok));  // ok is monotone over the lanes
  if (hits == 0) return wave_segment_of(ptr, w0, x);  // before the window (w0 > 0 here)
  if (hits == kWave && w0 + kWave < n)
    return w0 + kWave - 1 + wave_segment_of(ptr + w0 + kWave - 1, n - (w0 + kWave - 1), x);
  return w0 + hits - 1;
}

// The column of every edge of a tile from the column pointer: edge e belongs
// to the last column c with col_indptr[c] <= e.  Two wavefronts find the
// columns of the tile's first and last edge among [col_begin, col_end), the
// columns of the tile's batches; every column that starts inside
// the tile marks its first edge with its number (of several empty columns at
// one edge the last, the owner, wins), and a running maximum over the tile
// carries the marks forward.  Leaves column - c_lo in head[] and returns c_lo.
__device__ __forceinline__ int64_t tile_columns(const int64_t* __restrict__ col_indptr,
                                                int64_t col_begin, int64_t col_end, int64_t e0,
                                                int64_t e1, int64_t guess_lo, int64_t guess_hi,
                                                int32_t* head, int64_t* ends,
                                                int32_t* wave_max) {
  static_assert(kRelabelItems % 4 == 0, "a thread scans whole int4s of head[]");
  constexpr int kQuads = kRelabelItems / 4;
  const int wave = threadIdx.x / kWave;
  int4* quads = reinterpret_cast<int4*>(head) + threadIdx.x * kQuads;
#pragma unroll
  for (int q = 0; q < kQuads; ++q) quads[q] = make_int4(0, 0, 0, 0);
  if (wave < 2) {
    const int64_t c = wave_segment_near(col_indptr + col_begin, col_end - col_begin,
                                        wave == 0 ? e0 : e1 - 1,
                                        (wave == 0 ? guess_lo : guess_hi) - col_begin);
    if (lane_id() == 0) ends[wave] = col_begin + c;
  }
  __syncthreads();
  const int64_t c_lo = ends[0], c_hi = ends[1];
  for (int64_t c = c_lo + 1 + threadIdx.x; c <= c_hi; c += kBlock) {
    const int64_t off = col_indptr[c] - e0;
    if (off > 0 && off < kRelabelTile) atomicMax(&head[off], (int32_t)(c - c_lo));
  }
  __syncthreads();
  int4 m[kQuads];
  int32_t run = 0;  // running maximum over this thread's chunk, then over the lanes' chunks
#pragma unroll
  for (int q = 0; q < kQuads; ++q) {
    m[q] = quads[q];
    m[q].x = max(m[q].x, run);
    m[q].y = max(m[q].y, m[q].x);
    m[q].z = max(m[q].z, m[q].y);
    m[q].w = max(m[q].w, m[q].z);
    run = m[q].w;
  }
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int32_t o = __shfl_up(run, d, kWave);
    if (lane_id() >= d) run = max(run, o);
  }
  if (lane_id() == kWave - 1) wave_max[wave] = run;
  int32_t before = __shfl_up(run, 1, kWave);
  if (lane_id() == 0) before = 0;
  __syncthreads();
  for (int w = 0; w < wave; ++w) before = max(before, wave_max[w]);
#pragma unroll
  for (int q = 0; q < kQuads; ++q)
    quads[q] = make_int4(max(m[q].x, before), max(m[q].y, before), max(m[q].z, before),
                         max(m[q].w, before));
  __syncthreads();
  return c_lo;
}

// kByIndptr: the edges are grouped by column and col_indptr (k.S + 1 entries)
// says where each column's edges start; edge_col is not read.
struct LabelArgs {
  const int32_t* etile_batch;
  const uint32_t* first;
  const int64_t* unique_ptr;
  const int64_t* edge_col;
  const int64_t* col_indptr;
  int64_t* out_row;
  int64_t* out_col;
  int remap;
  int col_prefilled;  // out_col holds every column's place inside its batch already
};

template <bool kByIndptr>
__device__ __forceinline__ void relabel_tile(
    const Keys& k, const int32_t* __restrict__ etile_batch,
    const BatchInfo* __restrict__ batch, const uint32_t* __restrict__ first,
    const RankWord* __restrict__ words, const int64_t* __restrict__ group_off,
    const int64_t* __restrict__ unique_ptr, const int64_t* __restrict__ edge_col,
    const int64_t* __restrict__ col_indptr, int64_t* __restrict__ out_row,
    int64_t* __restrict__ out_col_or_null, int remap, int col_prefilled) {
  const int64_t num_tiles = ceil_div_dev(k.E, kRelabelTile);
  const int64_t tile = unit_of_block(num_tiles, remap);
  if (tile >= num_tiles) return;
  const int64_t e0 = tile * kRelabelTile;
  const BatchSpan span = batch_span(etile_batch, tile);
  int64_t col[kRelabelItems];
  __shared__ __align__(16) int32_t head[kByIndptr ? kRelabelTile : 4];
  __shared__ int64_t ends[2];
  __shared__ int32_t wave_max[kBlock / kWave];
  uint32_t row_first[kRelabelItems];
  BatchInfo info = batch[span.lo];
  int64_t rank0 = unique_ptr[span.lo];
  // Seeds of a batch are distinct <=> its last seed is a first occurrence of
  // rank ns - 1; the label of seed c is then its place among the seeds.
  const bool one_batch = span.lo == span.hi;
  bool seeds_distinct = false;
  if (one_batch && out_col_or_null && info.ns > 0) {
    const int64_t q = info.fb + info.ns - 1;
    seeds_distinct = ((words[q / kWave].bits >> (int)(q % kWave)) & 1ull) &&
                     rank_of(q, words, group_off) - rank0 == info.ns - 1;
  }
  // Column labels that the sampler wrote already (a column's place inside its
  // batch) are the labels of a batch with distinct seeds: nothing to do for the
  // column side of such a tile.  Any other tile writes them as usual.
  int64_t* out_col = col_prefilled && seeds_distinct ? nullptr : out_col_or_null;
  // A lane takes pairs of neighbouring edges, so that its labels leave as
  // 16-byte stores: item i is edge  e0 + (i / 2) * 2 * kBlock + 2 * lane + i % 2.
  auto edge_of = [e0](int i) {
    return e0 + (int64_t)(i >> 1) * (2 * kBlock) + 2 * (int)threadIdx.x + (i & 1);
  };
#pragma unroll
  for (int i = 0; i < kRelabelItems; ++i) {
    const int64_t e = edge_of(i);
    if (e >= k.E) break;
    if (!one_batch) info = batch[batch_in_span(k.rows_ptr, span, e)];
    // row key e of batch b sits at flat position
    //   fb + (seeds of b) + (e - rows_ptr[b])  =  e + seeds_ptr[b + 1]
    if (out_row) row_first[i] = first[e + info.s_lo + info.ns];
    if (out_col && !kByIndptr) col[i] = edge_col[e];
  }
  if (kByIndptr && out_col) {
    // (after the loads above have been issued: they travel during the search)
    const int64_t e1 = e0 + kRelabelTile < k.E ? e0 + kRelabelTile : k.E;
    const BatchInfo head_b = batch[span.lo], last = batch[span.hi];
    // an edge's share of its batch's edges, taken of the batch's columns
    auto guess = [](const BatchInfo& b, int64_t e) {
      const int64_t edges = b.n - b.ns;
      return b.s_lo + (edges > 0 ? (int64_t)((double)(e - b.r_lo) / (double)edges * (double)b.ns) : 0);
    };
    const int64_t c_lo = tile_columns(col_indptr, head_b.s_lo, last.s_lo + last.ns, e0, e1,
                                      guess(head_b, e0), guess(last, e1 - 1), head, ends,
                                      wave_max);
#pragma unroll
    for (int i = 0; i < kRelabelItems; ++i) col[i] = c_lo + head[edge_of(i) - e0];
  }
  struct Pair {
    int64_t v[2];
  };
  const bool wide_stores = (((uintptr_t)out_row | (uintptr_t)out_col) & 15) == 0;
#pragma unroll
  for (int i = 0; i < kRelabelItems; i += 2) {
    Pair row_label{{0, 0}}, col_label{{0, 0}};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t e = edge_of(i + j);
      if (e >= k.E) break;
      if (!one_batch) {
        const int64_t b = batch_in_span(k.rows_ptr, span, e);
        info = batch[b];
        rank0 = unique_ptr[b];
      }
      if (out_row) row_label.v[j] = rank_of(info.fb + row_first[i + j], words, group_off) - rank0;
      // seed c of batch b sits at flat position c + rows_ptr[b]
      if (out_col)
        col_label.v[j] =
            seeds_distinct
                ? col[i + j] - info.s_lo
                : rank_of(info.fb + first[col[i + j] + info.r_lo], words, group_off) - rank0;
    }
    const int64_t e = edge_of(i);
    if (e + 1 < k.E && wide_stores) {
      if (out_row) __builtin_memcpy(__builtin_assume_aligned(out_row + e, 16), &row_label, sizeof(Pair));
      if (out_col) __builtin_memcpy(__builtin_assume_aligned(out_col + e, 16), &col_label, sizeof(Pair));
    } else {
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (e + j < k.E) {
          if (out_row) out_row[e + j] = row_label.v[j];
          if (out_col) out_col[e + j] = col_label.v[j];
        }
    }
  }
}

template <bool kByIndptr>
__global__ __launch_bounds__(kBlock) void unique_relabel_kernel(
    Keys k, LabelArgs l, const BatchInfo* __restrict__ batch,
    const RankWord* __restrict__ words, const int64_t* __restrict__ group_off) {
  relabel_tile<kByIndptr>(k, l.etile_batch, batch, l.first, words, group_off, l.unique_ptr,
                          l.edge_col, l.col_indptr, l.out_row, l.out_col, l.remap,
                          l.col_prefilled);
}

// Both of the above in one launch: the first `label_blocks` work-groups label
// tiles of edges, the rest write the frontier.  Neither reads what the other
// writes; the short frontier work-groups fill the machine while the last
// labelling ones drain.
template <bool kByIndptr>
__global__ __launch_bounds__(kBlock) void unique_fill_relabel_kernel(
    Keys k, FillArgs f, LabelArgs l, unsigned label_blocks,
    const BatchInfo* __restrict__ batch, const RankWord* __restrict__ words,
    const int64_t* __restrict__ group_off) {
  if (blockIdx.x < label_blocks)
    relabel_tile<kByIndptr>(k, l.etile_batch, batch, l.first, words, group_off, l.unique_ptr,
                            l.edge_col, l.col_indptr, l.out_row, l.out_col, l.remap,
                            l.col_prefilled);
  else
    fill_group(blockIdx.x - label_blocks, k, f.flat_ptr, f.group_batch, batch, f.N, words,
               group_off, f.out_unique);
}

// No keys at all: every batch is empty.
__global__ __launch_bounds__(kBlock) void unique_empty_kernel(
    int64_t* __restrict__ unique_ptr, int64_t* unique_ptr_mirror, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  unique_ptr[i] = 0;
  if (unique_ptr_mirror) unique_ptr_mirror[i] = 0;
}

static int check_unique_args(const int64_t* seeds, const int64_t* seeds_ptr,
                             int64_t S, const int64_t* rows,
                             const int64_t* rows_ptr, int64_t E, int64_t B) {
  GS_REQUIRE(S >= 0 && E >= 0, "unique: negative size");
  GS_REQUIRE(B >= 1, "unique: num_batches must be >= 1, got %lld", (long long)B);
  // positions and ranks inside a batch are kept as 32-bit values
  GS_REQUIRE(S + E < (int64_t(1) << 31),
             "unique: at most 2^31 - 1 keys per call, got %lld", (long long)(S + E));
  GS_REQUIRE(S == 0 || seeds, "unique: null seeds");
  GS_REQUIRE(E == 0 || rows, "unique: null rows");
  GS_REQUIRE((seeds_ptr == nullptr) == (rows_ptr == nullptr),
             "unique: seeds_ptr and rows_ptr must both be given or both be null");
  GS_REQUIRE(seeds_ptr != nullptr || B == 1,
             "unique: %lld batches need seeds_ptr / rows_ptr", (long long)B);
  return GS_OK;
}

static int check_workspace(const UniqueWs& w, const void* workspace,
                           size_t workspace_bytes) {
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("unique workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
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
                    int64_t num_batches, int64_t* unique_ptr,
                    int64_t* unique_ptr_mirror, void* workspace,
                    size_t workspace_bytes, gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  GS_REQUIRE(unique_ptr, "unique_count: null unique_ptr");
  UniqueWs w = carve_unique(workspace, S, E, B);
  if ((rc = check_workspace(w, workspace, workspace_bytes)) != GS_OK) return rc;
  hipStream_t s = as_stream(stream);
  const UniqueTuning tn = tuning();
  const int64_t N = S + E;
  if (N == 0) {
    GS_LAUNCH("unique_plan", s,
              unique_empty_kernel<<<dim3((unsigned)ceil_div(B + 1, kBlock)),
                                    dim3(kBlock), 0, s>>>(unique_ptr,
                                                          unique_ptr_mirror, B + 1));
    return GS_OK;
  }
  const Keys k{seeds, seeds_ptr, S, rows, rows_ptr, E, B};
  const UnitTables units{w.max_tiles,  w.max_buckets,  w.groups,      w.etiles,
                         w.tile_batch, w.bucket_batch, w.group_batch, w.etile_batch,
                         w.bucket_base, w.bucket_cap};
  const dim3 unit_grid((unsigned)ceil_div(units.units(), kBlock));
  if (B <= kPlanMaxBatches) {
    GS_LAUNCH("unique_plan", s,
              unique_plan_kernel<<<unit_grid, dim3(kBlock), 0, s>>>(
                  k, N, tn.bucket_keys, w.batch, w.flat_ptr, w.tile_ptr, w.bucket_ptr,
                  w.region_ptr, w.bucket_cur, w.ovf_cur, w.pool_cur, w.wide_keys, units));
  } else {
    int64_t blocks = ceil_div(w.max_buckets + 1, kBlock * 4);
    if (blocks > 1024) blocks = 1024;
    GS_LAUNCH("unique_plan", s,
              unique_prep_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, s>>>(
                  k, tn.bucket_keys, w.batch, w.flat_ptr, w.tile_ptr, w.bucket_ptr,
                  w.region_ptr, w.bucket_cur, w.max_buckets, w.ovf_cur, w.pool_cur,
                  w.wide_keys));
    GS_LAUNCH("unique_units", s,
              unique_units_kernel<<<unit_grid, dim3(kBlock), 0, s>>>(
                  k, N, w.flat_ptr, w.tile_ptr, w.bucket_ptr, w.region_ptr, units));
  }
  const dim3 tile_grid((unsigned)grid_for_units(w.max_tiles, tn.remap));
  GS_LAUNCH("unique_scatter", s,
            unique_scatter_kernel<<<tile_grid, dim3(kScatterThreads), 0, s>>>(
                k, w.tile_batch, w.batch, w.bucket_cur, w.ovf_cur, w.packed, w.ovf_entry,
                w.ovf_bucket, w.first, w.max_tiles, tn.remap, w.wide_keys));
  GS_LAUNCH("unique_dedup", s,
            unique_dedup_kernel<512><<<dim3((unsigned)grid_for_units(w.max_buckets, tn.remap)),
                                       dim3(512), 0, s>>>(
                k, w.wide_keys, w.bucket_batch, w.batch, w.bucket_cur, w.bucket_base,
                w.bucket_cap, w.ovf_cur, w.packed, w.ovf_entry, w.ovf_bucket, w.spill,
                w.pool_cur, w.first, w.max_buckets, tn.remap));
  GS_LAUNCH("unique_flag", s,
            unique_flag_kernel<<<dim3((unsigned)w.groups), dim3(kBlock), 0, s>>>(
                w.flat_ptr, w.group_batch, N, w.first, w.words, w.group_cnt));
  GS_LAUNCH("unique_offsets", s,
            unique_offsets_kernel<<<dim3(1), dim3(kOffsetsThreads), 0, s>>>(
                w.flat_ptr, B, N, w.groups, w.group_cnt, w.group_off, w.words,
                unique_ptr, w.unique_ptr, unique_ptr_mirror));
  return GS_OK;
}

// The launches behind gs_unique_fill, gs_unique_relabel and gs_unique_fill_relabel.
static int launch_fill_relabel(const gs::Keys& k, const gs::UniqueWs& w, int64_t* out_unique,
                               const int64_t* edge_col, const int64_t* col_indptr,
                               int64_t* out_row, int64_t* out_col, int col_prefilled,
                               hipStream_t s) {
  using namespace gs;
  const UniqueTuning tn = tuning();
  const int64_t N = k.S + k.E;
  const bool fill = out_unique != nullptr && N > 0;
  const bool label = k.E > 0 && (out_row || out_col);
  const bool by_indptr = out_col && col_indptr;
  const FillArgs f{w.flat_ptr, w.group_batch, N, out_unique};
  const LabelArgs l{w.etile_batch, w.first, w.unique_ptr, by_indptr ? nullptr : edge_col,
                    by_indptr ? col_indptr : nullptr, out_row, out_col, tn.remap,
                    col_prefilled && by_indptr ? 1 : 0};
  const unsigned label_blocks =
      label ? (unsigned)grid_for_units(ceil_div(k.E, kRelabelTile), tn.remap) : 0u;
  if (fill && label) {
    const dim3 grid(label_blocks + (unsigned)w.groups);
    if (by_indptr)
      GS_LAUNCH("unique_fill_relabel", s,
                unique_fill_relabel_kernel<true><<<grid, dim3(kBlock), 0, s>>>(
                    k, f, l, label_blocks, w.batch, w.words, w.group_off));
    else
      GS_LAUNCH("unique_fill_relabel", s,
                unique_fill_relabel_kernel<false><<<grid, dim3(kBlock), 0, s>>>(
                    k, f, l, label_blocks, w.batch, w.words, w.group_off));
  } else if (fill) {
    GS_LAUNCH("unique_fill", s,
              unique_fill_kernel<<<dim3((unsigned)w.groups), dim3(kBlock), 0, s>>>(
                  k, f, w.batch, w.words, w.group_off));
  } else if (label) {
    if (by_indptr)
      GS_LAUNCH("unique_relabel", s,
                unique_relabel_kernel<true><<<dim3(label_blocks), dim3(kBlock), 0, s>>>(
                    k, l, w.batch, w.words, w.group_off));
    else
      GS_LAUNCH("unique_relabel", s,
                unique_relabel_kernel<false><<<dim3(label_blocks), dim3(kBlock), 0, s>>>(
                    k, l, w.batch, w.words, w.group_off));
  }
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
  if ((rc = check_workspace(w, workspace, workspace_bytes)) != GS_OK) return rc;
  if (S + E == 0) return GS_OK;
  GS_REQUIRE(out_unique, "unique_fill: null out_unique");
  const Keys k{seeds, seeds_ptr, S, rows, rows_ptr, E, B};
  return launch_fill_relabel(k, w, out_unique, nullptr, nullptr, nullptr, nullptr, 0,
                             as_stream(stream));
}

static int check_label_args(int64_t S, int64_t E, const int64_t* edge_col,
                            const int64_t* col_indptr, const int64_t* out_col) {
  GS_REQUIRE(out_col == nullptr || E == 0 || (edge_col != nullptr) != (col_indptr != nullptr),
             "unique_relabel: out_col needs edge_col or col_indptr (one of them)");
  GS_REQUIRE(col_indptr == nullptr || E == 0 || S > 0,
             "unique_relabel: %lld edges grouped by column but no seeds", (long long)E);
  return GS_OK;
}

int gs_unique_relabel(const int64_t* seeds, const int64_t* seeds_ptr,
                      int64_t num_seeds, const int64_t* rows,
                      const int64_t* rows_ptr, int64_t num_rows_keys,
                      int64_t num_batches, const int64_t* edge_col,
                      const int64_t* col_indptr, int64_t* out_row, int64_t* out_col,
                      int out_col_prefilled, void* workspace, size_t workspace_bytes,
                      gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  if ((rc = check_label_args(S, E, edge_col, col_indptr, out_col)) != GS_OK) return rc;
  UniqueWs w = carve_unique(workspace, S, E, B);
  if ((rc = check_workspace(w, workspace, workspace_bytes)) != GS_OK) return rc;
  const Keys k{seeds, seeds_ptr, S, rows, rows_ptr, E, B};
  return launch_fill_relabel(k, w, nullptr, edge_col, col_indptr, out_row, out_col,
                             out_col_prefilled, as_stream(stream));
}

int gs_unique_fill_relabel(const int64_t* seeds, const int64_t* seeds_ptr,
                           int64_t num_seeds, const int64_t* rows,
                           const int64_t* rows_ptr, int64_t num_rows_keys,
                           int64_t num_batches, const int64_t* unique_ptr,
                           int64_t* out_unique, const int64_t* edge_col,
                           const int64_t* col_indptr, int64_t* out_row, int64_t* out_col,
                           int out_col_prefilled, void* workspace, size_t workspace_bytes,
                           gs_stream_t stream) {
  using namespace gs;
  const int64_t S = num_seeds, E = num_rows_keys, B = num_batches;
  int rc = check_unique_args(seeds, seeds_ptr, S, rows, rows_ptr, E, B);
  if (rc != GS_OK) return rc;
  GS_REQUIRE(unique_ptr, "unique_fill_relabel: null unique_ptr");
  if ((rc = check_label_args(S, E, edge_col, col_indptr, out_col)) != GS_OK) return rc;
  UniqueWs w = carve_unique(workspace, S, E, B);
  if ((rc = check_workspace(w, workspace, workspace_bytes)) != GS_OK) return rc;
  GS_REQUIRE(S + E == 0 || out_unique, "unique_fill_relabel: null out_unique");
  const Keys k{seeds, seeds_ptr, S, rows, rows_ptr, E, B};
  return launch_fill_relabel(k, w, out_unique, edge_col, col_indptr, out_row, out_col,
                             out_col_prefilled, as_stream(stream));
}

}  // extern "C"
