// coosort.hip -- stable sort of edge positions by an id of at most 32 bits: the
// first half of turning an edge list into a matrix compressed by column (or by
// row).  Least significant digit first, 8 bits a pass, like a library radix
// sort of (id, position) pairs -- but between the passes an edge is 8 bytes (id
// and position, 32 bits each) where the 64-bit interface makes it 16, the
// positions of the first pass are never read (an edge's position is its index),
// and only the last pass writes 64-bit outputs.
//
// One counting pass reads the ids once and gives every pass the place where each
// of its 256 digit values starts.  A pass then runs tile by tile: a work-group
// takes a ticket (tiles are handed out in the order in which work-groups start,
// so every earlier tile is already running or done), ranks its 8192 edges by
// digit value in stable order, publishes how many edges of every digit value it
// holds, and learns how many the earlier tiles hold by walking back over what
// they have published -- per tile and digit value one 64-bit word, `state | count`,
// written and read with relaxed device-scope accesses, so that no fence is
// needed: the word is the message.  An earlier tile's word is either its own
// count (walk on) or already the sum over all tiles up to it (stop).  Meanwhile
// the tile's edges are put in order in LDS, so that they leave in runs of
// neighbouring addresses.  A wait for a word that has not been written yet is
// bounded; when the bound is reached the pass gives up on waiting, sets a flag in
// the first word of the workspace and writes into valid places all the same.
#include "common.h"

namespace gs {

constexpr int kCooBits = 8;
constexpr int kCooBins = 1 << kCooBits;
constexpr int kCooThreads = 512;
constexpr int kCooWaves = kCooThreads / kWave;
constexpr int kCooItems = 16;                          // edges per thread
constexpr int kCooChunk = kCooItems * kWave;           // consecutive edges a wavefront ranks
constexpr int kCooTile = kCooThreads * kCooItems;
constexpr int kCooMaxPasses = 4;                       // 32 bits
constexpr int kCooCountGroups = 1024;                  // work-groups of the counting pass
constexpr int kCooCopies = 8;                          // copies of the counters in a counting work-group
constexpr int kCooBaseThreads = 1024;
constexpr int kCooBaseShares = kCooBaseThreads / kCooBins;
constexpr uint32_t kCooSpinLimit = 1u << 16;
constexpr int kCooWindow = 4;                          // earlier tiles looked at in one round trip
static_assert(kCooChunk <= 65535, "a wavefront's counts are 16 bits wide");
static_assert(kCooBins <= kCooThreads, "a thread looks after at most one digit value");
static_assert(kCooBins == 4 * kWave, "one wavefront scans the tile's counts, four to a lane");

struct IdPos {
  uint32_t id, pos;
};

// Words of `flags`, the head of the workspace: the gave-up flag, then a ticket
// counter per pass.
constexpr int kCooGaveUp = 0;
constexpr int kCooTicket = 8;

// ---------------------------------------------------------------- counting
// Every work-group counts the digit values of all passes over its share of the
// ids and leaves its counts in a row of `partial`; on the way the grid clears the
// state words of the tiles.
__global__ __launch_bounds__(kCooThreads) void coosort_count_kernel(
    const int64_t* __restrict__ major, int64_t n, int passes,
    uint32_t* __restrict__ partial, uint4* __restrict__ clear, int64_t clear_quads) {
  __shared__ uint32_t h[kCooMaxPasses * kCooCopies * kCooBins];
  const int bins = passes * kCooBins;
  for (int i = threadIdx.x; i < bins * kCooCopies; i += kCooThreads) h[i] = 0;
  __syncthreads();
  const int64_t stride = (int64_t)gridDim.x * kCooThreads;
  const int64_t first = (int64_t)blockIdx.x * kCooThreads + threadIdx.x;
  // Every eighth lane shares a copy of the counters: ids of a power law put most
  // edges on a few values of the upper digits, ids that arrive in order on one,
  // and 64 additions to one LDS counter take 64 turns.
  uint32_t* mine = h + (lane_id() % kCooCopies) * kCooBins;
  auto count = [&](uint32_t id) {
    for (int p = 0; p < passes; ++p) {
      const uint32_t d = (id >> (p * kCooBits)) & (kCooBins - 1);
      uint32_t* at = &mine[p * kCooCopies * kCooBins + d];
      const uint64_t same = __ballot(d == (uint32_t)__builtin_amdgcn_readfirstlane(d));
      if (same != __ballot(true))
        atomicAdd(at, 1u);
      else if ((same & ((1ull << lane_id()) - 1ull)) == 0)  // one value in the wavefront: its first lane
        atomicAdd(at, (uint32_t)__popcll(same));
    }
  };
  if ((reinterpret_cast<uintptr_t>(major) & 15) == 0) {  // two ids a load
    const longlong2* pairs = reinterpret_cast<const longlong2*>(major);
    const int64_t num_pairs = n >> 1;
    for (int64_t q = first; q < num_pairs; q += stride) {
      const longlong2 v = pairs[q];
      count((uint32_t)v.x);
      count((uint32_t)v.y);
    }
    if (first == 0 && (n & 1)) count((uint32_t)major[n - 1]);
  } else {
    for (int64_t e = first; e < n; e += stride) count((uint32_t)major[e]);
  }
  for (int64_t q = first; q < clear_quads; q += stride) clear[q] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  uint32_t* row = partial + (int64_t)blockIdx.x * bins;
  for (int i = threadIdx.x; i < bins; i += kCooThreads) {
    const int p = i / kCooBins, d = i % kCooBins;
    uint32_t sum = 0;
#pragma unroll
    for (int c = 0; c < kCooCopies; ++c) sum += h[(p * kCooCopies + c) * kCooBins + d];
    row[i] = sum;
  }
}

// One work-group per pass: sums the rows of `partial` and scans the sums, so
// that base[pass][v] is the place of the first edge whose digit value is v.
__global__ __launch_bounds__(kCooBaseThreads) void coosort_bases_kernel(
    const uint32_t* __restrict__ partial, int groups, int passes,
    uint32_t* __restrict__ base, uint32_t* __restrict__ flags) {
  __shared__ uint32_t share[kCooBaseShares][kCooBins];
  __shared__ uint32_t smem[kCooBaseThreads / kWave + 1];
  const int p = blockIdx.x;
  const int bins = passes * kCooBins;
  const int d = threadIdx.x % kCooBins, q = threadIdx.x / kCooBins;
  uint32_t c = 0;
#pragma unroll 8
  for (int g = q; g < groups; g += kCooBaseShares) c += partial[(int64_t)g * bins + p * kCooBins + d];
  share[q][d] = c;
  __syncthreads();
  uint32_t sum = 0;
  if (threadIdx.x < kCooBins) {
#pragma unroll
    for (int i = 0; i < kCooBaseShares; ++i) sum += share[i][d];
  }
  // (every thread takes part in the scan; the first kCooBins hold the counts)
  uint32_t total;
  const uint32_t run = block_exclusive_sum<uint32_t, kCooBaseThreads>(sum, smem, &total);
  if (threadIdx.x < kCooBins) base[p * kCooBins + d] = run;
  if (threadIdx.x == kCooBaseThreads - 1) {
    flags[kCooTicket + p] = 0;
    if (p == 0) flags[kCooGaveUp] = 0;
  }
}

// ------------------------------------------------------------------- a pass
__device__ __forceinline__ uint64_t state_load(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void state_store(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// kFirst: the edges are read from `major` (the position of an edge is its
// index); otherwise from `src`.  kLast: ids and positions leave as 64-bit
// outputs; otherwise as 8-byte pairs in `dst`.  `pass` numbers the passes of a
// call from 0: its two states are 2 * pass + 2 (a tile's own count) and
// 2 * pass + 3 (the sum up to and including the tile), so the words of the pass
// before, and cleared ones, read as "not written yet".
constexpr int kCooStateShift = 60;
template <bool kFirst, bool kLast>
__global__ __launch_bounds__(kCooThreads, 4) void coosort_pass_kernel(
    const int64_t* __restrict__ major, const IdPos* __restrict__ src, IdPos* __restrict__ dst,
    int64_t* __restrict__ sorted_major, int64_t* __restrict__ perm, int64_t n, int shift,
    int pass, const uint32_t* __restrict__ base, uint64_t* state, uint32_t* flags) {
  __shared__ uint16_t cnt[kCooWaves][kCooBins];          // per wavefront: edges of a digit value so far
  __shared__ __align__(16) uint32_t start[kCooBins];     // where a digit value's edges start in the tile
  __shared__ uint32_t shift_out[kCooBins];               // (place in the output) - (place in the tile)
  __shared__ IdPos stage[kCooTile];
  __shared__ uint32_t tile_s;
  if (threadIdx.x == 0) tile_s = atomicAdd(&flags[kCooTicket + pass], 1u);
  {
    uint32_t* words = reinterpret_cast<uint32_t*>(&cnt[0][0]);
    for (int i = threadIdx.x; i < kCooWaves * kCooBins / 2; i += kCooThreads) words[i] = 0;
  }
  __syncthreads();
  const int64_t tile = tile_s;
  const int wave = threadIdx.x / kWave, lane = lane_id();
  const int64_t t0 = tile * kCooTile;
  const int64_t e0 = t0 + (int64_t)wave * kCooChunk + lane;
  // A wavefront takes kCooChunk consecutive edges, row by row of 64: the stable
  // order of the tile is (wavefront, row, lane).
  uint32_t id[kCooItems], pos[kCooItems];
#pragma unroll
  for (int i = 0; i < kCooItems; ++i) {
    const int64_t e = e0 + i * kWave;
    id[i] = pos[i] = 0;
    if (e < n) {
      if (kFirst) {
        id[i] = (uint32_t)major[e];
        pos[i] = (uint32_t)e;
      } else {
        const IdPos v = src[e];
        id[i] = v.id;
        pos[i] = v.pos;
      }
    }
  }
  // Rank inside the wavefront's chunk: the lanes of a row that hold the same
  // digit value find each other bit by bit; the lowest of them takes the
  // counter's value for all and adds their number.
  uint32_t rank[kCooItems];
  const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
  for (int i = 0; i < kCooItems; ++i) {
    const bool valid = e0 + i * kWave < n;
    const uint32_t d = (id[i] >> shift) & (kCooBins - 1);
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kCooBits; ++b) {
      const bool bit = (d >> b) & 1u;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const int leader = valid ? __builtin_ctzll(peers) : lane;
    uint32_t old = 0;
    if (valid && lane == leader) {
      old = cnt[wave][d];
      cnt[wave][d] = (uint16_t)(old + (uint32_t)__popcll(peers));
    }
    old = __shfl(old, leader, kWave);
    rank[i] = old + (uint32_t)__popcll(peers & below);
  }
  __syncthreads();
  // Per digit value: the wavefronts' counts become their offsets in the tile's
  // run of that value; the tile's count goes out for the later tiles to see.
  const uint64_t own_state = (uint64_t)(2 * pass + 2), sum_state = own_state + 1;
  constexpr uint64_t kCount = (1ull << kCooStateShift) - 1ull;
  uint64_t* mine = state + tile * kCooBins;
  uint32_t total = 0;
  if (threadIdx.x < kCooBins) {
    const int d = threadIdx.x;
#pragma unroll
    for (int w = 0; w < kCooWaves; ++w) {
      const uint32_t c = cnt[w][d];
      cnt[w][d] = (uint16_t)total;
      total += c;
    }
    state_store(mine + d, ((tile == 0 ? sum_state : own_state) << kCooStateShift) | total);
    start[d] = total;
  }
  __syncthreads();
  if (wave == 0) {  // exclusive scan of the tile's 256 counts, four to a lane
    const uint4 c = reinterpret_cast<uint4*>(start)[lane];
    const uint32_t sum = c.x + c.y + c.z + c.w;
    const uint32_t run = wave_inclusive_sum(sum) - sum;
    reinterpret_cast<uint4*>(start)[lane] =
        make_uint4(run, run + c.x, run + c.x + c.y, run + c.x + c.y + c.z);
  }
  __syncthreads();
  // The edges in the tile's order, in LDS.
#pragma unroll
  for (int i = 0; i < kCooItems; ++i) {
    if (e0 + i * kWave >= n) continue;
    const uint32_t d = (id[i] >> shift) & (kCooBins - 1);
    stage[start[d] + cnt[wave][d] + rank[i]] = IdPos{id[i], pos[i]};
  }
  // How many edges of my digit value the earlier tiles hold.
  if (threadIdx.x < kCooBins) {
    const int d = threadIdx.x;
    uint64_t before = 0;
    int64_t back = tile - 1;
    uint32_t spins = 0;
    // kCooWindow earlier tiles a round trip; tile 0 posts a sum, so the walk ends
    // there at the latest.
    while (back >= 0) {
      uint64_t w[kCooWindow];
#pragma unroll
      for (int k = 0; k < kCooWindow; ++k)
        w[k] = back - k >= 0 ? state_load(state + (back - k) * kCooBins + d) : 0;
      bool waiting = false;
#pragma unroll
      for (int k = 0; k < kCooWindow; ++k) {
        if (waiting || back < 0) continue;
        const uint64_t s = w[k] >> kCooStateShift;
        if (s == sum_state) {
          before += w[k] & kCount;
          back = -1;
        } else if (s == own_state) {
          before += w[k] & kCount;
          --back;
        } else {
          waiting = true;  // not written yet: ask again, from this tile on
        }
      }
      if (waiting && ++spins > kCooSpinLimit) {
        flags[kCooGaveUp] = 1;
        break;
      }
    }
    if (tile > 0) state_store(mine + d, (sum_state << kCooStateShift) | (before + total));
    shift_out[d] = base[d] + (uint32_t)before - start[d];
  }
  __syncthreads();
  const int64_t left = n - t0;
  const int here = (int)(left < kCooTile ? left : kCooTile);
#pragma unroll
  for (int i = 0; i < kCooItems; ++i) {
    const int j = i * kCooThreads + threadIdx.x;
    if (j >= here) break;
    const IdPos v = stage[j];
    const uint32_t out = (uint32_t)j + shift_out[(v.id >> shift) & (kCooBins - 1)];
    if (kLast) {
      sorted_major[out] = (int64_t)v.id;
      perm[out] = (int64_t)v.pos;
    } else {
      dst[out] = v;
    }
  }
}

// ------------------------------------------------------------------- host
struct CooSortWs {
  uint32_t* flags;
  uint32_t* partial;
  uint32_t* base;
  uint64_t* state;
  IdPos* buf[2];
  int64_t tiles;
  int groups;
  size_t total;
};

static CooSortWs carve_coosort(void* ws, int64_t nnz, int passes) {
  Carver c(ws);
  CooSortWs w;
  const size_t ids = (size_t)(nnz > 0 ? nnz : 1);
  w.tiles = ceil_div((int64_t)ids, kCooTile);
  w.groups = (int)(w.tiles < kCooCountGroups ? w.tiles : kCooCountGroups);
  w.flags = c.take<uint32_t>(64);  // first: the gave-up flag is the first word of the workspace
  w.partial = c.take<uint32_t>((size_t)kCooCountGroups * passes * kCooBins);
  w.base = c.take<uint32_t>((size_t)passes * kCooBins);
  w.state = c.take<uint64_t>((size_t)w.tiles * kCooBins);
  w.buf[0] = passes >= 2 ? c.take<IdPos>(ids) : nullptr;
  w.buf[1] = passes >= 3 ? c.take<IdPos>(ids) : nullptr;
  w.total = c.total();
  return w;
}

int coosort_passes(int id_bits) { return id_bits <= kCooBits ? 1 : (id_bits + kCooBits - 1) / kCooBits; }

size_t coosort_workspace_bytes(int64_t nnz, int id_bits) {
  return carve_coosort(nullptr, nnz, coosort_passes(id_bits)).total;
}

// sorted_major / perm = the ids and positions of `major` in stable id order, for
// ids below 2^id_bits, id_bits <= 32, 0 < nnz < 2^32.
int coosort_run(const int64_t* major, int64_t nnz, int id_bits, int64_t* sorted_major,
                int64_t* perm, void* workspace, hipStream_t s) {
  const int passes = coosort_passes(id_bits);
  const CooSortWs w = carve_coosort(workspace, nnz, passes);
  const int64_t clear_quads = w.tiles * kCooBins / 2;
  GS_LAUNCH("coo_sort_count", s,
            coosort_count_kernel<<<dim3((unsigned)w.groups), dim3(kCooThreads), 0, s>>>(
                major, nnz, passes, w.partial, reinterpret_cast<uint4*>(w.state), clear_quads));
  GS_LAUNCH("coo_sort_count", s,
            coosort_bases_kernel<<<dim3((unsigned)passes), dim3(kCooBaseThreads), 0, s>>>(
                w.partial, w.groups, passes, w.base, w.flags));
  const dim3 grid((unsigned)w.tiles);
  const IdPos* src = nullptr;
  for (int p = 0; p < passes; ++p) {
    const bool first = p == 0, last = p == passes - 1;
    IdPos* dst = last ? nullptr : w.buf[p % 2];
    const int shift = p * kCooBits;
    const uint32_t* base = w.base + p * kCooBins;
#define GS_COO_PASS(F, L)                                                                  \
  GS_LAUNCH("coo_sort_pass", s,                                                            \
            coosort_pass_kernel<F, L><<<grid, dim3(kCooThreads), 0, s>>>(                  \
                major, src, dst, sorted_major, perm, nnz, shift, p, base, w.state, w.flags))
    if (first && last)
      GS_COO_PASS(true, true);
    else if (first)
      GS_COO_PASS(true, false);
    else if (last)
      GS_COO_PASS(false, true);
    else
      GS_COO_PASS(false, false);
#undef GS_COO_PASS
    src = dst;
  }
  return GS_OK;
}

}  // namespace gs
