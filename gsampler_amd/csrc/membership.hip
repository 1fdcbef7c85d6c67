// membership.hip -- slicing across the compressed axis: keep the edges whose
// minor id (row id of a CSC, or any id array of a COO) belongs to a picked set
// and relabel that id to its position in the set.
//
//   count: hash the picked ids (smallest position wins for repeated ids); a
//          wave tests 256 consecutive edges as four coalesced rows whose
//          ballots are the chunk's flag words and counts the kept ones; scan
//          of the chunk counts; out_indptr[c] = kept edges before indptr[c].
//          The count pass also leaves, per chunk, the new ids (positions in
//          the picked set) of the chunk's kept edges in edge order.
//   fill : kept edge e goes to its rank (chunk offset + popcounts), edge order
//          preserved; its new id comes from the chunk's staged run, so the fill
//          pass reads neither the ids nor the table again.
//
// A table slot is  low 32 bits of the id << 32 | position in the picked set.
// While every picked id is below 2^32 - 1 those bits are the id, and an edge
// whose id is larger cannot match.  When a picked id is larger (an id of a very
// large graph, an id encoded as id + batch * num_rows) the insert pass raises a
// flag, and every match of the 32-bit halves is then confirmed against the
// picked id itself.
#include "common.h"
#include "hashtable.h"
#include "scan.h"

namespace gs {

constexpr int kMemberWords = kBlock / kWave;  // flag words per chunk of kBlock edges
constexpr int kMemberChunksPerWave = 8;
constexpr int kMemberAhead = 4;  // chunks of a wave whose loads are in flight together
static_assert(kMemberChunksPerWave % kMemberAhead == 0 && kMemberChunksPerWave * kMemberWords <= kWave,
              "a wave's flag words fit one word per lane");
constexpr int kMemberThreads = 1024;  // 16 waves share one staged table: 32 Ki edges per 32 KB copied
constexpr int kMemberLdsSlots = 4096;  // tables up to this size are staged in LDS (32 KB)
constexpr int64_t kMemberSmallEdges = int64_t(1) << 23;  // below: work-groups of kBlock threads

// A table too large for LDS is looked up in L2, one request per probe, and the
// flag pass then runs at the rate of those requests.  Most edges are not kept
// (a slice picks a small part of the rows), so a filter that does fit LDS sends
// them away first: a word of 32 bits per id group, three bits per picked id
// (a blocked Bloom filter; with up to eight ids per word about one absent id in
// twenty passes).  Only ids that pass go on to the table.
constexpr int kFilterWords = 16384;            // 64 KB of LDS
constexpr int kFilterGroupsPerCu = 2;          // work-groups of 1024 threads that fit a compute unit
constexpr int64_t kFilterMaxIds = 8 * kFilterWords;  // beyond: too many bits set to be worth a look

__device__ __forceinline__ uint32_t filter_word(uint32_t key) {
  return (key * 0x9E3779B1u) >> 18;  // top 14 bits: [0, kFilterWords)
}
__device__ __forceinline__ uint32_t filter_bits(uint32_t key) {
  const uint32_t h = key * 0x85EBCA6Bu;
  return (1u << (h >> 27)) | (1u << ((h >> 22) & 31u)) | (1u << ((h >> 17) & 31u));
}
static_assert(kFilterWords == 1 << 14, "filter_word keeps 14 bits");

struct MemberWs {
  uint64_t* table;     // [member_table_slots(num_picked)]
  uint64_t* flags;     // [chunks * kMemberWords]
  uint32_t* staged;    // [chunks * kBlock]: per chunk, the new ids of its kept edges, in order
  int64_t* chunk_off;  // [chunks + 1]
  int* wide;           // [1] set when a picked id does not fit the upper half of a slot
  uint32_t* filter;    // [kFilterWords] which ids may be in the table (for tables kept in L2)
  void* scan_ws;
  size_t scan_ws_bytes;
  int64_t chunks;
  size_t total;
};

// Slots of the table: four per picked id (fewer probes for the ids that are
// not there, which are most: 1.4 instead of 2.5 on average) while the table
// fits in LDS or stays a small part of a die's L2, else two.
constexpr int64_t kMemberRoomyIds = 65536;   // 4 slots * 8 B * 65536 = 2 MB
static uint64_t member_table_slots(int64_t num_picked) {
  const uint64_t roomy = (uint64_t)(4 * num_picked + 2), tight = (uint64_t)(2 * num_picked + 2);
  if (roomy <= (uint64_t)kMemberLdsSlots) return roomy;   // in LDS, roomy
  if (tight <= (uint64_t)kMemberLdsSlots) return tight;   // still in LDS
  return num_picked <= kMemberRoomyIds ? roomy : tight;   // in L2
}

static MemberWs carve_member(void* ws, int64_t nnz, int64_t num_picked) {
  Carver c(ws);
  MemberWs w;
  w.chunks = ceil_div(nnz > 0 ? nnz : 1, kBlock);
  w.table = c.take<uint64_t>((size_t)member_table_slots(num_picked));
  w.flags = c.take<uint64_t>((size_t)w.chunks * kMemberWords);
  w.staged = c.take<uint32_t>((size_t)w.chunks * kBlock);
  w.chunk_off = c.take<int64_t>((size_t)w.chunks + 1);
  w.wide = c.take<int>(1);
  w.filter = c.take<uint32_t>((size_t)kFilterWords);
  w.scan_ws_bytes = scan_workspace_bytes(w.chunks + 1);
  w.scan_ws = c.take<char>(w.scan_ws_bytes);
  w.total = c.total();
  return w;
}

// The look-ups run once per edge, so they are kept to 32-bit arithmetic: an
// admissible id fits 32 bits, the home slot is one multiply and one
// multiply-high, and a probe compares the upper half of a packed slot.
constexpr uint32_t kNoKey = 0xFFFFFFFFu;  // upper half of the empty slot; no admissible id

__device__ __forceinline__ uint32_t member_home(uint32_t key, uint32_t cap) {
  return __umulhi(key * 0x9E3779B1u, cap);
}

// 32-bit form of an id when every picked id fits 32 bits: kNoKey for one that
// no picked id can equal
__device__ __forceinline__ uint32_t member_key(uint64_t id) {
  return id <= kMaxPackedKey ? (uint32_t)id : kNoKey;
}
// 32-bit tag of any id: its low half, kept clear of kNoKey
__device__ __forceinline__ uint32_t member_tag(uint64_t id) {
  const uint32_t t = (uint32_t)id;
  return t == kNoKey ? kNoKey - 1 : t;
}

// *wide must be 0 before the launch.  Two picked ids with the same tag are the
// same id unless one of them is wide, so matches are always confirmed here (the
// picked set is small next to the edges).
__device__ __forceinline__ void member_insert_one(const int64_t* __restrict__ picked, int64_t i,
                                                  uint64_t* table, uint32_t cap,
                                                  int* __restrict__ wide, uint32_t* filter) {
  const uint64_t id = (uint64_t)picked[i];
  if (id > kMaxPackedKey) *wide = 1;  // every writer stores the same value
  const uint32_t key = member_tag(id);
  if (filter) atomicOr(filter + filter_word(key), filter_bits(key));
  const uint64_t mine = ((uint64_t)key << 32) | (uint64_t)i;
  uint32_t slot = member_home(key, cap);
  for (uint32_t probes = 0; probes < cap; ++probes) {  // the table has free slots: ends early
    uint64_t cur = __hip_atomic_load(table + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (cur == kEmptySlot) {
      cur = atomicCAS((unsigned long long*)(table + slot), (unsigned long long)kEmptySlot,
                      (unsigned long long)mine);
      if (cur == kEmptySlot) return;
    }
    // a slot only ever holds positions of one id; a repeated id keeps its smallest
    if ((uint32_t)(cur >> 32) == key && (uint64_t)picked[(uint32_t)cur] == id) {
      atomicMin((unsigned long long*)(table + slot), (unsigned long long)mine);
      return;
    }
    if (++slot == cap) slot = 0;
  }
}

__global__ __launch_bounds__(kBlock) void member_insert_kernel(
    const int64_t* __restrict__ picked, int64_t n, uint64_t* table, uint32_t cap,
    int* __restrict__ wide, uint32_t* filter) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  member_insert_one(picked, i, table, cap, wide, filter);
}

// Both in one work-group, for a table small enough (the picked set of a
// layer-wise sampler): clear, barrier, insert.
constexpr int kMemberSetupThreads = 1024;
__global__ __launch_bounds__(kMemberSetupThreads) void member_setup_kernel(
    const int64_t* __restrict__ picked, int64_t n, uint64_t* table, uint32_t cap,
    int* __restrict__ wide) {
  for (uint32_t i = threadIdx.x; i < cap; i += kMemberSetupThreads) table[i] = kEmptySlot;
  if (threadIdx.x == 0) *wide = 0;
  // the table is read and written below by other threads of this work-group
  __threadfence_block();
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += kMemberSetupThreads)
    member_insert_one(picked, i, table, cap, wide, nullptr);
}

// Empties the table and lowers the wide-id flag.
__global__ __launch_bounds__(kBlock) void member_clear_kernel(uint64_t* table, int64_t n,
                                                              int* __restrict__ wide,
                                                              uint32_t* filter) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i == 0) *wide = 0;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  if (filter)
    for (int64_t j = i; j < kFilterWords; j += stride) filter[j] = 0u;
  for (; i < n; i += stride) table[i] = kEmptySlot;
}

// A small table (the picked set of a layer-wise sampler is a few hundred ids)
// is copied into LDS once per work-group, keys and positions apart: 64 lanes
// probing 64 different slots cost the vector cache a tag look-up each, the LDS
// a few cycles in all.
template <bool kInLds, bool kWithValues>
struct MemberTable {
  const uint64_t* slots;
  const uint32_t* keys;
  const uint32_t* values;
  uint32_t cap;

  __device__ __forceinline__ void stage(const uint64_t* __restrict__ table, uint32_t capacity,
                                        uint32_t* lds_keys, uint32_t* lds_values) {
    slots = table;
    keys = lds_keys;
    values = lds_values;
    cap = capacity;
    if (!kInLds) return;
    for (uint32_t i = threadIdx.x; i < capacity; i += blockDim.x) {
      const uint64_t t = table[i];
      lds_keys[i] = (uint32_t)(t >> 32);
      if (kWithValues) lds_values[i] = (uint32_t)t;
    }
    __syncthreads();
  }
  __device__ __forceinline__ uint32_t key_at(uint32_t slot) const {
    return kInLds ? keys[slot] : (uint32_t)(slots[slot] >> 32);
  }
  __device__ __forceinline__ uint32_t value_at(uint32_t slot) const {
    return kInLds ? values[slot] : (uint32_t)slots[slot];
  }

  // N look-ups in step: the probes of a round are issued together, so a lane
  // waits for the longest of its N probe runs instead of their sum.  slot[j]
  // is where key[j] sits, cap when it is absent (or kNoKey).
  template <int N>
  __device__ __forceinline__ void find_many(const uint32_t (&key)[N], uint32_t (&slot)[N]) const {
    uint32_t open = 0;  // bit j: key j is still probing
#pragma unroll
    for (int j = 0; j < N; ++j) {
      slot[j] = cap;
      if (key[j] != kNoKey) {
        slot[j] = member_home(key[j], cap);
        open |= 1u << j;
      }
    }
    for (uint32_t probes = 0; open != 0 && probes < cap; ++probes) {
      uint32_t cur[N];
#pragma unroll
      for (int j = 0; j < N; ++j) cur[j] = (open >> j) & 1u ? key_at(slot[j]) : 0u;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        if (!((open >> j) & 1u)) continue;
        if (cur[j] == key[j]) {
          open &= ~(1u << j);
        } else if (cur[j] == kNoKey) {
          open &= ~(1u << j);
          slot[j] = cap;
        } else if (++slot[j] == cap) {
          slot[j] = 0;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < N; ++j)
      if ((open >> j) & 1u) slot[j] = cap;  // probe budget spent: cannot happen with free slots
  }

  // One look-up whose tag matches are confirmed against the picked ids (the
  // path of picked sets with ids of 2^32 - 1 and above).
  __device__ __forceinline__ uint32_t find_confirmed(uint64_t id,
                                                     const int64_t* __restrict__ picked) const {
    const uint32_t tag = member_tag(id);
    uint32_t slot = member_home(tag, cap);
    for (uint32_t probes = 0; probes < cap; ++probes) {
      const uint32_t cur = key_at(slot);
      if (cur == kNoKey) return cap;
      if (cur == tag && (uint64_t)picked[value_at(slot)] == id) return slot;
      if (++slot == cap) slot = 0;
    }
    return cap;
  }
};

// The same small table, rebuilt in LDS as buckets of four keys: a look-up reads
// one bucket (16 bytes, one instruction) and compares four keys, and goes on to
// the next bucket only from a full one.  With at most two keys per bucket on
// average nearly every look-up ends at its first bucket, where the linear table
// makes a wave repeat its probe loop until the longest of its 256 probe runs
// has ended -- the pass is bound by the instructions it issues.  For picked
// sets whose ids all fit 32 bits (a match of the key is then a match of the id).
constexpr int kMemberBuckets = kMemberLdsSlots / 4;
struct BucketTable {
  const uint4* keys;       // [kMemberBuckets] filled from .x on; kNoKey = free
  const uint32_t* values;  // [kMemberLdsSlots] position in the picked set, by slot

  __device__ __forceinline__ static uint32_t home(uint32_t key) {
    return __umulhi(key * 0x9E3779B1u, (uint32_t)kMemberBuckets);
  }

  // fill: a counter per bucket, only used here
  __device__ __forceinline__ void stage(const uint64_t* __restrict__ table, uint32_t capacity,
                                        uint32_t* lds_keys, uint32_t* lds_values,
                                        uint32_t* fill) {
    keys = reinterpret_cast<const uint4*>(lds_keys);
    values = lds_values;
    for (uint32_t i = threadIdx.x; i < (uint32_t)kMemberLdsSlots; i += blockDim.x)
      lds_keys[i] = kNoKey;
    for (uint32_t i = threadIdx.x; i < (uint32_t)kMemberBuckets; i += blockDim.x) fill[i] = 0;
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < capacity; i += blockDim.x) {
      const uint64_t t = table[i];
      if (t == kEmptySlot) continue;
      const uint32_t key = (uint32_t)(t >> 32);
      uint32_t b = home(key);
      for (int tries = 0; tries < kMemberBuckets; ++tries) {  // fewer keys than slots: ends early
        const uint32_t at = atomicAdd(&fill[b], 1u);
        if (at < 4u) {
          lds_keys[b * 4 + at] = key;
          lds_values[b * 4 + at] = (uint32_t)t;
          break;
        }
        b = (b + 1) & (kMemberBuckets - 1);
      }
    }
    __syncthreads();
  }

  // N look-ups in step; slot[j] is where key[j] sits, kMemberLdsSlots when it
  // is absent (or kNoKey).
  template <int N>
  __device__ __forceinline__ void find_many(const uint32_t (&key)[N], uint32_t (&slot)[N]) const {
    uint32_t b[N];
    uint32_t open = 0;  // bit j: key j goes on to the next bucket
#pragma unroll
    for (int j = 0; j < N; ++j) {
      slot[j] = kMemberLdsSlots;
      b[j] = home(key[j]);
      if (key[j] != kNoKey) open |= 1u << j;
    }
    for (int rounds = 0; open != 0 && rounds < kMemberBuckets; ++rounds) {
      uint4 k[N];
#pragma unroll
      for (int j = 0; j < N; ++j) k[j] = keys[b[j]];
#pragma unroll
      for (int j = 0; j < N; ++j) {
        if (!((open >> j) & 1u)) continue;
        const int hit = k[j].x == key[j] ? 0 : k[j].y == key[j] ? 1 : k[j].z == key[j] ? 2
                        : k[j].w == key[j] ? 3 : -1;
        if (hit >= 0) {
          slot[j] = b[j] * 4 + hit;
          open &= ~(1u << j);
        } else if (k[j].w == kNoKey) {
          open &= ~(1u << j);  // a bucket with room would hold the key
        } else {
          b[j] = (b[j] + 1) & (kMemberBuckets - 1);
        }
      }
    }
  }
};

// kThreads: work-group size.  A large one shares a staged table among more
// edges; a small one spreads a short edge list over all compute units.
// IdT: int64_t, or int32_t when the ids are read from a matrix's narrow copy.
// kView: the edges are those of a column slice read in place.
template <bool kInLds, int kThreads, typename IdT, bool kView>
__global__ __launch_bounds__(kThreads) void member_flag_kernel(
    const IdT* __restrict__ ids, int64_t nnz,
    const uint64_t* __restrict__ global_table, uint32_t cap,
    const int64_t* __restrict__ picked, const int* __restrict__ wide_flag,
    uint64_t* __restrict__ flags, int64_t* __restrict__ chunk_count,
    uint32_t* __restrict__ staged, const uint32_t* __restrict__ filter, SliceView view) {
  __shared__ __align__(16) uint32_t lds_keys[kInLds ? kMemberLdsSlots : 1];
  __shared__ uint32_t lds_values[kInLds ? kMemberLdsSlots : 1];
  __shared__ uint32_t lds_fill[kInLds ? kMemberBuckets : 1];
  __shared__ uint32_t lds_filter[kInLds ? 1 : kFilterWords];
  const bool wide = *wide_flag != 0;  // the same for every thread of the launch
  const bool bucketed = kInLds && !wide;
  const bool filtered = !kInLds && !wide && filter != nullptr;
  if (filtered) {
    for (int i = threadIdx.x; i < kFilterWords; i += kThreads) lds_filter[i] = filter[i];
    __syncthreads();
  }
  MemberTable<kInLds, true> table;
  BucketTable buckets;
  if (bucketed) {
    buckets.stage(global_table, cap, lds_keys, lds_values, lds_fill);
  } else {
    table.stage(global_table, cap, lds_keys, lds_values);
  }
  const uint32_t absent = bucketed ? (uint32_t)kMemberLdsSlots : cap;
  const int64_t num_chunks = ceil_div_dev(nnz, kBlock);
  const int lane = lane_id();
  // A wave takes runs of kMemberChunksPerWave chunks, the work-groups of the
  // launch striding over the runs (a launch with fewer work-groups than runs
  // stages its tables once per work-group, not once per run).
  // The ids of kMemberAhead chunks are requested together, before anything is
  // stored: a store between a load and its use makes the wait for the load
  // (loads and stores count down one in-order counter) a wait for everything.
  const int64_t num_runs = ceil_div_dev(num_chunks, kMemberChunksPerWave);
  for (int64_t run = (int64_t)blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
       run < num_runs; run += (int64_t)gridDim.x * (kThreads / kWave)) {
  // With a view the edges are those of a column slice that was never written:
  // the run's columns are looked up once, on the scalar unit, and an edge's id
  // is read from the parent's array.
  SliceView::Run vrun{};
  vrun.split = INT64_MAX;  // no view: every edge at distance 0, offset 0
  bool scattered = false;  // the same in every lane
  if (kView) {
    const int64_t e_first = run * kMemberChunksPerWave * kBlock;
    const int64_t e_stop = e_first + kMemberChunksPerWave * kBlock;
    vrun = view.run(e_first, (e_stop < nnz ? e_stop : nnz) - 1);
    scattered = !vrun.near();
  }
  // id of edge e, or of the last edge for a lane past the end: on a scattered
  // run the look-up shuffles, so all lanes go through it together
  auto id_of = [&](int64_t e) -> uint64_t {
    if (e >= nnz) e = nnz - 1;
    if (!kView) return (uint64_t)(int64_t)ids[e];
    if (!scattered) return (uint64_t)((int64_t)ids[vrun.place(e)] + vrun.id_offset(e));
    int64_t c, offset;
    const int64_t p = view.position(vrun, e, &c, &offset);
    return (uint64_t)((int64_t)ids[p] + offset);
  };
  for (int part = 0; part < kMemberChunksPerWave / kMemberAhead; ++part) {
    const int64_t chunk0 = run * kMemberChunksPerWave + part * kMemberAhead;
    if (chunk0 >= num_chunks) break;
    uint32_t keys[kMemberAhead][kMemberWords];
    if (!kView || !scattered) {
#pragma unroll
      for (int c = 0; c < kMemberAhead; ++c)
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          const int64_t e = (chunk0 + c) * kBlock + j * kWave + lane;
          keys[c][j] =
              e >= nnz ? kNoKey
              : kView  ? member_key((uint64_t)((int64_t)ids[vrun.place(e)] + vrun.id_offset(e)))
                       : member_key((uint64_t)(int64_t)ids[e]);
        }
    } else {
#pragma unroll
      for (int c = 0; c < kMemberAhead; ++c)
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          const int64_t e = (chunk0 + c) * kBlock + j * kWave + lane;
          const uint64_t id = id_of(e);
          keys[c][j] = e < nnz ? member_key(id) : kNoKey;
        }
    }
    if (filtered) {
#pragma unroll
      for (int c = 0; c < kMemberAhead; ++c)
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          const uint32_t bits = filter_bits(keys[c][j]);
          if ((lds_filter[filter_word(keys[c][j])] & bits) != bits) keys[c][j] = kNoKey;
        }
    }
    // a table in L2 answers after a round trip: the few look-ups that the filter
    // lets through go through their probe rounds together for all chunks of the part
    uint32_t all_slots[kMemberAhead * kMemberWords];
    if (filtered) {
      uint32_t all_keys[kMemberAhead * kMemberWords];
#pragma unroll
      for (int c = 0; c < kMemberAhead; ++c)
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) all_keys[c * kMemberWords + j] = keys[c][j];
      table.find_many(all_keys, all_slots);
    }
#pragma unroll
    for (int c = 0; c < kMemberAhead; ++c) {
      const int64_t chunk = chunk0 + c;
      if (chunk >= num_chunks) break;
      uint32_t slot[kMemberWords];
      uint64_t word[kMemberWords];
      if (bucketed) {
        buckets.find_many(keys[c], slot);
      } else if (!wide) {
        if (!filtered) {
          table.find_many(keys[c], slot);
        } else {
#pragma unroll
          for (int j = 0; j < kMemberWords; ++j) slot[j] = all_slots[c * kMemberWords + j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          const int64_t e = chunk * kBlock + j * kWave + lane;
          const uint64_t id = id_of(e);
          slot[j] = e < nnz ? table.find_confirmed(id, picked) : cap;
        }
      }
#pragma unroll
      for (int j = 0; j < kMemberWords; ++j) word[j] = __ballot(slot[j] < absent);
      {
        int before = 0;  // kept edges of the chunk in front of this row of 64
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          if (slot[j] < absent)
            staged[chunk * kBlock + before + __popcll(word[j] & ((1ull << lane) - 1))] =
                bucketed ? buckets.values[slot[j]] : table.value_at(slot[j]);
          before += __popcll(word[j]);
        }
      }
      if (lane == 0) {
        int total = 0;
#pragma unroll
        for (int j = 0; j < kMemberWords; ++j) {
          flags[chunk * kMemberWords + j] = word[j];
          total += __popcll(word[j]);
        }
        chunk_count[chunk] = total;
        if (chunk == num_chunks - 1) chunk_count[num_chunks] = 0;
      }
    }
  }
  }
}

// Kept edges at positions < e.
__device__ __forceinline__ int64_t member_rank_before(
    int64_t e, const uint64_t* __restrict__ flags,
    const int64_t* __restrict__ chunk_off) {
  const int64_t chunk = e / kBlock;
  int64_t r = chunk_off[chunk];
  const int in_chunk = (int)(e - chunk * kBlock);
  const int full = in_chunk / kWave, rem = in_chunk % kWave;
  for (int w = 0; w < full; ++w) r += __popcll(flags[chunk * kMemberWords + w]);
  if (rem) r += __popcll(flags[chunk * kMemberWords + full] & ((1ull << rem) - 1));
  return r;
}

__global__ __launch_bounds__(kBlock) void member_indptr_kernel(
    const int64_t* __restrict__ indptr, int64_t num_major,
    const uint64_t* __restrict__ flags, const int64_t* __restrict__ chunk_off,
    int64_t nnz, int64_t* __restrict__ out_indptr, int64_t* __restrict__ out_total) {
  const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t num_chunks = ceil_div_dev(nnz, kBlock);
  if (c == 0 && out_total) *out_total = nnz > 0 ? chunk_off[num_chunks] : 0;
  if (indptr == nullptr || c > num_major) return;
  const int64_t e = indptr[c];
  out_indptr[c] = nnz == 0 ? 0
                  : (e >= nnz ? chunk_off[num_chunks] : member_rank_before(e, flags, chunk_off));
}

// A wave writes the kept edges of kMemberChunksPerWave consecutive chunks.  What
// it needs to know about them arrives in one round trip (lane l holds flag word
// l of the wave's chunks, the first lanes also a chunk offset each); the columns
// of the wave's first and last edge take a search each on the scalar unit (one
// column covers the whole span unless columns are short); then the staged ids of all
// chunks of a part are requested together, and only then anything is stored.
// kEdgeMajor: the id on the other axis comes from edge_major (an edge list)
// instead of the compressed pointer.
// kView: the edges are those of a column slice read in place (without it none of
// the view's look-ups is compiled in).
template <bool kEdgeMajor, bool kView>
__global__ __launch_bounds__(kBlock) void member_fill_kernel(
    int64_t nnz, const uint64_t* __restrict__ flags, const int64_t* __restrict__ chunk_off,
    const uint32_t* __restrict__ staged, const int64_t* __restrict__ indptr,
    int64_t num_major, const int64_t* __restrict__ edge_major,
    int64_t* __restrict__ out_major, int64_t* __restrict__ out_minor,
    int64_t* __restrict__ out_select, SliceView view) {
  const int64_t num_chunks = ceil_div_dev(nnz, kBlock);
  const int64_t wave = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  const int lane = lane_id();
  const int64_t first_chunk = wave * kMemberChunksPerWave;
  if (first_chunk >= num_chunks) return;
  const int64_t my_word = first_chunk * kMemberWords + lane;
  const uint64_t lane_word =
      lane < kMemberChunksPerWave * kMemberWords && my_word < num_chunks * kMemberWords
          ? flags[my_word]
          : 0ull;
  const int64_t lane_off =
      lane < kMemberChunksPerWave && first_chunk + lane < num_chunks ? chunk_off[first_chunk + lane]
                                                                    : 0;
  const int64_t e_first = first_chunk * kBlock;
  const int64_t e_end =
      (first_chunk + kMemberChunksPerWave) * kBlock < nnz ? (first_chunk + kMemberChunksPerWave) * kBlock
                                                          : nnz;
  SegmentSpan span{0, 0};
  SliceView::Run vrun{};
  if (kView) {  // indptr is the view's column pointer: one look-up serves both
    vrun = view.run(e_first, e_end - 1);
    span = vrun.span;
  } else if (out_major && !kEdgeMajor) {
    span = segment_span(indptr, num_major, e_first, e_end - 1);
  }
#pragma unroll
  for (int part = 0; part < kMemberChunksPerWave / kMemberAhead; ++part) {
    const int c0 = part * kMemberAhead;
    if (first_chunk + c0 >= num_chunks) return;
    uint32_t minor[kMemberAhead][kMemberWords];
    int64_t major[kMemberAhead][kMemberWords];
#pragma unroll
    for (int c = 0; c < kMemberAhead; ++c) {
      int before = 0;
#pragma unroll
      for (int j = 0; j < kMemberWords; ++j) {
        const uint64_t word =
            __shfl((unsigned long long)lane_word, (c0 + c) * kMemberWords + j, kWave);
        const int64_t e = (first_chunk + c0 + c) * kBlock + j * kWave + lane;
        minor[c][j] = 0;
        major[c][j] = 0;
        if ((word >> lane) & 1ull) {
          minor[c][j] = staged[(first_chunk + c0 + c) * kBlock + before +
                               __popcll(word & ((1ull << lane) - 1))];
          if (kEdgeMajor) major[c][j] = edge_major[e];
        }
        before += __popcll(word);
      }
    }
#pragma unroll
    for (int c = 0; c < kMemberAhead; ++c) {
      const int64_t out0 = __shfl((long long)lane_off, c0 + c, kWave);
      int before = 0;
#pragma unroll
      for (int j = 0; j < kMemberWords; ++j) {
        const uint64_t word =
            __shfl((unsigned long long)lane_word, (c0 + c) * kMemberWords + j, kWave);
        const int64_t e = (first_chunk + c0 + c) * kBlock + j * kWave + lane;
        // with a view: the edge's place in the parent and its column in the slice
        // (on a scattered run the look-up shuffles: all lanes take it, kept or not)
        int64_t parent_pos = 0, slice_col = 0;
        if (kView) {
          const int64_t ec = e < nnz ? e : nnz - 1;
          if (vrun.near()) {
            parent_pos = vrun.place(ec);
            slice_col = vrun.column(ec);
          } else {
            int64_t offset;
            parent_pos = view.position(vrun, ec, &slice_col, &offset);
          }
        }
        if ((word >> lane) & 1ull) {
          const int64_t pos = out0 + before + __popcll(word & ((1ull << lane) - 1));
          out_minor[pos] = (int64_t)minor[c][j];
          if (kView) {
            out_select[pos] = parent_pos;
            if (out_major) out_major[pos] = slice_col;
          } else {
            out_select[pos] = e;
            if (out_major) out_major[pos] = kEdgeMajor ? major[c][j] : span.segment_at(indptr, e);
          }
        }
        before += __popcll(word);
      }
    }
  }
}

}  // namespace gs

extern "C" {

size_t gs_minor_slice_workspace_bytes(int64_t nnz, int64_t num_picked) {
  if (nnz < 0 || num_picked < 0) return 0;
  return gs::carve_member(nullptr, nnz, num_picked).total;
}

static int minor_slice_count_impl(const int64_t* ids, const int32_t* ids32, int64_t nnz,
                                  const int64_t* picked,
                                  int64_t num_picked, const int64_t* indptr,
                                  int64_t num_major, int64_t* out_indptr,
                                  int64_t* out_total, void* workspace,
                                  size_t workspace_bytes, gs_stream_t stream,
                                  gs::SliceView view) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_picked >= 0 && num_major >= 0,
             "minor_slice_count: negative size");
  GS_REQUIRE((nnz == 0 || ids || ids32) && (num_picked == 0 || picked),
             "minor_slice_count: null pointer");
  GS_REQUIRE((indptr == nullptr) == (out_indptr == nullptr),
             "minor_slice_count: indptr and out_indptr go together");
  GS_REQUIRE(out_indptr || out_total, "minor_slice_count: nothing to write");
  // positions among the picked ids are 32-bit values and the table (two slots
  // per id) is addressed with 32-bit arithmetic
  GS_REQUIRE(num_picked < (int64_t(1) << 30),
             "minor_slice_count: at most 2^30 - 1 picked ids, got %lld", (long long)num_picked);
  MemberWs w = carve_member(workspace, nnz, num_picked);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("minor_slice workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  const uint32_t cap = (uint32_t)member_table_slots(num_picked);
  const bool in_lds = cap <= (uint64_t)kMemberLdsSlots;
  uint32_t* filter = !in_lds && num_picked <= kFilterMaxIds ? w.filter : nullptr;
  if (in_lds) {
    GS_LAUNCH("member_insert", s,
              member_setup_kernel<<<dim3(1), dim3(kMemberSetupThreads), 0, s>>>(
                  picked, num_picked, w.table, cap, w.wide));
  } else {
    GS_LAUNCH("member_clear", s,
              member_clear_kernel<<<dim3((unsigned)ceil_div((int64_t)cap, kBlock * 4)),
                                    dim3(kBlock), 0, s>>>(w.table, (int64_t)cap, w.wide, filter));
    GS_LAUNCH("member_insert", s,
              member_insert_kernel<<<dim3((unsigned)ceil_div(num_picked, kBlock)),
                                     dim3(kBlock), 0, s>>>(picked, num_picked,
                                                           w.table, cap, w.wide, filter));
  }
  if (nnz > 0) {
    const bool small = nnz < kMemberSmallEdges;
    const int threads = small ? kBlock : kMemberThreads;
    int64_t blocks = ceil_div(w.chunks, (threads / kWave) * kMemberChunksPerWave);
    // a work-group that stages the 64 KB filter does so once and strides over its runs
    const int64_t resident = (int64_t)(kFilterGroupsPerCu * kMemberThreads / threads) * num_compute_units();
    if (filter && blocks > resident) blocks = resident;
    const dim3 grid((unsigned)blocks);
#define GS_MEMBER_FLAG_AS(LDS, THREADS, IDT, IDS, VIEW)                                       \
  GS_LAUNCH("member_flag", s,                                                                 \
            (member_flag_kernel<LDS, THREADS, IDT, VIEW>)<<<grid, dim3(THREADS), 0, s>>>(     \
                IDS, nnz, w.table, cap, picked, w.wide, w.flags, w.chunk_off, w.staged,       \
                filter, view))
#define GS_MEMBER_FLAG(LDS, THREADS)                                                          \
  do {                                                                                        \
    const bool in_place = view.sub_indptr != nullptr;                                         \
    if (ids32 && in_place) GS_MEMBER_FLAG_AS(LDS, THREADS, int32_t, ids32, true);             \
    else if (ids32) GS_MEMBER_FLAG_AS(LDS, THREADS, int32_t, ids32, false);                   \
    else if (in_place) GS_MEMBER_FLAG_AS(LDS, THREADS, int64_t, ids, true);                   \
    else GS_MEMBER_FLAG_AS(LDS, THREADS, int64_t, ids, false);                                \
  } while (0)
    if (in_lds && small) GS_MEMBER_FLAG(true, kBlock);
    else if (in_lds) GS_MEMBER_FLAG(true, kMemberThreads);
    else if (small) GS_MEMBER_FLAG(false, kBlock);
    else GS_MEMBER_FLAG(false, kMemberThreads);
#undef GS_MEMBER_FLAG
#undef GS_MEMBER_FLAG_AS
    int rc = exclusive_scan_i64(w.chunk_off, w.chunk_off, w.chunks + 1, w.scan_ws,
                                w.scan_ws_bytes, s);
    if (rc != GS_OK) return rc;
  }
  const int64_t n = indptr ? num_major + 1 : 1;
  GS_LAUNCH("member_indptr", s,
            member_indptr_kernel<<<dim3((unsigned)ceil_div(n, kBlock)),
                                   dim3(kBlock), 0, s>>>(indptr, num_major, w.flags,
                                                         w.chunk_off, nnz,
                                                         out_indptr, out_total));
  return GS_OK;
}

static int minor_slice_fill_impl(const int64_t* ids, int64_t nnz, int64_t num_picked,
                                 const int64_t* indptr, int64_t num_major,
                                 const int64_t* edge_major, int64_t* out_major,
                                 int64_t* out_minor, int64_t* out_select,
                                 void* workspace, size_t workspace_bytes,
                                 gs_stream_t stream, gs::SliceView view) {
  using namespace gs;
  GS_REQUIRE(nnz >= 0 && num_picked >= 0 && num_major >= 0,
             "minor_slice_fill: negative size");
  if (nnz == 0) return GS_OK;
  GS_REQUIRE(ids, "minor_slice_fill: null ids");
  GS_REQUIRE(out_major == nullptr || edge_major != nullptr || indptr != nullptr,
             "minor_slice_fill: out_major needs edge_major or indptr");
  MemberWs w = carve_member(workspace, nnz, num_picked);
  if (workspace == nullptr || workspace_bytes < w.total) {
    set_error("minor_slice workspace too small: %zu < %zu", workspace_bytes, w.total);
    return GS_ERR_WORKSPACE;
  }
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)ceil_div(w.chunks, (kBlock / kWave) * kMemberChunksPerWave));
#define GS_MEMBER_FILL(MAJOR, VIEW)                                                    \
  GS_LAUNCH("member_fill", s,                                                          \
            (member_fill_kernel<MAJOR, VIEW>)<<<grid, dim3(kBlock), 0, s>>>(           \
                nnz, w.flags, w.chunk_off, w.staged, indptr, num_major, edge_major,    \
                out_major, out_minor, out_select, view))
  if (view.sub_indptr != nullptr) {
    GS_REQUIRE(!edge_major, "minor_slice_fill: a slice read in place has no edge list");
    GS_MEMBER_FILL(false, true);
  } else if (edge_major) {
    GS_MEMBER_FILL(true, false);
  } else {
    GS_MEMBER_FILL(false, false);
  }
#undef GS_MEMBER_FILL
  return GS_OK;
}

int gs_minor_slice_count(const int64_t* ids, int64_t nnz, const int64_t* picked,
                         int64_t num_picked, const int64_t* indptr,
                         int64_t num_major, int64_t* out_indptr,
                         int64_t* out_total, void* workspace,
                         size_t workspace_bytes, gs_stream_t stream) {
  return minor_slice_count_impl(ids, nullptr, nnz, picked, num_picked, indptr, num_major,
                                out_indptr, out_total, workspace, workspace_bytes, stream,
                                gs::no_view());
}

int gs_minor_slice_fill(const int64_t* ids, int64_t nnz, int64_t num_picked,
                        const int64_t* indptr, int64_t num_major,
                        const int64_t* edge_major, int64_t* out_major,
                        int64_t* out_minor, int64_t* out_select,
                        void* workspace, size_t workspace_bytes,
                        gs_stream_t stream) {
  return minor_slice_fill_impl(ids, nnz, num_picked, indptr, num_major, edge_major, out_major,
                               out_minor, out_select, workspace, workspace_bytes, stream,
                               gs::no_view());
}

static int check_slice_view(const int64_t* indptr, const int64_t* indices, const int64_t* cols,
                            int64_t num_cols_picked, const int64_t* sub_indptr,
                            int64_t slice_nnz, const char* who) {
  using namespace gs;
  GS_REQUIRE(num_cols_picked >= 0 && slice_nnz >= 0, "%s: negative size", who);
  GS_REQUIRE(sub_indptr, "%s: null sub_indptr", who);
  GS_REQUIRE(slice_nnz == 0 || (indptr && indices && cols && num_cols_picked > 0),
             "%s: null pointer", who);
  return GS_OK;
}

int gs_col_row_slice_count(const int64_t* indptr, const int64_t* indices,
                           const int32_t* indices32, const int64_t* cols,
                           const int64_t* key_offset, int64_t num_cols_picked,
                           const int64_t* sub_indptr, int64_t slice_nnz,
                           const int64_t* rows, int64_t num_rows_picked,
                           int64_t* out_indptr, int64_t* out_total, void* workspace,
                           size_t workspace_bytes, gs_stream_t stream) {
  int rc = check_slice_view(indptr, indices, cols, num_cols_picked, sub_indptr, slice_nnz,
                            "col_row_slice_count");
  if (rc != GS_OK) return rc;
  const gs::SliceView view{sub_indptr, cols, indptr, key_offset, num_cols_picked};
  return minor_slice_count_impl(indices, indices32, slice_nnz, rows, num_rows_picked, sub_indptr,
                                num_cols_picked, out_indptr, out_total, workspace,
                                workspace_bytes, stream, view);
}

int gs_col_row_slice_fill(const int64_t* indptr, const int64_t* indices, const int64_t* cols,
                          int64_t num_cols_picked, const int64_t* sub_indptr,
                          int64_t slice_nnz, int64_t num_rows_picked, int64_t* out_major,
                          int64_t* out_minor, int64_t* out_select, void* workspace,
                          size_t workspace_bytes, gs_stream_t stream) {
  int rc = check_slice_view(indptr, indices, cols, num_cols_picked, sub_indptr, slice_nnz,
                            "col_row_slice_fill");
  if (rc != GS_OK) return rc;
  const gs::SliceView view{sub_indptr, cols, indptr, nullptr, num_cols_picked};
  return minor_slice_fill_impl(indices, slice_nnz, num_rows_picked, sub_indptr,
                               num_cols_picked, nullptr, out_major, out_minor, out_select,
                               workspace, workspace_bytes, stream, view);
}

}  // extern "C"
