// hashtable.h -- open-addressing table of packed 64-bit slots shared by the
// unique/relabel and membership (row slicing) kernels.
//
// A slot is  key << 32 | value  (key and value < 2^32 - 1), the empty slot is
// all ones.  Insertion with "smallest value wins" is one 64-bit atomicMin on
// the slot once the key owns it; probing is linear so that a probe run stays
// inside one 128-byte line most of the time.  Capacity is any positive number
// (the home slot is a multiply-shift range reduction, not a mask).
#ifndef GSAMPLER_CSRC_HASHTABLE_H_
#define GSAMPLER_CSRC_HASHTABLE_H_

#include "common.h"

namespace gs {

constexpr uint64_t kEmptySlot = ~0ull;
constexpr uint64_t kMaxPackedKey = 0xFFFFFFFEull;

__device__ __forceinline__ uint32_t hash32(uint64_t key) {
  return (uint32_t)((key * 0x9E3779B97F4A7C15ull) >> 32);
}

__device__ __forceinline__ uint64_t home_slot(uint64_t key, uint64_t cap) {
  return ((uint64_t)hash32(key) * cap) >> 32;
}

// Inserts (key, value), keeping the smallest value per key.  Returns whether
// this value was the smallest seen for the key at that moment (false means a
// smaller one is already there, for good: values only ever decrease).  The
// probe budget (cap) only guards against a table too small for its keys.
__device__ __forceinline__ bool table_insert_min(uint64_t* tab, uint64_t cap,
                                                 uint64_t key, uint64_t value) {
  const uint64_t mine = (key << 32) | value;
  uint64_t slot = home_slot(key, cap);
  for (uint64_t probes = 0; probes < cap; ++probes) {
    uint64_t cur = tab[slot];
    if (cur == kEmptySlot) {
      cur = atomicCAS((unsigned long long*)(tab + slot),
                      (unsigned long long)kEmptySlot, (unsigned long long)mine);
      if (cur == kEmptySlot) return true;
    }
    if ((cur >> 32) == key) {
      // a stale read can only cost an atomic, never a wrong answer
      if (cur < mine) return false;
      const uint64_t old =
          atomicMin((unsigned long long*)(tab + slot), (unsigned long long)mine);
      return old >= mine;
    }
    if (++slot == cap) slot = 0;
  }
  return true;
}

// Slot that holds `key`, or cap when the key is absent.
__device__ __forceinline__ uint64_t table_find(const uint64_t* tab, uint64_t cap,
                                               uint64_t key) {
  uint64_t slot = home_slot(key, cap);
  for (uint64_t probes = 0; probes < cap; ++probes) {
    const uint64_t cur = tab[slot];
    if ((cur >> 32) == key) return slot;
    if (cur == kEmptySlot) return cap;
    if (++slot == cap) slot = 0;
  }
  return cap;
}

// Fills n 64-bit words (table initialisation; also used instead of
// hipMemsetAsync so that callers may capture the launches in a HIP graph).
// A template only so that every translation unit instantiates its own copy.
template <int kUnused = 0>
__global__ __launch_bounds__(kBlock) void table_fill_kernel(uint64_t* table,
                                                            int64_t n,
                                                            uint64_t value) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (; i < n; i += stride) table[i] = value;
}

}  // namespace gs

#endif  // GSAMPLER_CSRC_HASHTABLE_H_
