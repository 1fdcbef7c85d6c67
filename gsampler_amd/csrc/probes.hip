// probes.hip -- yardsticks for the measurements that the gather kernels of this
// library are quoted against: what this GPU delivers to a plain streaming copy,
// and how many scattered 128-byte lines per second it delivers when every lane
// of every wavefront asks for a line of its own (the access pattern behind a
// random pick).  Measurement helpers only; no operator calls them.
#include "common.h"

namespace gs {

// 16 bytes per lane and instruction, four in flight per lane.
constexpr int kCopyItems = 4;
__global__ __launch_bounds__(kBlock) void probe_copy_kernel(const uint4* __restrict__ src,
                                                            uint4* __restrict__ dst, int64_t n) {
  const int64_t base = (int64_t)blockIdx.x * kBlock * kCopyItems + threadIdx.x;
  uint4 v[kCopyItems];
#pragma unroll
  for (int i = 0; i < kCopyItems; ++i) {
    const int64_t j = base + (int64_t)i * kBlock;
    if (j < n) v[i] = src[j];
  }
#pragma unroll
  for (int i = 0; i < kCopyItems; ++i) {
    const int64_t j = base + (int64_t)i * kBlock;
    if (j < n) dst[j] = v[i];
  }
}

// Lane g reads `bytes_per_pick` (4 or 8) bytes from line hash(g, salt) of a table
// of num_lines 128-byte lines; kAhead picks per lane in flight.  The sums go to
// out[lane's first pick] so that the loads are live; `ordered` visits the same
// lines in address order instead (sorted picks: what reuse inside L2 would buy).
constexpr int kPickAhead = 4;
__global__ __launch_bounds__(kBlock) void probe_line_gather_kernel(
    const uint32_t* __restrict__ table, uint64_t num_lines, int64_t num_picks, uint64_t salt,
    int ordered, uint32_t* __restrict__ out) {
  const int64_t g0 = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kPickAhead;
  uint32_t v[kPickAhead];
#pragma unroll
  for (int i = 0; i < kPickAhead; ++i) {
    const int64_t g = g0 + i;
    v[i] = 0;
    if (g >= num_picks) continue;
    uint64_t line;
    if (ordered) {
      line = (uint64_t)(((unsigned __int128)(uint64_t)g * num_lines) / (uint64_t)num_picks);
    } else {
      uint64_t h = ((uint64_t)g + salt) * 0x9E3779B97F4A7C15ull;
      h ^= h >> 29;
      h *= 0xBF58476D1CE4E5B9ull;
      h ^= h >> 32;
      line = __umul64hi(h, num_lines);
    }
    v[i] = table[line * 32 + (uint32_t)(g & 31)];
  }
  uint32_t sum = 0;
#pragma unroll
  for (int i = 0; i < kPickAhead; ++i) sum += v[i];
  if (g0 < num_picks) out[g0 / kPickAhead] = sum;
}

}  // namespace gs

extern "C" {

int gs_probe_stream_copy(const void* src, void* dst, int64_t bytes, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(bytes >= 0 && bytes % 16 == 0, "probe_stream_copy: bytes must be a multiple of 16");
  GS_REQUIRE(bytes == 0 || (src && dst), "probe_stream_copy: null pointer");
  GS_REQUIRE((((uintptr_t)src | (uintptr_t)dst) & 15) == 0, "probe_stream_copy: unaligned pointer");
  if (bytes == 0) return GS_OK;
  const int64_t n = bytes / 16;
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("probe_copy", s,
            probe_copy_kernel<<<dim3((unsigned)ceil_div(n, (int64_t)kBlock * kCopyItems)),
                                dim3(kBlock), 0, s>>>((const uint4*)src, (uint4*)dst, n));
  return GS_OK;
}

int gs_probe_line_gather(const void* table, int64_t table_bytes, int64_t num_picks,
                         uint64_t salt, int ordered, void* out, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(table_bytes >= 128 && num_picks >= 0, "probe_line_gather: bad size");
  GS_REQUIRE(num_picks == 0 || (table && out), "probe_line_gather: null pointer");
  if (num_picks == 0) return GS_OK;
  hipStream_t s = as_stream(stream);
  const int64_t threads = ceil_div(num_picks, (int64_t)kPickAhead);
  GS_LAUNCH("probe_line_gather", s,
            probe_line_gather_kernel<<<dim3((unsigned)ceil_div(threads, (int64_t)kBlock)),
                                       dim3(kBlock), 0, s>>>(
                (const uint32_t*)table, (uint64_t)(table_bytes / 128), num_picks, salt, ordered,
                (uint32_t*)out));
  return GS_OK;
}

}  // extern "C"
