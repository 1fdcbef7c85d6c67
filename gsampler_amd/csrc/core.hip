// core.hip -- error plumbing and the device-wide exclusive scan.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "scan.h"

namespace gs {

static thread_local std::string g_last_error;

void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
}

int hip_fail(hipError_t e, const char* what, const char* file, int line) {
  set_error("HIP error %d (%s) at %s:%d in %s", (int)e, hipGetErrorString(e),
            file, line, what);
  return GS_ERR_HIP;
}

// ------------------------------------------------------------- profiling
namespace {
struct ProfPending {
  const char* name;
  hipEvent_t start, stop;
};
struct ProfTotal {
  std::string name;
  long long calls;
  double ms;
};
std::mutex g_prof_mutex;
bool g_prof_on = false;
std::vector<ProfPending> g_prof_pending;
std::vector<hipEvent_t> g_prof_pool;
std::vector<ProfTotal> g_prof_totals;

hipEvent_t prof_event() {
  if (!g_prof_pool.empty()) {
    hipEvent_t e = g_prof_pool.back();
    g_prof_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}

// Folds finished event pairs into the per-name totals (waits for them).
void prof_drain() {
  for (ProfPending& p : g_prof_pending) {
    float ms = 0.f;
    if (p.start && p.stop && hipEventSynchronize(p.stop) == hipSuccess &&
        hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
      ProfTotal* t = nullptr;
      for (ProfTotal& x : g_prof_totals)
        if (x.name == p.name) t = &x;
      if (!t) {
        g_prof_totals.push_back(ProfTotal{p.name, 0, 0.0});
        t = &g_prof_totals.back();
      }
      t->calls += 1;
      t->ms += ms;
    }
    if (p.start) g_prof_pool.push_back(p.start);
    if (p.stop) g_prof_pool.push_back(p.stop);
  }
  g_prof_pending.clear();
}
}  // namespace

bool profile_enabled() { return g_prof_on; }

void profile_begin(const char* name, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  ProfPending p{name, prof_event(), prof_event()};
  if (p.start) (void)hipEventRecord(p.start, stream);
  g_prof_pending.push_back(p);
}

void profile_end(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  if (g_prof_pending.empty()) return;
  ProfPending& p = g_prof_pending.back();
  if (p.stop) (void)hipEventRecord(p.stop, stream);
  if (g_prof_pending.size() >= 4096) prof_drain();
}

// ------------------------------------------------------------------ scan
// Three launches: per-tile sums, a single-block scan of the tile sums, and a
// per-tile down-sweep.  A tile is kScanTile consecutive values.

__global__ __launch_bounds__(kBlock) void scan_tile_sums_kernel(
    const int64_t* __restrict__ in, int64_t n, int64_t* __restrict__ tile_sums) {
  __shared__ int64_t smem[kBlock / kWave + 1];
  const int64_t base = (int64_t)blockIdx.x * kScanTile + threadIdx.x;
  int64_t s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    const int64_t i = base + k * kBlock;  // the order of an integer sum does not matter
    if (i < n) s += in[i];
  }
  int64_t total;
  block_exclusive_sum(s, smem, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// One block scans `num_tiles` values in place (exclusive), chunk by chunk.
__global__ __launch_bounds__(kBlock) void scan_spine_kernel(int64_t* tile_sums,
                                                            int64_t num_tiles) {
  __shared__ int64_t smem[kBlock / kWave + 1];
  int64_t carry = 0;
  for (int64_t start = 0; start < num_tiles; start += kBlock) {
    int64_t i = start + threadIdx.x;
    int64_t v = i < num_tiles ? tile_sums[i] : 0;
    int64_t total;
    int64_t ex = block_exclusive_sum(v, smem, &total);
    if (i < num_tiles) tile_sums[i] = carry + ex;
    carry += total;
  }
}

// Tile t adds the sums of the tiles before it: already scanned by
// scan_spine_kernel (kSpineDone), or summed here by the tile itself
// (kSpineDone == false, for spines short enough that a launch costs more).
// Inside a tile every wavefront owns a contiguous quarter and walks it in
// rounds of 128 values, two neighbouring values (16 bytes) per lane, so each
// load and store of a wavefront covers one contiguous kilobyte; the running sum
// travels from round to round in a register and the four wavefronts meet once.
constexpr int kScanRounds = kScanItems / 2;
static_assert(kScanItems % 2 == 0, "a lane takes pairs of values");

template <bool kSpineDone>
__global__ __launch_bounds__(kBlock) void scan_down_kernel(
    const int64_t* in, int64_t* out, int64_t n,
    const int64_t* __restrict__ tile_sums, int64_t* last_mirror) {
  __shared__ int64_t smem[kBlock / kWave + 1];
  __shared__ int64_t wave_total[kBlock / kWave];
  struct Pair {
    int64_t v[2];
  };
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int64_t wave0 = (int64_t)blockIdx.x * kScanTile + (int64_t)wave * (kScanTile / (kBlock / kWave));
  Pair held[kScanRounds];
#pragma unroll
  for (int r = 0; r < kScanRounds; ++r) {
    const int64_t i = wave0 + r * (2 * kWave) + 2 * lane;
    held[r] = Pair{{0, 0}};
    if (i + 1 < n)
      __builtin_memcpy(&held[r], in + i, sizeof(Pair));
    else if (i < n)
      held[r].v[0] = in[i];
  }
  int64_t before = 0;
  if (kSpineDone) {
    before = tile_sums[blockIdx.x];
  } else {
    int64_t part = 0;
    for (int64_t t = threadIdx.x; t < (int64_t)blockIdx.x; t += kBlock)
      part += tile_sums[t];
    int64_t ignored = block_exclusive_sum(part, smem, &before);
    (void)ignored;
  }
  // exclusive sums inside the wavefront's quarter
  int64_t ex[kScanRounds];
  int64_t running = 0;
#pragma unroll
  for (int r = 0; r < kScanRounds; ++r) {
    const int64_t own = held[r].v[0] + held[r].v[1];
    const int64_t incl = wave_inclusive_sum(own);
    ex[r] = running + incl - own;
    running += __shfl(incl, kWave - 1, kWave);
  }
  if (lane == 0) wave_total[wave] = running;
  __syncthreads();
  for (int w = 0; w < wave; ++w) before += wave_total[w];
#pragma unroll
  for (int r = 0; r < kScanRounds; ++r) {
    const int64_t i = wave0 + r * (2 * kWave) + 2 * lane;
    const Pair result{{before + ex[r], before + ex[r] + held[r].v[0]}};
    if (i + 1 < n)
      __builtin_memcpy(out + i, &result, sizeof(Pair));
    else if (i < n)
      out[i] = result.v[0];
    if (last_mirror) {
      if (i == n - 1) *last_mirror = result.v[0];
      if (i + 1 == n - 1) *last_mirror = result.v[1];
    }
  }
}

constexpr int64_t kShortSpine = 4096;  // tiles

int num_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

size_t scan_workspace_bytes(int64_t n) {
  int64_t tiles = n > 0 ? ceil_div(n, kScanTile) : 1;
  return align_up((size_t)tiles * sizeof(int64_t), 256);
}

int exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n, void* ws,
                       size_t ws_bytes, hipStream_t stream, bool sums_ready,
                       int64_t* last_mirror) {
  if (n <= 0) return GS_OK;
  if (ws_bytes < scan_workspace_bytes(n) || ws == nullptr) {
    set_error("scan workspace too small: %zu < %zu", ws_bytes,
              scan_workspace_bytes(n));
    return GS_ERR_WORKSPACE;
  }
  int64_t* tile_sums = (int64_t*)ws;
  const int64_t tiles = ceil_div(n, kScanTile);
  if (tiles == 1) {  // nothing before the only tile
    GS_LAUNCH("scan_down", stream,
              scan_down_kernel<false><<<dim3(1), dim3(kBlock), 0, stream>>>(
                  in, out, n, tile_sums, last_mirror));
    return GS_OK;
  }
  if (!sums_ready)
    GS_LAUNCH("scan_tile_sums", stream,
              scan_tile_sums_kernel<<<dim3((unsigned)tiles), dim3(kBlock), 0,
                                      stream>>>(in, n, tile_sums));
  if (tiles <= kShortSpine) {
    GS_LAUNCH("scan_down", stream,
              scan_down_kernel<false><<<dim3((unsigned)tiles), dim3(kBlock), 0,
                                        stream>>>(in, out, n, tile_sums, last_mirror));
    return GS_OK;
  }
  GS_LAUNCH("scan_spine", stream,
            scan_spine_kernel<<<dim3(1), dim3(kBlock), 0, stream>>>(tile_sums,
                                                                    tiles));
  GS_LAUNCH("scan_down", stream,
            scan_down_kernel<true><<<dim3((unsigned)tiles), dim3(kBlock), 0,
                                      stream>>>(in, out, n, tile_sums, last_mirror));
  return GS_OK;
}

// n values from one array to another; the destination may be pinned host memory.
__global__ __launch_bounds__(kBlock) void copy_i64_kernel(const int64_t* __restrict__ src,
                                                          int64_t n, int64_t* __restrict__ dst) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace gs

extern "C" {

int gs_copy_i64(const int64_t* src, int64_t n, int64_t* dst, gs_stream_t stream) {
  using namespace gs;
  GS_REQUIRE(n >= 0, "copy_i64: negative length %lld", (long long)n);
  if (n == 0) return GS_OK;
  GS_REQUIRE(src && dst, "copy_i64: null pointer");
  hipStream_t s = as_stream(stream);
  GS_LAUNCH("copy_i64", s,
            copy_i64_kernel<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, s>>>(src, n,
                                                                                          dst));
  return GS_OK;
}

const char* gs_last_error(void) { return gs::g_last_error.c_str(); }

int gs_abi_version(void) { return 7; }

void gs_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(gs::g_prof_mutex);
  gs::g_prof_on = on != 0;
}

void gs_profile_reset(void) {
  std::lock_guard<std::mutex> lock(gs::g_prof_mutex);
  gs::prof_drain();
  gs::g_prof_totals.clear();
}

int gs_profile_count(void) {
  std::lock_guard<std::mutex> lock(gs::g_prof_mutex);
  gs::prof_drain();
  return (int)gs::g_prof_totals.size();
}

int gs_profile_get(int index, char* name, size_t name_bytes, long long* calls,
                   double* total_ms) {
  std::lock_guard<std::mutex> lock(gs::g_prof_mutex);
  if (index < 0 || index >= (int)gs::g_prof_totals.size()) {
    gs::set_error("profile_get: index %d out of range", index);
    return GS_ERR_INVALID;
  }
  const auto& t = gs::g_prof_totals[(size_t)index];
  if (name && name_bytes > 0) {
    strncpy(name, t.name.c_str(), name_bytes - 1);
    name[name_bytes - 1] = 0;
  }
  if (calls) *calls = t.calls;
  if (total_ms) *total_ms = t.ms;
  return GS_OK;
}

size_t gs_scan_workspace_bytes(int64_t n) { return gs::scan_workspace_bytes(n); }

int gs_exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n,
                          void* workspace, size_t workspace_bytes,
                          gs_stream_t stream) {
  GS_REQUIRE(n >= 0, "scan: negative length %lld", (long long)n);
  GS_REQUIRE(n == 0 || (in && out), "scan: null pointer");
  return gs::exclusive_scan_i64(in, out, n, workspace, workspace_bytes,
                                gs::as_stream(stream));
}

}  // extern "C"
