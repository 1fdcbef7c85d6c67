// scan.h -- device-wide exclusive prefix sum over int64 (internal interface).
#ifndef GSAMPLER_CSRC_SCAN_H_
#define GSAMPLER_CSRC_SCAN_H_

#include "common.h"

namespace gs {

constexpr int kScanItems = 8;                    // values per thread
constexpr int kScanTile = kBlock * kScanItems;   // values per block

size_t scan_workspace_bytes(int64_t n);
// in == out is allowed.  Runs on `stream`, never synchronises.
//   sums_ready   the producer of `in` has already left the sum of every tile of
//                kScanTile consecutive values in the workspace (tile t covers
//                values [t * kScanTile, (t + 1) * kScanTile)), so the pass
//                that adds them up is skipped
//   last_mirror  nullable; also receives out[n - 1] (may be pinned host memory)
int exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n, void* ws,
                       size_t ws_bytes, hipStream_t stream, bool sums_ready = false,
                       int64_t* last_mirror = nullptr);

}  // namespace gs

#endif  // GSAMPLER_CSRC_SCAN_H_
