// scan.h -- device-wide exclusive prefix sum over int64 (internal interface).
#ifndef GSAMPLER_CSRC_SCAN_H_
#define GSAMPLER_CSRC_SCAN_H_

#include "common.h"

namespace gs {

constexpr int kScanItems = 8;                    // values per thread
constexpr int kScanTile = kBlock * kScanItems;   // values per block

size_t scan_workspace_bytes(int64_t n);
// in == out is allowed.  Runs on `stream`, never synchronises.
int exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n, void* ws,
                       size_t ws_bytes, hipStream_t stream);

}  // namespace gs

#endif  // GSAMPLER_CSRC_SCAN_H_
