// Shared host-side helpers for the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>

#include "kvax_amd.h"

namespace kvax {

// Records a formatted message for kvax_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(KVAX_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return KVAX_OK;
}

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// Rows per streamed LDS tile in the attention kernels, and the granularity of the tile summaries.
constexpr int kTileRows = 64;

// Enqueues the tile-summary kernel: for every kTileRows-row tile of a [batch, len] id pair writes
// two int4 {seg_min, seg_max, pos_min, pos_max} (rows sharing the segment id of the tile's first
// non-padding row; all other non-padding rows) to out[batch][n_tiles][2]; an empty part is
// {INT_MAX, INT_MIN, INT_MAX, INT_MIN}.  Up to two sequences per launch.
struct TileSummaryJob {
  const int32_t* pos;
  const int32_t* seg;
  void* out;  // int4 [batch, cdiv(len, kTileRows), 2]
  int len;
};
int launch_tile_summaries(const TileSummaryJob* jobs, int num_jobs, int batch, hipStream_t stream);
inline size_t tile_summary_bytes(int batch, int len) {
  return (size_t)batch * cdiv(len, kTileRows) * 32;
}

}  // namespace kvax
