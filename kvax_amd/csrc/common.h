// Shared host-side helpers for the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <mutex>

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

// Raises a kernel's dynamic LDS limit once per device, safely under concurrent host threads: the
// first caller on a device sets the attribute, every caller gets the result of that attempt.  One
// static instance per kernel instantiation.
class LdsReservation {
 public:
  template <class K>
  int ensure(K kernel, int bytes, const char* what) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
      return fail(KVAX_ELAUNCH, "cannot identify the current device for %s", what);
    PerDevice& d = per_device_[dev];
    std::call_once(d.once, [&] {
      d.status = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    });
    if (d.status != hipSuccess)
      return fail(KVAX_ELAUNCH, "cannot reserve %d bytes of LDS for %s: %s", bytes, what,
                  hipGetErrorString(d.status));
    return KVAX_OK;
  }

 private:
  static constexpr int kMaxDevices = 64;
  struct PerDevice {
    std::once_flag once;
    hipError_t status = hipSuccess;
  };
  PerDevice per_device_[kMaxDevices];
};

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
// `zero` (optional): `batch` + kQueueCounters int32 counters the kernel clears: the arrival counters
// of a following launch_tile_order() and the item queues of the dK/dV kernel (one per XCD).
constexpr int kQueueCounters = 8;
int launch_tile_summaries(const TileSummaryJob* jobs, int num_jobs, int batch, hipStream_t stream,
                          int32_t* zero = nullptr);
inline size_t tile_summary_bytes(int batch, int len) {
  return (size_t)batch * cdiv(len, kTileRows) * 32;
}


// Live-tile lists, built once per call for all query heads.  For every (batch row, item of
// `rows_per_item` = 32 * waves query rows) the kernel merges the block-mask ranges of the mask blocks
// the item covers, tests the kv tiles of the range against the id summaries of each wavefront's 32
// rows and writes the tiles that are live for at least one wavefront, in ascending order:
//   list[0] = number of entries, list[1], list[2] = first tile and end of the mask-free tile range,
//   list[4 + j] = tile index | (mask of the wavefronts it is live for) << 24
// (the same list serves every query head of the batch row).  Only the wide forward kernel reads these
// lists; the other attention kernels work theirs out in LDS per work-group, which measured the same.
// Lists are `tile_list_stride(n_kv_tiles)` words apart.
struct TileListJob {
  const int32_t* q_pos;
  const int32_t* q_seg;
  const int32_t* mask[4];  // lower, upper, lower_full, upper_full over the query blocks, [batch, n_qblocks]
  const void* kv_tiles;    // summaries of the kv sequence, int4 [batch, n_kv_tiles, 2]
  uint32_t* lists;         // out: [batch, cdiv(q_len, rows_per_item), tile_list_stride]
  int q_len, kv_len;
  int qbs, kbs;            // block sizes of the mask along the query and the kv axis
  int n_qblocks, n_kv_tiles;
  int waves;               // wavefronts per item: 4 or 8
};
int launch_tile_lists(const TileListJob& job, int batch, hipStream_t stream);
__host__ __device__ inline size_t tile_list_stride(int n_kv_tiles) { return (size_t)(4 + n_kv_tiles + 3) / 4 * 4; }
inline size_t tile_list_bytes(int batch, int q_len, int rows_per_item, int kv_len) {
  return (size_t)batch * cdiv(q_len, rows_per_item) * tile_list_stride(cdiv(kv_len, kTileRows)) * sizeof(uint32_t);
}
// Above this size the lists are not built and a call that asks for the wide forward kernel runs the
// default one (the size grows with q_len * kv_len / 16384 * 4 bytes: 0.26 MB for 32k x 32k).
#ifndef KVAX_MAX_TILE_LIST_MB
#define KVAX_MAX_TILE_LIST_MB 64
#endif
constexpr size_t kMaxTileListBytes = (size_t)KVAX_MAX_TILE_LIST_MB << 20;

// Work-item ordering.  A work item is `sub` consecutive tiles of one sequence (the rows one
// work-group owns); its work is the number of tiles of the other sequence that at least one of its
// tiles can interact with according to the summaries.  Writes, per batch row, the dispatch order of
// the items: those with more than the row's mean work in index order, then the others by decreasing
// work (ties: lower index first), so that the launch ends on short items; entries of items whose
// work is zero carry the flag kDeadItem.  One launch; `ws` holds
// the order (the result, int32 [batch, n_items], at the start), then the work counts, one
// arrival counter per batch row and kQueueCounters item counters for the kernel that consumes the
// order, all of which launch_tile_summaries() must have zeroed (pass it tile_order_counters(ws, ...)).
constexpr int kDeadItem = 1 << 30;  // flag on an entry of the order: the item's work count is zero
struct TileOrderJob {
  const void* own;   // summaries of the items' sequence, int4 [batch, n_own, 2]
  const void* opp;   // summaries of the streamed sequence, int4 [batch, n_opp, 2]
  int32_t* ws;       // tile_order_bytes(batch, n_items)
  int n_own, n_opp, sub, n_items;
  int own_is_query;  // the items are query rows or key rows
};
int launch_tile_order(const TileOrderJob& job, int batch, hipStream_t stream);
inline size_t tile_order_bytes(int batch, int n_items) {
  return (((size_t)batch * (2 * n_items + 1) + kQueueCounters) * sizeof(int32_t) + 15) / 16 * 16;
}
inline int32_t* tile_order_counters(int32_t* ws, int batch, int n_items) {
  return ws + (size_t)batch * 2 * n_items;
}
// Below this many items per batch row the dispatch order is left alone (decode, short prompts).
constexpr int kMinOrderedItems = 16;
// Above this many the ranking no longer fits the order kernel's LDS (and its cost is quadratic).
constexpr int kMaxOrderedItems = 8192;

}  // namespace kvax
