// Per-tile id summaries used by the attention kernels to skip tiles.
//
// The block mask handed in by the caller is authoritative for *what* is attended, but the
// reference heuristic that produces it over-covers when positions restart per document
// (kvax/ops/mask_creator.py:110-115 compares block-wide position extremes), so a kernel that
// visits every tile of [lower, upper) does up to 2x useless work.  A tile can be dropped when
// no (query, key) pair of it can pass the element mask; that is decided conservatively from
// min/max segment id and position of the tile's non-padding rows.  Each tile is summarised in
// two parts -- the rows that share the segment id of its first non-padding row, and the rest --
// so that a tile straddling a document boundary does not look attendable to everything.
#include "common.h"
#include "fa_common.h"

namespace kvax {
namespace {

struct Params {
  TileSummaryJob jobs[2];
};

__global__ __launch_bounds__(256) void tile_summaries_kernel(Params p) {
  const TileSummaryJob& job = p.jobs[blockIdx.z];
  const int lane = threadIdx.x % 64;
  const int n_tiles = (job.len + kTileRows - 1) / kTileRows;
  const int tile = blockIdx.x * 4 + threadIdx.x / 64;
  if (tile >= n_tiles) return;
  const int b = blockIdx.y;
  const int t = tile * kTileRows + lane;
  int32_t seg = -1, pos = 0;
  if (t < job.len) {
    seg = job.seg[(size_t)b * job.len + t];
    pos = job.pos[(size_t)b * job.len + t];
  }
  const TileParts parts = wave_parts(seg != -1, seg, pos);
  if (lane == 0) {
    int4* out = reinterpret_cast<int4*>(job.out) + 2 * ((size_t)b * n_tiles + tile);
    out[0] = parts.a;
    out[1] = parts.b;
  }
}

}  // namespace

int launch_tile_summaries(const TileSummaryJob* jobs, int num_jobs, int batch, hipStream_t stream) {
  static_assert(kTileRows == 64, "one lane per row");
  Params p{};
  int max_tiles = 0;
  for (int i = 0; i < num_jobs; i++) {
    p.jobs[i] = jobs[i];
    max_tiles = max_tiles > cdiv(jobs[i].len, kTileRows) ? max_tiles : cdiv(jobs[i].len, kTileRows);
  }
  if (max_tiles == 0 || batch == 0) return KVAX_OK;
  hipLaunchKernelGGL(tile_summaries_kernel, dim3(cdiv(max_tiles, 4), batch, num_jobs), dim3(256), 0,
                     stream, p);
  return check_launch("tile_summaries_kernel");
}

}  // namespace kvax
