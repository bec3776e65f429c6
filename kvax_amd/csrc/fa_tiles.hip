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
  int32_t* zero;  // counters to clear (one per batch row, then kQueueCounters more), or null
};

__global__ __launch_bounds__(256) void tile_summaries_kernel(Params p) {
  const TileSummaryJob& job = p.jobs[blockIdx.z];
  const int lane = threadIdx.x % 64;
  if (p.zero && blockIdx.x == 0 && blockIdx.z == 0) {
    if (threadIdx.x == 0) p.zero[blockIdx.y] = 0;
    if (blockIdx.y == 0 && threadIdx.x < kQueueCounters) p.zero[gridDim.y + threadIdx.x] = 0;
  }
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

__device__ __forceinline__ const int4* summaries_of(const void* base, int b, int n_tiles) {
  return reinterpret_cast<const int4*>(base) + 2 * (size_t)b * n_tiles;
}

// One wavefront per work item counts the opposing tiles the item can interact with; the last
// work-group of a batch row to finish (arrival counter) then ranks the row's items: the rank of an
// item is the number of items that go before it.
__global__ __launch_bounds__(256) void tile_order_kernel(TileOrderJob job, int batch) {
  __shared__ int is_last;
  const int lane = threadIdx.x % 64;
  const int item = blockIdx.x * 4 + threadIdx.x / 64;
  const int b = blockIdx.y;
  int32_t* order = job.ws + (size_t)b * job.n_items;
  int32_t* work = job.ws + (size_t)batch * job.n_items + (size_t)b * job.n_items;
  int32_t* counter = job.ws + (size_t)batch * 2 * job.n_items + b;
  if (item < job.n_items) {
    const int4* own = summaries_of(job.own, b, job.n_own);
    const int4* opp = summaries_of(job.opp, b, job.n_opp);
    constexpr int kMaxSub = 4;
    TileParts mine[kMaxSub];
#pragma unroll
    for (int s = 0; s < kMaxSub; s++) {
      const int t = item * job.sub + s;
      const bool have = s < job.sub && t < job.n_own;
      mine[s].a = have ? own[2 * t] : empty_summary();
      mine[s].b = have ? own[2 * t + 1] : empty_summary();
    }
    int count = 0;
#pragma unroll 4
    for (int t = lane; t < job.n_opp; t += 64) {
      TileParts other;
      other.a = opp[2 * t];
      other.b = opp[2 * t + 1];
      bool live = false;
#pragma unroll
      for (int s = 0; s < kMaxSub; s++)
        live |= job.own_is_query ? !parts_cannot_attend(mine[s], other) : !parts_cannot_attend(other, mine[s]);
      count += live;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) count += __shfl_xor(count, off);
    if (lane == 0) {
      __hip_atomic_store(work + item, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __threadfence();  // the count is visible device-wide before this work-group's arrival is
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) is_last = atomicAdd(counter, 1) == (int)gridDim.x - 1;
  __syncthreads();
  if (!is_last) return;
  __threadfence();
  // Heavy items (work above the row's mean) keep their index order: neighbours stream the same
  // tiles of the other sequence at about the same time, which is what keeps those tiles in L2, and
  // they carry most of the traffic.  Light items follow by decreasing work and fill the gaps at the
  // end of the launch.
  // Both rules in one sort key (unique per item): heavy items index, light items
  // n * (1 + max work - work) + index; the rank of an item is the number of smaller keys.
  extern __shared__ __attribute__((aligned(16))) int keys[];  // n_items values, padded to a multiple of 4
  __shared__ int total;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int part = 0;
  for (int i = threadIdx.x; i < job.n_items; i += 256) {
    keys[i] = __hip_atomic_load(work + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    part += keys[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
  if (lane == 0) atomicAdd(&total, part);
  __syncthreads();
  const int light_max = total / job.n_items;  // work <= this: light
  const int padded = (job.n_items + 3) & ~3;
  for (int i = threadIdx.x; i < padded; i += 256) {
    const int w = i < job.n_items ? keys[i] : 0;
    int key = 0x7fffffff;  // padding: larger than every real key
    if (i < job.n_items) key = w > light_max ? i : job.n_items * (1 + job.n_opp - w) + i;
    keys[i] = key;  // same thread read keys[i] above
  }
  __syncthreads();
  for (int i = threadIdx.x; i < job.n_items; i += 256) {
    const int mine = keys[i];
    int rank = 0;
#pragma unroll 4
    for (int j = 0; j < padded; j += 4) {
      const int4 k = *reinterpret_cast<const int4*>(keys + j);
      rank += (k.x < mine) + (k.y < mine) + (k.z < mine) + (k.w < mine);
    }
    // an item without any work (it ranks among the last) is marked, so that its consumer need not find out
    order[rank] = mine == job.n_items * (1 + job.n_opp) + i ? i | kDeadItem : i;
  }
}

// See TileListJob.  One work-group per (item, batch row) with the item's wavefronts, each taking the 32
// rows it owns in the attention kernels.
template <int NW>
__global__ __launch_bounds__(NW * 64) void tile_lists_kernel(TileListJob job) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int item = blockIdx.x, b = blockIdx.y;
  constexpr int kRows = NW * 32;
  const int q0 = item * kRows;
  // range of the item: union of [lower, upper) over its mask blocks, intersection of the full ranges
  int lo = 0x7fffffff, hi = 0, flo = 0, fhi = 0x7fffffff;
  {
    const int qb0 = q0 / job.qbs, qb1 = min((q0 + kRows - 1) / job.qbs, job.n_qblocks - 1);
    for (int qb = qb0; qb <= qb1; qb++) {
      const int64_t mi = (int64_t)b * job.n_qblocks + qb;
      const int l_ = job.mask[0][mi] * job.kbs, u_ = job.mask[1][mi] * job.kbs;
      flo = max(flo, job.mask[2][mi] * job.kbs);
      fhi = min(fhi, job.mask[3][mi] * job.kbs);
      if (u_ > l_) {
        lo = min(lo, l_);
        hi = max(hi, u_);
      }
    }
  }
  hi = min(hi, job.kv_len);
  const int t_lo = lo / kTileRows;
  const int t_hi = hi > lo ? (hi + kTileRows - 1) / kTileRows : t_lo;
  const int tf_lo = (flo + kTileRows - 1) / kTileRows, tf_hi = fhi / kTileRows;

  // the wavefront's rows (both half-waves hold the same 32)
  const int row = q0 + wave * 32 + lane % 32;
  const bool in = row < job.q_len;
  const int qi = in ? row : 0;
  const int seg = job.q_seg[(int64_t)b * job.q_len + qi], pos = job.q_pos[(int64_t)b * job.q_len + qi];
  const int64_t mi = (int64_t)b * job.n_qblocks + qi / job.qbs;
  const int col_lo = job.mask[0][mi] * job.kbs;
  const int col_width = max(min(job.mask[1][mi] * job.kbs, job.kv_len) - col_lo, 0);
  const int4* kv_summaries = reinterpret_cast<const int4*>(job.kv_tiles) + 2 * (int64_t)b * job.n_kv_tiles;
  const WordSummaries first_word = load_word_summaries(kv_summaries, t_lo >> 6, t_lo, t_hi, lane);
  TileParts mine[1];
  mine[0] = wave_parts(in && seg != -1 && col_width > 0, seg, pos);

  int* live_count = reinterpret_cast<int*>(smem);
  unsigned long long* live_bits = reinterpret_cast<unsigned long long*>(smem + 16);
  const int word0 = t_lo >> 6;
  const int words = t_hi > t_lo ? ((t_hi - 1) >> 6) - word0 + 1 : 0;
  uint32_t* live_list = reinterpret_cast<uint32_t*>(live_bits + NW * (cdiv_dev(job.n_kv_tiles, 64) + 1));
  mark_live_tiles<true, 1>(kv_summaries, mine, t_lo, t_hi, live_bits + wave * words, word0, lane, first_word);
  __syncthreads();
  if (wave == 0) compact_live_tiles<NW>(live_bits, words, word0, live_list, live_count, lane);
  __syncthreads();
  const int n = *live_count;
  uint32_t* out = job.lists + ((size_t)b * gridDim.x + item) * tile_list_stride(job.n_kv_tiles);
  if (threadIdx.x == 0)
    *reinterpret_cast<uint4*>(out) = make_uint4((uint32_t)n, (uint32_t)tf_lo, (uint32_t)tf_hi, 0u);
  for (int j = threadIdx.x; j < n; j += NW * 64) out[4 + j] = live_list[j];
}

}  // namespace

int launch_tile_lists(const TileListJob& job, int batch, hipStream_t stream) {
  if (job.waves != 4 && job.waves != 8) return fail(KVAX_EINVAL, "tile lists for items of %d wavefronts", job.waves);
  const int items = cdiv(job.q_len, job.waves * 32);
  if (items == 0 || batch == 0) return KVAX_OK;
  const int smem = live_tiles_bytes(job.waves, job.n_kv_tiles);
  if (smem > kLdsPerCu)
    return fail(KVAX_EUNSUPPORTED, "kv_len %d needs %d bytes of LDS for tile bitmaps (limit %d)", job.kv_len, smem, kLdsPerCu);
  if (job.waves == 4) {
    static LdsReservation reservation;
    if (int rc = reservation.ensure(tile_lists_kernel<4>, kLdsPerCu, "the tile list kernel")) return rc;
    hipLaunchKernelGGL(tile_lists_kernel<4>, dim3(items, batch), dim3(256), smem, stream, job);
  } else {
    static LdsReservation reservation;
    if (int rc = reservation.ensure(tile_lists_kernel<8>, kLdsPerCu, "the tile list kernel")) return rc;
    hipLaunchKernelGGL(tile_lists_kernel<8>, dim3(items, batch), dim3(512), smem, stream, job);
  }
  return check_launch("tile_lists_kernel");
}

int launch_tile_order(const TileOrderJob& job, int batch, hipStream_t stream) {
  if (job.sub < 1 || job.sub > 4) return fail(KVAX_EINVAL, "work items of %d tiles", job.sub);
  // the sort keys must fit 31 bits
  if (job.n_items > kMaxOrderedItems || (int64_t)job.n_items * (job.n_opp + 2) >= 0x7fffffff)
    return fail(KVAX_EINVAL, "%d work items over %d tiles to order", job.n_items, job.n_opp);
  if (job.n_items == 0 || batch == 0) return KVAX_OK;
  hipLaunchKernelGGL(tile_order_kernel, dim3(cdiv(job.n_items, 4), batch), dim3(256),
                     (job.n_items + 3) / 4 * 4 * sizeof(int), stream, job, batch);
  return check_launch("tile_order_kernel");
}

int launch_tile_summaries(const TileSummaryJob* jobs, int num_jobs, int batch, hipStream_t stream,
                          int32_t* zero) {
  static_assert(kTileRows == 64, "one lane per row");
  Params p{};
  p.zero = zero;
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
