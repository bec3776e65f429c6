// Block-mask builder for gfx950.
//
// Function computed: reference kvax/ops/mask_creator.py:26-152 (device loop) plus the host
// wrapper around it (:212-259, :317-333), bit for bit.  Algorithm: not the reference's.  Every
// quantity the reference loop uses is a per-block minimum or maximum, so the mask is a function
// of four int32 summaries per block:
//
//   pass 1  block_summaries_kernel   one wavefront per block: coalesced reads of positions and
//                                    segment ids, butterfly min/max across the 64 lanes,
//                                    one int4 {seg_min, seg_max, pos_min, pos_max} per block;
//   pass 2  block_bounds_kernel      one wavefront per outer block: lane i tests inner block
//                                    64*c + i, a wave ballot turns the 64 verdicts into a bit
//                                    mask, first/last set bit give lower/upper (and the same
//                                    for the "full" predicate); sentinel fix-ups applied in
//                                    place.
//
// Work is O(S + n_outer * n_inner / 64) instead of the reference's O(n_outer * S) re-reads.
#include "common.h"

namespace kvax {
namespace {

constexpr int kWave = 64;
constexpr int kWavesPerGroup = 4;
constexpr int32_t kInt32Max = 0x7fffffff;
constexpr int32_t kInt32Min = -kInt32Max - 1;

struct SummaryJob {
  const int32_t* pos;  // [batch, len]
  const int32_t* seg;
  int4* out;           // [batch, n_blocks]
  int len;
  int block_size;
  int n_blocks;
  int32_t pos_fill;    // position given to virtual tail padding
};

struct SummaryParams {
  SummaryJob jobs[2 * KVAX_MAX_MASKS];
  int num_jobs;
  int32_t pad_id;  // segment id that replaces -1
};

__device__ __forceinline__ int32_t wave_min(int32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = min(v, __shfl_xor(v, off));
  return v;
}
__device__ __forceinline__ int32_t wave_max(int32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off));
  return v;
}

// grid: (ceil(max_blocks / kWavesPerGroup), batch, num_jobs)
__global__ __launch_bounds__(kWave* kWavesPerGroup) void block_summaries_kernel(SummaryParams p) {
  const SummaryJob& job = p.jobs[blockIdx.z];
  const int lane = threadIdx.x % kWave;
  const int block = blockIdx.x * kWavesPerGroup + threadIdx.x / kWave;
  if (block >= job.n_blocks) return;
  const int b = blockIdx.y;
  const int32_t* pos = job.pos + (size_t)b * job.len;
  const int32_t* seg = job.seg + (size_t)b * job.len;
  const int start = block * job.block_size;
  int32_t smin = kInt32Max, smax = kInt32Min, pmin = kInt32Max, pmax = kInt32Min;
  for (int i = lane; i < job.block_size; i += kWave) {
    const int t = start + i;
    int32_t s = -1, q = job.pos_fill;
    if (t < job.len) {
      s = seg[t];
      q = pos[t];
    }
    if (s == -1) s = p.pad_id;
    smin = min(smin, s);
    smax = max(smax, s);
    pmin = min(pmin, q);
    pmax = max(pmax, q);
  }
  smin = wave_min(smin);
  smax = wave_max(smax);
  pmin = wave_min(pmin);
  pmax = wave_max(pmax);
  if (lane == 0) job.out[(size_t)b * job.n_blocks + block] = make_int4(smin, smax, pmin, pmax);
}

struct BoundsJob {
  const int4* outer;  // [batch, n_outer]
  const int4* inner;  // [batch, n_inner_total]
  int32_t* lower;
  int32_t* upper;
  int32_t* lower_full;
  int32_t* upper_full;
  int n_outer;
  int n_inner_total;  // inner blocks per batch row (all shards)
  int num_shards;     // >1 only for kv-outer masks under context parallelism
  int kv_outer;
};

struct BoundsParams {
  BoundsJob jobs[KVAX_MAX_MASKS];
  int num_jobs;
  int32_t pad_id;
  int skip_pad;
};

// grid: (ceil(max_outer / kWavesPerGroup), batch * max_shards, num_jobs)
__global__ __launch_bounds__(kWave* kWavesPerGroup) void block_bounds_kernel(BoundsParams p, int max_shards) {
  const BoundsJob& job = p.jobs[blockIdx.z];
  const int lane = threadIdx.x % kWave;
  const int o = blockIdx.x * kWavesPerGroup + threadIdx.x / kWave;
  const int b = blockIdx.y / max_shards;
  const int shard = blockIdx.y % max_shards;
  if (o >= job.n_outer || shard >= job.num_shards) return;
  const int n_inner = job.n_inner_total / job.num_shards;
  const int4 os = job.outer[(size_t)b * job.n_outer + o];
  const int4* inner = job.inner + (size_t)b * job.n_inner_total + (size_t)shard * n_inner;
  const bool osame = os.x == os.y;
  int lower = n_inner, upper = 0, lower_full = n_inner, upper_full = 0;
  if (p.skip_pad && osame && os.x == p.pad_id) {
    lower = upper = lower_full = upper_full = 0;
  } else {
    for (int base = 0; base < n_inner; base += kWave) {
      const int i = base + lane;
      bool attend = false, full = false;
      if (i < n_inner) {
        const int4 is = inner[i];
        const bool seg_overlap = is.x <= os.y && os.x <= is.y;
        bool attend_pos, full_pos;
        if (!job.kv_outer) {
          attend_pos = os.w >= is.z;  // max query position >= min kv position
          full_pos = os.z >= is.w;    // min query position >= max kv position
        } else {
          attend_pos = is.w >= os.z;
          full_pos = is.z >= os.w;
        }
        attend = attend_pos && seg_overlap;
        if (p.skip_pad && is.x == p.pad_id) attend = false;
        full = osame && (is.x == is.y) && full_pos && attend;
      }
      const unsigned long long am = __ballot(attend);
      const unsigned long long fm = __ballot(full);
      if (am) {
        lower = min(lower, base + (int)__ffsll((long long)am) - 1);
        upper = max(upper, base + 64 - (int)__clzll((long long)am));
      }
      if (fm) {
        lower_full = min(lower_full, base + (int)__ffsll((long long)fm) - 1);
        upper_full = max(upper_full, base + 64 - (int)__clzll((long long)fm));
      }
    }
  }
  if (lower == n_inner) lower = upper;
  if (lower_full == n_inner) lower_full = job.kv_outer ? upper : lower;
  if (upper_full < lower_full) upper_full = lower_full;
  if (lane == 0) {
    const size_t idx = ((size_t)b * job.num_shards + shard) * job.n_outer + o;
    job.lower[idx] = lower;
    job.upper[idx] = upper;
    job.lower_full[idx] = lower_full;
    job.upper_full[idx] = upper_full;
  }
}

struct SummaryKey {
  bool kv;
  int block_size;
  int n_blocks;
  size_t offset;  // in int4 units inside the workspace
};

// Distinct (sequence, block size) pairs needed by the masks; returns total int4 count per batch.
int plan_summaries(int q_len, int kv_len, const kvax_mask_desc* masks, int num_masks,
                   SummaryKey* keys, int* q_key, int* kv_key, size_t batch, size_t* total) {
  int n = 0;
  size_t off = 0;
  for (int m = 0; m < num_masks; m++) {
    for (int side = 0; side < 2; side++) {
      const bool kv = side == 1;
      const int bs = kv ? masks[m].kv_block_size : masks[m].query_block_size;
      int found = -1;
      for (int k = 0; k < n; k++)
        if (keys[k].kv == kv && keys[k].block_size == bs) found = k;
      if (found < 0) {
        found = n++;
        keys[found] = {kv, bs, cdiv(kv ? kv_len : q_len, bs), off};
        off += batch * (size_t)keys[found].n_blocks;
      }
      (kv ? kv_key : q_key)[m] = found;
    }
  }
  *total = off;
  return n;
}

int validate(int batch, int q_len, int kv_len, const kvax_mask_desc* masks, int num_masks) {
  if (batch < 0 || q_len < 0 || kv_len < 0) return fail(KVAX_EINVAL, "negative batch or length");
  if (num_masks < 1 || num_masks > KVAX_MAX_MASKS)
    return fail(KVAX_EINVAL, "num_masks must be in [1, %d], got %d", KVAX_MAX_MASKS, num_masks);
  if (!masks) return fail(KVAX_EINVAL, "masks is null");
  for (int m = 0; m < num_masks; m++)
    if (masks[m].query_block_size <= 0 || masks[m].kv_block_size <= 0)
      return fail(KVAX_EINVAL, "mask %d: block sizes must be positive", m);
  return KVAX_OK;
}

}  // namespace
}  // namespace kvax

using namespace kvax;

extern "C" size_t kvax_mask_workspace_bytes(int batch, int q_len, int kv_len,
                                            const kvax_mask_desc* masks, int num_masks) {
  if (validate(batch, q_len, kv_len, masks, num_masks) != KVAX_OK) return 0;
  SummaryKey keys[2 * KVAX_MAX_MASKS];
  int qk[KVAX_MAX_MASKS], kk[KVAX_MAX_MASKS];
  size_t total = 0;
  plan_summaries(q_len, kv_len, masks, num_masks, keys, qk, kk, (size_t)batch, &total);
  return total * sizeof(int4);
}

extern "C" int kvax_mask_build(const int32_t* q_pos, const int32_t* q_seg, const int32_t* kv_pos,
                               const int32_t* kv_seg, int batch, int q_len, int kv_len,
                               int num_q_shards, int skip_pad_tokens, const kvax_mask_desc* masks,
                               int num_masks, void* workspace, size_t workspace_bytes,
                               kvax_stream_t stream_) {
  if (int rc = validate(batch, q_len, kv_len, masks, num_masks)) return rc;
  if (num_q_shards < 1) return fail(KVAX_EINVAL, "num_q_shards must be >= 1");
  hipStream_t stream = (hipStream_t)stream_;
  SummaryKey keys[2 * KVAX_MAX_MASKS];
  int qk[KVAX_MAX_MASKS], kk[KVAX_MAX_MASKS];
  size_t total = 0;
  const int num_keys =
      plan_summaries(q_len, kv_len, masks, num_masks, keys, qk, kk, (size_t)batch, &total);
  if (batch == 0) return KVAX_OK;
  if (total * sizeof(int4) > workspace_bytes || (total && !workspace))
    return fail(KVAX_EWORKSPACE, "workspace of %zu bytes needed, %zu given", total * sizeof(int4),
                workspace_bytes);
  if ((q_len && (!q_pos || !q_seg)) || (kv_len && (!kv_pos || !kv_seg)))
    return fail(KVAX_EINVAL, "null id array");
  if (((uintptr_t)workspace) % sizeof(int4))
    return fail(KVAX_EINVAL, "workspace must be 16-byte aligned");

  // The id that replaces -1 is (padded kv length + 1) and so depends on the mask's kv block
  // size.  Masks whose kv block sizes pad kv_len to the same length share one summary pass;
  // otherwise each mask is built by its own pair of launches with its own id.
  int32_t pad_ids[KVAX_MAX_MASKS];
  bool same_pad = true;
  for (int m = 0; m < num_masks; m++) {
    pad_ids[m] = cdiv(kv_len, masks[m].kv_block_size) * masks[m].kv_block_size + 1;
    if (pad_ids[m] != pad_ids[0]) same_pad = false;
  }
  if (!same_pad) {
    // Different padded kv lengths: build the masks one call at a time so each uses its own id.
    for (int m = 0; m < num_masks; m++) {
      int rc = kvax_mask_build(q_pos, q_seg, kv_pos, kv_seg, batch, q_len, kv_len, num_q_shards,
                               skip_pad_tokens, masks + m, 1, workspace, workspace_bytes, stream_);
      if (rc) return rc;
    }
    return KVAX_OK;
  }

  SummaryParams sp{};
  sp.num_jobs = num_keys;
  sp.pad_id = pad_ids[0];
  int max_blocks = 0;
  for (int k = 0; k < num_keys; k++) {
    SummaryJob& j = sp.jobs[k];
    j.pos = keys[k].kv ? kv_pos : q_pos;
    j.seg = keys[k].kv ? kv_seg : q_seg;
    j.out = (int4*)workspace + keys[k].offset;
    j.len = keys[k].kv ? kv_len : q_len;
    j.block_size = keys[k].block_size;
    j.n_blocks = keys[k].n_blocks;
    j.pos_fill = keys[k].kv ? kInt32Max : -1;
    max_blocks = max_blocks > j.n_blocks ? max_blocks : j.n_blocks;
  }
  BoundsParams bp{};
  bp.num_jobs = num_masks;
  bp.pad_id = pad_ids[0];
  bp.skip_pad = skip_pad_tokens != 0;
  int max_outer = 0, max_shards = 1;
  for (int m = 0; m < num_masks; m++) {
    const kvax_mask_desc& d = masks[m];
    BoundsJob& j = bp.jobs[m];
    const SummaryKey& qs = keys[qk[m]];
    const SummaryKey& ks = keys[kk[m]];
    j.kv_outer = d.kv_outer != 0;
    const SummaryKey& outer = j.kv_outer ? ks : qs;
    const SummaryKey& inner = j.kv_outer ? qs : ks;
    j.outer = (const int4*)workspace + outer.offset;
    j.inner = (const int4*)workspace + inner.offset;
    j.n_outer = outer.n_blocks;
    j.n_inner_total = inner.n_blocks;
    if (j.n_outer > 0 && (!d.lower || !d.upper || !d.lower_full || !d.upper_full))
      return fail(KVAX_EINVAL, "mask %d: null output pointer", m);
    j.num_shards = 1;
    if (num_q_shards > 1) {
      if (q_len % num_q_shards || (q_len / num_q_shards) % d.query_block_size)
        return fail(KVAX_EINVAL,
                    "mask %d: q_len %d does not split into %d shards of whole %d-token blocks", m,
                    q_len, num_q_shards, d.query_block_size);
      if (j.kv_outer) j.num_shards = num_q_shards;
    }
    j.lower = d.lower;
    j.upper = d.upper;
    j.lower_full = d.lower_full;
    j.upper_full = d.upper_full;
    max_outer = max_outer > j.n_outer ? max_outer : j.n_outer;
    max_shards = max_shards > j.num_shards ? max_shards : j.num_shards;
  }
  if (max_blocks > 0) {
    dim3 grid(cdiv(max_blocks, kWavesPerGroup), batch, num_keys);
    hipLaunchKernelGGL(block_summaries_kernel, grid, dim3(kWave * kWavesPerGroup), 0, stream, sp);
    if (int rc = check_launch("block_summaries_kernel")) return rc;
  }
  if (max_outer > 0) {
    dim3 grid(cdiv(max_outer, kWavesPerGroup), batch * max_shards, num_masks);
    hipLaunchKernelGGL(block_bounds_kernel, grid, dim3(kWave * kWavesPerGroup), 0, stream, bp,
                       max_shards);
    if (int rc = check_launch("block_bounds_kernel")) return rc;
  }
  return KVAX_OK;
}
