// Flash-attention backward for gfx950: dQ kernel (query-stationary; also produces delta) and dK/dV
// kernel (kv-stationary, all query heads of a GQA group reduced in registers), run in that order.
//
// Semantics: reference kvax/ops/flash_attention_triton.py:373-410 (delta = rowsum(O * dO)),
// :526-617 / :620-871 (dQ: P = exp2(S * scale * log2e - lse), dS = P * (dP - delta),
// dQ = scale * dS K) and :413-523 / :874-1191 (dV = P^T dO, dK = scale * dS^T Q, summed over the
// query heads of each kv head as :1855-1868 does).  P and dS are rounded to the input dtype
// before the second contractions, as in the reference.  Padding tokens take part in nothing and
// get exact-zero gradients.
//
// Layout trick shared with the forward: each contraction is arranged so that the tile produced
// by the first MFMA stage (P or dS in C layout: one column per lane) is directly the B operand
// of the second stage, whose A operand is gathered with transposing LDS reads.
//   dQ kernel:    S^T, dP^T [kv x q]  ->  dQ^T [d x q]  += K^T [d x kv]  dS^T [kv x q]
//   dK/dV kernel: S,   dP   [q x kv]  ->  dV^T [d x kv] += dO^T [d x q]  P  [q x kv]
//                                         dK^T [d x kv] += Q^T  [d x q]  dS [q x kv]
// The dK/dV kernel passes P between the two wavefronts of a pair through LDS (see there); no
// atomics are used and the result is deterministic.
#include "common.h"
#include "fa_common.h"

namespace kvax {
int validate_fa_common(const kvax_fa_args* a);

namespace {

constexpr int kTile = kTileRows;  // rows of the streamed operand per LDS stage

struct BwdParams {
  const char* q;
  const char* k;
  const char* v;
  const char* out;
  const char* dout;
  char* dq;
  char* dk;
  char* dv;
  const float* lse;
  float* delta;
  const int32_t* q_pos;
  const int32_t* q_seg;
  const int32_t* kv_pos;
  const int32_t* kv_seg;
  const int32_t* dq_mask[4];
  const int32_t* dkdv_mask[4];
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int64_t do_sb, do_ss, do_sh;
  int64_t dq_sb, dq_ss, dq_sh;
  int64_t dk_sb, dk_ss, dk_sh;
  int64_t dv_sb, dv_ss, dv_sh;
  int batch, q_len, kv_len, num_heads, num_kv_heads, group;
  int bq, bk;  // backward block sizes: the dQ mask has query blocks of bk and kv blocks of bq
  int n_dq_blocks, n_kv_blocks;
  int num_tiles, total_items;
  int dkdv_f32;  // dK / dV are fp32 tensors (strides still in elements)
  const int4* kv_tiles;  // tile summaries [batch, n_kv_tiles, 2]
  const int4* q_tiles;   // tile summaries [batch, n_q_tiles, 2]
  int n_kv_tiles, n_q_tiles;
  int list_tiles;  // dK/dV kernel: query tiles per chunk of the live-tile bookkeeping
  int32_t* order_ws;           // room for the dK/dV dispatch order and its scratch
  const int32_t* dkdv_order;   // dispatch order of the kv tiles [batch, tiles], or null
  int32_t* dkdv_queue;         // dK/dV kernel: one item counter per XCD, zero at launch
  int flags;
  float scale, scale_log2;
  float scale_log2_abs;  // |scale| * log2(e) > 0, used with K negated when the scale is negative
  uint32_t k_sign;       // 0x80008000 when the scale is negative
};

// ---------------------------------------------------------------------------------------------
// Merged range of the streamed axis for a work-group that covers several mask blocks of the
// stationary axis: union of [lower, upper), intersection of [lower_full, upper_full), in elements.
// ---------------------------------------------------------------------------------------------
struct Range {
  int lo, hi, flo, fhi;
};

__device__ __forceinline__ Range merged_range(const int32_t* const mask[4], int64_t base, int blk0,
                                              int blk1, int unit, int limit) {
  Range r{0x7fffffff, 0, 0, 0x7fffffff};
  for (int blk = blk0; blk <= blk1; blk++) {
    const int l_ = mask[0][base + blk] * unit, u_ = mask[1][base + blk] * unit;
    r.flo = max(r.flo, mask[2][base + blk] * unit);
    r.fhi = min(r.fhi, mask[3][base + blk] * unit);
    if (u_ > l_) {
      r.lo = min(r.lo, l_);
      r.hi = max(r.hi, u_);
    }
  }
  r.hi = min(r.hi, limit);
  return r;
}

// ---------------------------------------------------------------------------------------------
// dQ: one work-group = NW wavefronts x 32 query rows of one (batch, head); streams the live K/V
// tiles through a ring of LDS stages filled by asynchronous copies.
// ---------------------------------------------------------------------------------------------
template <int D, int STAGES>
struct DqSmem {
  static constexpr int kTileBytes = kTile * D * 2;  // swizzled, unpadded
  static constexpr int kStage = 2 * kTileBytes + 2 * kTile * 4;
  static constexpr int kTotal = STAGES * kStage;
};

template <class Tr, int D, int NW, int WPS, int STAGES>
__global__ __launch_bounds__(NW * 64, WPS) void fa_bwd_dq_kernel(const BwdParams p) {
  using vec8 = typename Tr::vec8;
  using Smem = DqSmem<D, STAGES>;
  constexpr int TQ = NW * 32;
  constexpr int KSTEPS = D / 16;
  constexpr int DT = D / 32;
  constexpr int RB = D * 2;
  constexpr int kCopies = 2 * async_tile_copies_per_wave<kTile, D, NW>() + 1;
  static_assert(STAGES == 2 || STAGES == 3, "the loop below keeps STAGES - 1 tiles in flight");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;  // wave-uniform on purpose
  const int c = lane % 32, h = lane / 32;

  int group, rank, g;
  const ItemMap items{p.batch * p.num_kv_heads, p.num_tiles, p.group};
  if (!items.decode(blockIdx.x, group, rank, g)) return;
  const int kv_head = group % p.num_kv_heads;
  const int b = group / p.num_kv_heads;
  const int q_tile = p.num_tiles - 1 - rank;
  const int head = kv_head * p.group + g;
  const int q0 = q_tile * TQ;

  const int32_t* kv_seg = p.kv_seg + (int64_t)b * p.kv_len;
  const int32_t* kv_pos = p.kv_pos + (int64_t)b * p.kv_len;
  const char* kbase = p.k + ((int64_t)b * p.k_sb + (int64_t)kv_head * p.k_sh) * 2;
  const char* vbase = p.v + ((int64_t)b * p.v_sb + (int64_t)kv_head * p.v_sh) * 2;

  const int qbs = p.bk, kbs = p.bq;  // the dQ mask swaps the backward block sizes
  const int64_t mbase = (int64_t)b * p.n_dq_blocks;
  const Range r = merged_range(p.dq_mask, mbase, q0 / qbs,
                               min((q0 + TQ - 1) / qbs, p.n_dq_blocks - 1), kbs, p.kv_len);
  const int t_lo = r.lo / kTile;
  const int t_hi = r.hi > r.lo ? (r.hi + kTile - 1) / kTile : t_lo;
  const int tf_lo = (r.flo + kTile - 1) / kTile, tf_hi = r.fhi / kTile;

  if (t_hi <= t_lo) {
    // No row of the tile can attend to anything (padding queries): zeros for dQ and delta, and
    // nothing is read.  Whole rows, 16 bytes per lane.
    constexpr int kChunks = D * 2 / 16;
    const int rows = min(TQ, p.q_len - q0);
    char* dq0 = p.dq + ((int64_t)b * p.dq_sb + (int64_t)head * p.dq_sh) * 2;
    for (int i = tid; i < rows * kChunks; i += NW * 64)
      *reinterpret_cast<uint4*>(dq0 + (int64_t)(q0 + i / kChunks) * p.dq_ss * 2 + (i % kChunks) * 16) =
          make_uint4(0, 0, 0, 0);
    for (int i = tid; i < rows; i += NW * 64)
      p.delta[((int64_t)b * p.num_heads + head) * p.q_len + q0 + i] = 0.f;
    return;
  }

  // per-lane query column.  Its ids, its row of the block mask and lse are read without waiting
  // for one another (index 0 stands in for rows beyond the sequence), as are dO, O, Q and the first
  // 64 tile summaries below: one trip to memory for the whole prologue instead of several in a row.
  const int qrow = q0 + wave * 32 + c;
  const bool in = qrow < p.q_len;
  const int qi = in ? qrow : 0;
  const int qseg_raw = p.q_seg[(int64_t)b * p.q_len + qi];
  const int qpos_raw = p.q_pos[(int64_t)b * p.q_len + qi];
  const int lower_raw = p.dq_mask[0][mbase + qi / qbs], upper_raw = p.dq_mask[1][mbase + qi / qbs];
  const float lse_raw = p.lse[((int64_t)b * p.num_heads + head) * p.q_len + qi];
  const int4* kv_summaries = p.kv_tiles + 2 * (int64_t)b * p.n_kv_tiles;
  const WordSummaries first_word = load_word_summaries(kv_summaries, t_lo >> 6, t_lo, t_hi, lane);
  // dO fragments (B operand of dP^T = V dO^T): lane holds 8 consecutive head-dim elements per
  // step, i.e. half of its row; with the same half of O they give delta = rowsum(O * dO)
  // (reference attn_bwd_preprocess, flash_attention_triton.py:373-410), which is also written out
  // for the dK/dV kernel.
  uint4 draw[KSTEPS];
  // Q fragments (B operand of S^T = K Q^T), requested with dO and O so that their latency does not
  // follow that of the live-tile bookkeeping below
  uint4 qraw[KSTEPS], oraw[KSTEPS];
  {
    // rows beyond the sequence read row 0 and are zeroed afterwards: no load sits behind a branch
    const char* qr = p.q + ((int64_t)b * p.q_sb + (int64_t)head * p.q_sh + (int64_t)qi * p.q_ss) * 2;
    const char* dr = p.dout + ((int64_t)b * p.do_sb + (int64_t)head * p.do_sh + (int64_t)qi * p.do_ss) * 2;
    const char* orow = p.out + ((int64_t)b * p.o_sb + (int64_t)head * p.o_sh + (int64_t)qi * p.o_ss) * 2;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      draw[ks] = *reinterpret_cast<const uint4*>(dr + (16 * ks + 8 * h) * 2);
      oraw[ks] = *reinterpret_cast<const uint4*>(orow + (16 * ks + 8 * h) * 2);
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qraw[ks] = make_uint4(0, 0, 0, 0);
    if (t_hi > t_lo) {  // wave-uniform: nothing to attend to, no Q
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) qraw[ks] = *reinterpret_cast<const uint4*>(qr + (16 * ks + 8 * h) * 2);
    }
  }
  float delta_q = 0.f;
  {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (!in) draw[ks] = oraw[ks] = qraw[ks] = make_uint4(0, 0, 0, 0);
      const uint4 o4 = oraw[ks];
      const uint32_t ow[4] = {o4.x, o4.y, o4.z, o4.w}, gw[4] = {draw[ks].x, draw[ks].y, draw[ks].z, draw[ks].w};
#pragma unroll
      for (int w = 0; w < 4; w++) {
        delta_q += Tr::to_float((uint16_t)(ow[w] & 0xffff)) * Tr::to_float((uint16_t)(gw[w] & 0xffff));
        delta_q += Tr::to_float((uint16_t)(ow[w] >> 16)) * Tr::to_float((uint16_t)(gw[w] >> 16));
      }
    }
    delta_q += xor32(delta_q);
    if (in && h == 0) p.delta[((int64_t)b * p.num_heads + head) * p.q_len + qrow] = delta_q;
  }
  const int qseg = in ? qseg_raw : -1;
  const int qpos = in ? qpos_raw : 0;
  int col_lo = 0;
  unsigned col_width = 0;
  float lse_q = 0.f;
  if (in && qseg != -1) {
    col_lo = lower_raw * kbs;
    col_width = (unsigned)max(min(upper_raw * kbs, p.kv_len) - col_lo, 0);
    lse_q = lse_raw;
  }
  TileParts mine[1];
  mine[0] = wave_parts(col_width > 0, qseg, qpos);

  // live kv tiles of [t_lo, t_hi): per-wave bitmaps, compacted into one list
  int* live_count = reinterpret_cast<int*>(smem + Smem::kTotal);
  unsigned long long* live_bits = reinterpret_cast<unsigned long long*>(smem + Smem::kTotal + 16);
  const int word0 = t_lo >> 6;
  const int words = t_hi > t_lo ? ((t_hi - 1) >> 6) - word0 + 1 : 0;
  const uint32_t* live_list = reinterpret_cast<const uint32_t*>(live_bits + NW * (cdiv_dev(p.n_kv_tiles, 64) + 1));
  mark_live_tiles<true, 1>(kv_summaries, mine, t_lo, t_hi, live_bits + wave * words, word0, lane, first_word);
  __syncthreads();
  if (wave == 0)
    compact_live_tiles<NW>(live_bits, words, word0, const_cast<uint32_t*>(live_list), live_count, lane);
  __syncthreads();
  const int n_live = *live_count;

  f32x16 dq[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) dq[dt][i] = 0.f;

  if (n_live > 0) {
    vec8 qf[KSTEPS], dof[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      qf[ks] = __builtin_bit_cast(vec8, qraw[ks]);
      dof[ks] = __builtin_bit_cast(vec8, draw[ks]);
    }
    int nat_off[KSTEPS], tr_off[DT][2];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) nat_off[ks] = nat_offset<D>(c, ks, h);
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      tr_off[dt][0] = tr_offset<D>(lane, dt, 0);
      tr_off[dt][1] = tr_offset<D>(lane, dt, 1);
    }

    const uint32_t smem_addr = (uint32_t)(uintptr_t)smem;
    const int32_t* id_src = (wave & 1) ? kv_pos : kv_seg;
    const AsyncTileCopy<kTile, D, NW> copy_k(p.k_ss * 2, wave, lane), copy_v(p.v_ss * 2, wave, lane);
    auto issue = [&](int tile, int stage) {
      const uint32_t base = smem_addr + stage * Smem::kStage;
      copy_k(kbase, tile * kTile, p.kv_len, base);
      copy_v(vbase, tile * kTile, p.kv_len, base + Smem::kTileBytes);
      async_copy_b32(id_src + min(tile * kTile + lane, p.kv_len - 1),
                     __builtin_amdgcn_readfirstlane(base + 2 * Smem::kTileBytes + (wave & 1) * (kTile * 4)));
    };

    uint32_t e0 = live_list[0];
    uint32_t e1 = n_live > 1 ? live_list[1] : 0;
    uint32_t e2 = n_live > 2 ? live_list[2] : 0;
    issue(e0 & 0xffffff, 0);
    if (STAGES == 3 && n_live > 1) issue(e1 & 0xffffff, 1);

    int stage = 0;
    for (int i = 0; i < n_live; i++) {
      if (STAGES == 3 && i + 1 < n_live) wait_vmcnt<kCopies>(); else wait_vmcnt<0>();
      __syncthreads();
      const uint32_t e3 = i + 3 < n_live ? live_list[i + 3] : 0;
      if (STAGES == 3) {
        if (i + 2 < n_live) issue(e2 & 0xffffff, stage >= 1 ? stage - 1 : STAGES - 1);  // (stage + 2) % 3
      } else {
        if (i + 1 < n_live) issue(e1 & 0xffffff, stage ^ 1);
      }
      const int t = e0 & 0xffffff;

      if ((e0 >> (24 + wave)) & 1) {
        const int kv0 = t * kTile;
        const char* ktile = smem + stage * Smem::kStage;
        const char* vtile = ktile + Smem::kTileBytes;
        const int32_t* ids = reinterpret_cast<const int32_t*>(ktile + 2 * Smem::kTileBytes);
        const bool full = t >= tf_lo && t < tf_hi;

#pragma unroll 1
        for (int kt = 0; kt < 2; kt++) {
          // S^T = K Q^T and dP^T = V dO^T for 32 kv rows: 16 MFMAs, operand reads four ahead
          f32x16 s, dp;
#pragma unroll
          for (int i2 = 0; i2 < 16; i2++) s[i2] = 0.f, dp[i2] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ks++) {
            const vec8 ka = *reinterpret_cast<const vec8*>(ktile + 32 * kt * RB + nat_off[ks]);
            const vec8 va = *reinterpret_cast<const vec8*>(vtile + 32 * kt * RB + nat_off[ks]);
            s = Tr::mfma(ka, qf[ks], s);
            dp = Tr::mfma(va, dof[ks], dp);
          }
          __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
          for (int i2 = 0; i2 < 2 * KSTEPS - 4; i2++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
          // K^T operands of this block's dQ update, requested before the element-wise work
          vec8 ta[DT];
#pragma unroll
          for (int dt = 0; dt < DT; dt++)
            ta[dt] = tr_read_a_swz<Tr>(ktile + 32 * kt * RB, tr_off[dt][0], tr_off[dt][1]);
#pragma unroll
          for (int i2 = 0; i2 < 16; i2++) s[i2] = fast_exp2(__builtin_fmaf(s[i2], p.scale_log2, -lse_q));
          if (!full)
            mask_c_tile<true>(s, ids, ids + kTile, 32 * kt, kv0, h, qseg, qpos, col_lo, col_width, 0.f);
#pragma unroll
          for (int i2 = 0; i2 < 16; i2++) s[i2] *= dp[i2] - delta_q;
          // dQ^T += K^T dS^T
#pragma unroll
          for (int st = 0; st < 2; st++) {
            const vec8 dsb = pack8<Tr>(s[8 * st + 0], s[8 * st + 1], s[8 * st + 2], s[8 * st + 3],
                                       s[8 * st + 4], s[8 * st + 5], s[8 * st + 6], s[8 * st + 7]);
            vec8 tb[DT];  // second half's operands, requested before the first half's MFMAs
            if (st == 0) {
#pragma unroll
              for (int dt = 0; dt < DT; dt++)
                tb[dt] = tr_read_a_swz<Tr>(ktile + (32 * kt + 16) * RB, tr_off[dt][0], tr_off[dt][1]);
            }
#pragma unroll
            for (int dt = 0; dt < DT; dt++) dq[dt] = Tr::mfma(ta[dt], dsb, dq[dt]);
            if (st == 0) {
#pragma unroll
              for (int dt = 0; dt < DT; dt++) ta[dt] = tb[dt];
            }
          }
        }
      }
      e0 = e1, e1 = e2, e2 = e3;
      stage = stage == STAGES - 1 ? 0 : stage + 1;
    }
  }

  {
    // Rows that attend to nothing (padding) get exact zeros.  Their accumulator is not zero when the
    // block mask declares padding-against-padding blocks mask-free (masks built without skipping
    // padding): the element mask, which is what excludes them, is not applied there.
    // The rows leave through LDS (each wavefront its own part of the tile space, which is done with)
    // as whole rows, 16 bytes per lane, instead of 8-byte pieces of 32 rows per store; rows are
    // swizzled by the row index against bank conflicts.
    const bool dead = col_width == 0;
    __syncthreads();  // every wavefront has read its last tile
    constexpr int kRowBytes = D * 2, kChunks = kRowBytes / 16, kRowsPerStore = 64 / kChunks;
    char* stage = smem + wave * (32 * kRowBytes);
    char* mine = stage + c * kRowBytes;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        uint2 u;
        u.x = Tr::pack2(dq[dt][4 * g4 + 0] * p.scale, dq[dt][4 * g4 + 1] * p.scale);
        u.y = Tr::pack2(dq[dt][4 * g4 + 2] * p.scale, dq[dt][4 * g4 + 3] * p.scale);
        if (dead) u = make_uint2(0, 0);
        *reinterpret_cast<uint2*>(mine + (((4 * dt + g4) ^ (c & (kChunks - 1))) * 16) + 8 * h) = u;
      }
    char* dq0 = p.dq + ((int64_t)b * p.dq_sb + (int64_t)head * p.dq_sh) * 2;
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += kRowsPerStore) {
      const int row = r0 + lane / kChunks, chunk = lane % kChunks;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + row * kRowBytes + ((chunk ^ (row & (kChunks - 1))) * 16));
      const int qr = q0 + wave * 32 + row;
      if (qr < p.q_len) *reinterpret_cast<uint4*>(dq0 + (int64_t)qr * p.dq_ss * 2 + chunk * 16) = v;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// dK/dV: one work-group = 128 kv rows of one (batch, kv head), 8 wavefronts in 4 pairs.  Both
// wavefronts of a pair own the same 32 kv rows and share a SIMD; they split the work by role:
//   P wave, tile t:  S = Q K^T,  P = exp2(S * c - lse) -> LDS,  dV^T += dO^T P
//   S wave, tile t:  dS = P * (dP - delta) and dK^T += Q^T dS of tile t - 1 (P from LDS, dP kept
//                    in registers), then dP = dO V^T of tile t
// so that each holds one accumulator tile set and one fragment set (K or V) - half the registers
// of doing both, which is what lets two wavefronts run per SIMD.  The S wave running one tile
// behind means one barrier per tile, and at any time one wavefront of the pair has element-wise
// work while the other has MFMAs.  The work-group streams the live Q / dO tiles of every query
// head of the group; Q tiles stay one step longer than dO tiles, hence separate rings.
// ---------------------------------------------------------------------------------------------
// Shape of a dK/dV work-group per head_dim.  Up to 128 it is 8 wavefronts (4 role pairs, 128 kv
// rows) at two per SIMD, stepping through 64-row query tiles.  At 256 a wavefront's fragments and
// accumulators need more than half a SIMD's registers, so it is 4 wavefronts (2 pairs, 64 kv rows) at
// one per SIMD, and the Q / dO rings only fit in LDS with 32-row steps: a 64-row tile of the live
// list is then taken as two steps.
template <int D>
struct DkdvCfg {
  static constexpr int kPairs = D > 128 ? 2 : 4;
  static constexpr int kStepRows = D > 128 ? 32 : 64;  // query rows per step (and LDS stage)
  static constexpr int kWps = D > 128 ? 1 : 2;         // wavefronts per SIMD
  static constexpr int kWaves = 2 * kPairs;
  static constexpr int kKvRows = 32 * kPairs;          // kv rows per work-group
  static constexpr int kUnits = kStepRows / 32;        // 32-row MFMA units per step
  static constexpr int kSub = kTile / kStepRows;       // steps per 64-row tile of the live list
};

template <int D>
struct DkdvSmem {
  using Cfg = DkdvCfg<D>;
  static constexpr int kTileBytes = Cfg::kStepRows * D * 2;  // swizzled, unpadded
  // lse, delta, seg, pos: 64 entries each whatever the step size (a wave-wide copy brings 64)
  static constexpr int kRowData = 4 * kTile * 4;
  static constexpr int kQStages = 4, kDoStages = 3;
  static constexpr int kQ = 0;
  static constexpr int kDo = kQ + kQStages * kTileBytes;
  static constexpr int kRows = kDo + kDoStages * kTileBytes;
  static constexpr int kExchange = kRows + kQStages * kRowData;
  // per pair two slots of P (one kStepRows x 32 tile, 16 bits per element): written for step s while
  // the slot of step s - 1 is read
  static constexpr int kSlotBytes = Cfg::kUnits * 2 * 1024;
  static constexpr int kTotal = kExchange + Cfg::kPairs * 2 * kSlotBytes;
};

template <class Tr, int D>
__global__ __launch_bounds__(DkdvCfg<D>::kWaves * 64, DkdvCfg<D>::kWps) void fa_bwd_dkdv_kernel(const BwdParams p) {
  using vec8 = typename Tr::vec8;
  using Smem = DkdvSmem<D>;
  using Cfg = DkdvCfg<D>;
  constexpr int NW = Cfg::kWaves;
  constexpr int NP = Cfg::kPairs;
  constexpr int TKV = Cfg::kKvRows;
  constexpr int SR = Cfg::kStepRows;
  constexpr int UNITS = Cfg::kUnits;
  constexpr int SUB = Cfg::kSub;
  constexpr int KSTEPS = D / 16;
  constexpr int DT = D / 32;
  constexpr int RB = D * 2;
  // only the P waves issue tile copies: they are the ones with slack before the barrier.  Each
  // also copies its share of the four row-data arrays.
  constexpr int kRowCopies = 4 / NP;
  constexpr int kCopies = 2 * async_tile_copies_per_wave<SR, D, NP>() + kRowCopies;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;  // wave-uniform on purpose
  const int c = lane % 32, h = lane / 32;
  const int pair = wave % NP;
  const bool p_wave = wave < NP;  // role, wave-uniform

  // The launch is one work-group per compute unit, and each takes work items (128 kv rows of one
  // batch row and kv head) from the queues (see ItemQueue) until none is left.  The ticket for the
  // next item is drawn when the current one's step loop has ended, so that its latency hides behind
  // the final stores and an item is never held back by a long one.
  const ItemMap items{p.batch * p.num_kv_heads, p.num_tiles, 1};
  ItemQueue work{p.dkdv_queue, p.total_items, (int)(blockIdx.x % 8)};  // thread 0's
  int* next_item = reinterpret_cast<int*>(smem + Smem::kTotal) + 1;
  if (tid == 0) *next_item = work.resolve(work.draw());
  __syncthreads();
  for (int item = *next_item; item >= 0; item = *next_item) {
  __syncthreads();  // every wavefront has read next_item
  int ticket = 0;
  // kv tiles in the computed dispatch order (without one: early tiles first, which see the most
  // queries under a causal mask)
  int group, rank, member;
  if (items.decode(item, group, rank, member)) {
  const int kv_head = group % p.num_kv_heads;
  const int b = group / p.num_kv_heads;
  const int entry = p.dkdv_order ? p.dkdv_order[(int64_t)b * p.num_tiles + rank] : rank;
  const int kv_tile = entry & (kDeadItem - 1);
  const int k0 = kv_tile * TKV;
  if (entry & kDeadItem) {
    // no query tile can interact with these kv rows (known from the ordering pass): zeros, no bookkeeping
    if (tid == 0) ticket = work.draw();
    const int row_bytes = D * (p.dkdv_f32 ? 4 : 2), chunks = row_bytes / 16;
    const int rows = min(TKV, p.kv_len - k0);
    for (int i = tid; i < rows * chunks; i += NW * 64) {
      const int64_t row = k0 + i / chunks;
      const int at = (i % chunks) * 16;
      *reinterpret_cast<uint4*>(p.dk + ((int64_t)b * p.dk_sb + (int64_t)kv_head * p.dk_sh + row * p.dk_ss) * (row_bytes / D) + at) = make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4*>(p.dv + ((int64_t)b * p.dv_sb + (int64_t)kv_head * p.dv_sh + row * p.dv_ss) * (row_bytes / D) + at) = make_uint4(0, 0, 0, 0);
    }
  } else {

  const int kbs = p.bk, qbs = p.bq;
  const int64_t mbase = (int64_t)b * p.n_kv_blocks;
  const Range r = merged_range(p.dkdv_mask, mbase, k0 / kbs,
                               min((k0 + TKV - 1) / kbs, p.n_kv_blocks - 1), qbs, p.q_len);
  const int t_lo = r.lo / kTile;
  const int t_hi = r.hi > r.lo ? (r.hi + kTile - 1) / kTile : t_lo;
  const int tf_lo = (r.flo + kTile - 1) / kTile, tf_hi = r.fhi / kTile;

  // per-lane kv column (the same for both wavefronts of a pair)
  const int kvcol = k0 + pair * 32 + c;
  const bool in = kvcol < p.kv_len;
  const int kvseg = in ? p.kv_seg[(int64_t)b * p.kv_len + kvcol] : -1;
  const int kvpos = in ? p.kv_pos[(int64_t)b * p.kv_len + kvcol] : 0;
  int col_lo = 0;
  unsigned col_width = 0;
  if (in && kvseg != -1) {
    col_lo = p.dkdv_mask[0][mbase + kvcol / kbs] * qbs;
    // queries at or beyond q_len never count (their LDS rows hold a copy of the last row)
    col_width = (unsigned)max(min(p.dkdv_mask[1][mbase + kvcol / kbs] * qbs, p.q_len) - col_lo, 0);
  }
  TileParts mine[1];
  mine[0] = wave_parts(col_width > 0, kvseg, kvpos);

  f32x16 acc[DT];  // dV^T (P wave) or dK^T (S wave): rows = head dim, columns = the lane's kv row
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[dt][i] = 0.f;

  // The query range is walked in chunks of at most p.list_tiles tiles, the number whose live-tile
  // bookkeeping fits in the LDS left over (one chunk unless the query sequence is very long).
  int* live_count = reinterpret_cast<int*>(smem + Smem::kTotal);
  unsigned long long* live_bits = reinterpret_cast<unsigned long long*>(smem + Smem::kTotal + 16);
  const uint32_t* live_list = reinterpret_cast<const uint32_t*>(live_bits + NW * (cdiv_dev(p.list_tiles, 64) + 1));
  for (int c_lo = t_lo; c_lo < t_hi; c_lo += p.list_tiles) {
  const int c_hi = min(c_lo + p.list_tiles, t_hi);
  // live query tiles of [c_lo, c_hi) (the same for every head of the group; both wavefronts of a
  // pair mark the same tiles)
  const int word0 = c_lo >> 6;
  const int words = ((c_hi - 1) >> 6) - word0 + 1;
  const int4* q_summaries = p.q_tiles + 2 * (int64_t)b * p.n_q_tiles;
  mark_live_tiles<false, 1>(q_summaries, mine, c_lo, c_hi, live_bits + wave * words, word0, lane,
                            load_word_summaries(q_summaries, word0, c_lo, c_hi, lane));
  __syncthreads();
  if (wave == 0)
    // highest query tile first: every kv work-group of a document ends on the document's last query
    // tiles, so walking backwards the work-groups that run together stream the same Q/dO tiles at
    // the same time (they start at different tiles when walking forwards) and share them in L2
    compact_live_tiles<NW, true>(live_bits, words, word0, const_cast<uint32_t*>(live_list), live_count, lane);
  __syncthreads();
  const int n_live = *live_count;
  const int steps = n_live * p.group * SUB;  // every head of the group walks the same list

  if (steps > 0) {
    // stationary fragments: K (negated when the scale is negative) for the P wave, V for the S wave
    vec8 frag[KSTEPS];
    {
      const char* base = p_wave ? p.k + ((int64_t)b * p.k_sb + (int64_t)kv_head * p.k_sh + (int64_t)(in ? kvcol : 0) * p.k_ss) * 2
                                : p.v + ((int64_t)b * p.v_sb + (int64_t)kv_head * p.v_sh + (int64_t)(in ? kvcol : 0) * p.v_ss) * 2;
      const uint32_t sign = p_wave ? p.k_sign : 0u;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        uint4 u = make_uint4(0, 0, 0, 0);
        if (in) u = *reinterpret_cast<const uint4*>(base + (16 * ks + 8 * h) * 2);
        u.x ^= sign, u.y ^= sign, u.z ^= sign, u.w ^= sign;
        frag[ks] = __builtin_bit_cast(vec8, u);
      }
    }
    int nat_off[KSTEPS], tr_off[DT][2];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) nat_off[ks] = nat_offset<D>(c, ks, h);
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      tr_off[dt][0] = tr_offset<D>(lane, dt, 0);
      tr_off[dt][1] = tr_offset<D>(lane, dt, 1);
    }

    const uint32_t smem_addr = (uint32_t)(uintptr_t)smem;
    const AsyncTileCopy<SR, D, NP> copy_q(p.q_ss * 2, pair, lane), copy_do(p.do_ss * 2, pair, lane);
    // Step s = (head s / n_live of the group, list entry s % n_live); its Q tile and row data go to
    // slot s % 4 of their rings, its dO tile to slot s % 3.  The issuing side keeps its own cursor
    // (list index, per-head base pointers) and advances it by additions only: divisions and 64-bit
    // multiplies per copy are serial scalar work of the issuing wave.
    const int head0 = kv_head * p.group;
    const char* is_q = p.q + ((int64_t)b * p.q_sb + (int64_t)head0 * p.q_sh) * 2;
    const char* is_do = p.dout + ((int64_t)b * p.do_sb + (int64_t)head0 * p.do_sh) * 2;
    // row-data arrays this wave copies (array w of lse, delta, seg, pos for w = pair, pair + NP, ...):
    // lse and delta are per head, seg and pos per batch row
    const char* is_rows[kRowCopies];
    int64_t rows_per_head[kRowCopies];
#pragma unroll
    for (int r = 0; r < kRowCopies; r++) {
      const int which = pair + r * NP;
      is_rows[r] = which == 0   ? (const char*)(p.lse + ((int64_t)b * p.num_heads + head0) * p.q_len)
                   : which == 1 ? (const char*)(p.delta + ((int64_t)b * p.num_heads + head0) * p.q_len)
                   : which == 2 ? (const char*)(p.q_seg + (int64_t)b * p.q_len)
                                : (const char*)(p.q_pos + (int64_t)b * p.q_len);
      rows_per_head[r] = which < 2 ? (int64_t)p.q_len * 4 : 0;
    }
    int is_li = 0, is_sub = 0;
    uint32_t is_entry = live_list[0];
    auto issue_next = [&](int q_slot, int do_slot) {
      const int qr0 = (int)(is_entry & 0xffffff) * kTile + is_sub * SR;
      copy_q(is_q, qr0, p.q_len, smem_addr + Smem::kQ + q_slot * Smem::kTileBytes);
      copy_do(is_do, qr0, p.q_len, smem_addr + Smem::kDo + do_slot * Smem::kTileBytes);
#pragma unroll
      for (int r = 0; r < kRowCopies; r++)
        async_copy_b32(is_rows[r] + (int64_t)min(qr0 + lane, p.q_len - 1) * 4,
                       __builtin_amdgcn_readfirstlane(smem_addr + Smem::kRows + q_slot * Smem::kRowData +
                                                      (pair + r * NP) * (kTile * 4)));
      if (++is_sub == SUB) {
        is_sub = 0;
        if (++is_li == n_live) {
          is_li = 0;
          is_q += p.q_sh * 2;
          is_do += p.do_sh * 2;
#pragma unroll
          for (int r = 0; r < kRowCopies; r++) is_rows[r] += rows_per_head[r];
        }
        is_entry = live_list[is_li];
      }
    };

    // P of the pair's tiles, 16-bit floats with a 10-bit mantissa whatever the tensor dtype:
    // [slot][unit mt][half st] x 64 lanes x 16 bytes, in the lane order of the C tile
    char* exchange = smem + Smem::kExchange + pair * 2 * Smem::kSlotBytes + lane * 16;

    // S wave, second part of a tile: dS = P * (dP - delta) rounded to the input dtype (masked
    // entries have P = 0), dK^T += Q^T dS.  x = dP of that tile.
    auto finish_dk = [&](const f32x16 (&x)[UNITS], const char* qtile, const float* delta_rows, const char* pslot) {
      vec8 ta[2][DT];
#pragma unroll
      for (int st = 0; st < 2; st++)
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
          ta[st][dt] = tr_read_a_swz<Tr>(qtile + 16 * st * RB, tr_off[dt][0], tr_off[dt][1]);
#pragma unroll
      for (int mt = 0; mt < UNITS; mt++) {
        vec8 dsb[2];
#pragma unroll
        for (int st = 0; st < 2; st++) {
          const uint4 e = *reinterpret_cast<const uint4*>(pslot + (2 * mt + st) * 1024);
          const uint32_t w[4] = {e.x, e.y, e.z, e.w};
          const float4 d0 = *reinterpret_cast<const float4*>(delta_rows + 32 * mt + 8 * (2 * st) + 4 * h);
          const float4 d1 = *reinterpret_cast<const float4*>(delta_rows + 32 * mt + 8 * (2 * st + 1) + 4 * h);
          const float dl[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
          float ds[8];
#pragma unroll
          for (int j = 0; j < 4; j++) {
            ds[2 * j] = F16::to_float((uint16_t)(w[j] & 0xffff)) * (x[mt][8 * st + 2 * j] - dl[2 * j]);
            ds[2 * j + 1] = F16::to_float((uint16_t)(w[j] >> 16)) * (x[mt][8 * st + 2 * j + 1] - dl[2 * j + 1]);
          }
          dsb[st] = pack8<Tr>(ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]);
        }
        vec8 tb[2][DT];  // operands of the next unit, requested before this unit's MFMAs
        if (mt + 1 < UNITS) {
#pragma unroll
          for (int st = 0; st < 2; st++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
              tb[st][dt] = tr_read_a_swz<Tr>(qtile + (32 * (mt + 1) + 16 * st) * RB, tr_off[dt][0], tr_off[dt][1]);
        }
#pragma unroll
        for (int st = 0; st < 2; st++)
#pragma unroll
          for (int dt = 0; dt < DT; dt++) acc[dt] = Tr::mfma(ta[st][dt], dsb[st], acc[dt]);
        if (mt + 1 < UNITS) {
#pragma unroll
          for (int st = 0; st < 2; st++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) ta[st][dt] = tb[st][dt];
        }
      }
    };

    int li = 0, sub = 0;           // list index and sub-step of the current step
    uint32_t e0 = live_list[0];    // its entry
    uint32_t ep = 0;               // entry of the previous step
    if (p_wave) {
      issue_next(0, 0);
      if (steps > 1) issue_next(1, 1);
    }

    f32x16 x[UNITS];  // S of this step (P wave) / dP carried from the previous step (S wave)
    int q_slot = 0, do_slot = 0, q_prev = 0;
    for (int step = 0; step < steps; step++) {
      // the rows of this step have landed; every wavefront is done with the previous step
      if (p_wave) {
        if (step + 1 < steps) wait_vmcnt<kCopies>(); else wait_vmcnt<0>();
      }
      __syncthreads();
      if (p_wave && step + 2 < steps) issue_next((q_slot + 2) & 3, do_slot >= 1 ? do_slot - 1 : 2);
      const int t = e0 & 0xffffff;
      const bool active = (e0 >> (24 + wave)) & 1, active_prev = (ep >> (24 + wave)) & 1;
      const int qr0 = t * kTile + sub * SR;
      const char* qtile = smem + Smem::kQ + q_slot * Smem::kTileBytes;
      const char* dotile = smem + Smem::kDo + do_slot * Smem::kTileBytes;
      const float* rowdata = reinterpret_cast<const float*>(smem + Smem::kRows + q_slot * Smem::kRowData);
      const int32_t* rowids = reinterpret_cast<const int32_t*>(rowdata + 2 * kTile);
      const bool full = t >= tf_lo && t < tf_hi;

      if (!p_wave && active_prev)
        finish_dk(x, smem + Smem::kQ + q_prev * Smem::kTileBytes,
                  reinterpret_cast<const float*>(smem + Smem::kRows + q_prev * Smem::kRowData) + kTile,
                  exchange + ((step - 1) & 1) * Smem::kSlotBytes);

      // 8 * UNITS * KSTEPS / 8 MFMAs per wavefront, S = Q K^T (P wave) or dP = dO V^T (S wave), the
      // 32-row units interleaved; operand reads run four ahead of the MFMAs
      const char* rows_a = p_wave ? qtile : dotile;
      if (active) {
#pragma unroll
        for (int mt = 0; mt < UNITS; mt++)
#pragma unroll
          for (int i = 0; i < 16; i++) x[mt][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++)
#pragma unroll
          for (int mt = 0; mt < UNITS; mt++)
            x[mt] = Tr::mfma(*reinterpret_cast<const vec8*>(rows_a + 32 * mt * RB + nat_off[ks]), frag[ks], x[mt]);
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < UNITS * KSTEPS - 4; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      }

      if (p_wave && active) {
        // operands of dV's first unit, requested before the element-wise work
        vec8 ta[2][DT];
#pragma unroll
        for (int st = 0; st < 2; st++)
#pragma unroll
          for (int dt = 0; dt < DT; dt++)
            ta[st][dt] = tr_read_a_swz<Tr>(dotile + 16 * st * RB, tr_off[dt][0], tr_off[dt][1]);
        vec8 pb[UNITS][2];
        char* pslot = exchange + (step & 1) * Smem::kSlotBytes;
#pragma unroll
        for (int mt = 0; mt < UNITS; mt++) {
          f32x16& sc = x[mt];
          if (!full)  // raw scores: masked -> -inf, so that P = exp2(-inf) = 0 (scale_log2_abs > 0)
            mask_c_tile<false>(sc, rowids, rowids + kTile, 32 * mt, qr0, h, kvseg, kvpos, col_lo,
                               col_width, -INFINITY);
#pragma unroll
          for (int g4 = 0; g4 < 4; g4++) {
            const float4 l4 = *reinterpret_cast<const float4*>(rowdata + 32 * mt + 8 * g4 + 4 * h);
            sc[4 * g4 + 0] = fast_exp2(__builtin_fmaf(sc[4 * g4 + 0], p.scale_log2_abs, -l4.x));
            sc[4 * g4 + 1] = fast_exp2(__builtin_fmaf(sc[4 * g4 + 1], p.scale_log2_abs, -l4.y));
            sc[4 * g4 + 2] = fast_exp2(__builtin_fmaf(sc[4 * g4 + 2], p.scale_log2_abs, -l4.z));
            sc[4 * g4 + 3] = fast_exp2(__builtin_fmaf(sc[4 * g4 + 3], p.scale_log2_abs, -l4.w));
          }
#pragma unroll
          for (int st = 0; st < 2; st++) {
            pb[mt][st] = pack8<Tr>(sc[8 * st + 0], sc[8 * st + 1], sc[8 * st + 2], sc[8 * st + 3],
                                   sc[8 * st + 4], sc[8 * st + 5], sc[8 * st + 6], sc[8 * st + 7]);
            const uint4 e = make_uint4(F16::pack2(sc[8 * st + 0], sc[8 * st + 1]), F16::pack2(sc[8 * st + 2], sc[8 * st + 3]),
                                       F16::pack2(sc[8 * st + 4], sc[8 * st + 5]), F16::pack2(sc[8 * st + 6], sc[8 * st + 7]));
            *reinterpret_cast<uint4*>(pslot + (2 * mt + st) * 1024) = e;
          }
        }
        // dV^T += dO^T P
#pragma unroll
        for (int mt = 0; mt < UNITS; mt++) {
          vec8 tb[2][DT];
          if (mt + 1 < UNITS) {
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
              for (int dt = 0; dt < DT; dt++)
                tb[st][dt] = tr_read_a_swz<Tr>(dotile + (32 * (mt + 1) + 16 * st) * RB, tr_off[dt][0], tr_off[dt][1]);
          }
#pragma unroll
          for (int st = 0; st < 2; st++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) acc[dt] = Tr::mfma(ta[st][dt], pb[mt][st], acc[dt]);
          if (mt + 1 < UNITS) {
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
              for (int dt = 0; dt < DT; dt++) ta[st][dt] = tb[st][dt];
          }
        }
      }
      ep = e0;
      if (++sub == SUB) {
        sub = 0;
        li = li + 1 == n_live ? 0 : li + 1;
        e0 = live_list[li];
      }
      q_prev = q_slot;
      q_slot = (q_slot + 1) & 3;
      do_slot = do_slot == 2 ? 0 : do_slot + 1;
    }
    // the S wave still owes the last tile
    __syncthreads();
    if (!p_wave && ((ep >> (24 + wave)) & 1))
      finish_dk(x, smem + Smem::kQ + q_prev * Smem::kTileBytes,
                reinterpret_cast<const float*>(smem + Smem::kRows + q_prev * Smem::kRowData) + kTile,
                exchange + ((steps - 1) & 1) * Smem::kSlotBytes);
  }
  __syncthreads();  // the next chunk reuses the bookkeeping, the rings and the exchange slots
  }

  if (tid == 0) ticket = work.draw();
  // ---- epilogue: the P wave holds dV^T, the S wave dK^T (times the scale) ----------------------
  // A lane holds 4 consecutive head-dim elements of its kv row per register group, so storing from
  // the registers would touch 32 rows with 8 or 16 bytes each per instruction.  Each wavefront
  // instead passes its 32 x D tile through its own part of the LDS (the rings are free by now),
  // 128 head-dim columns at a time, and writes whole rows: 16 bytes per lane, consecutive lanes
  // consecutive chunks of a row.  Rows are swizzled by the row index so that neither side has bank
  // conflicts.
  {
    const bool dead = col_width == 0;  // padding keys: exact zeros (see the dQ kernel's epilogue)
    const float mul = p_wave ? 1.f : p.scale;
    char* base = p_wave ? p.dv : p.dk;
    const int64_t sb = p_wave ? p.dv_sb : p.dk_sb, sh = p_wave ? p.dv_sh : p.dk_sh, ss = p_wave ? p.dv_ss : p.dk_ss;
    constexpr int PC = D < 128 ? D : 128;  // columns per pass
    constexpr int kDtPerPass = PC / 32;
    const int esize = p.dkdv_f32 ? 4 : 2;
    const int row_bytes = PC * esize;             // 128, 256 or 512
    const int chunks = row_bytes / 16;            // 8, 16 or 32 per row
    char* stage = smem + wave * (32 * PC * 4);    // room for the fp32 case
    const int64_t tile_off = (int64_t)b * sb + (int64_t)kv_head * sh + (int64_t)(k0 + pair * 32) * ss;
#pragma unroll
    for (int pass = 0; pass < D / PC; pass++) {
      char* mine = stage + c * row_bytes;
      if (p.dkdv_f32) {
#pragma unroll
        for (int d = 0; d < kDtPerPass; d++)
#pragma unroll
          for (int g4 = 0; g4 < 4; g4++) {
            const f32x16& a = acc[pass * kDtPerPass + d];
            const int chunk = 8 * d + 2 * g4 + h;
            *reinterpret_cast<float4*>(mine + ((chunk ^ (c & (chunks - 1))) * 16)) =
                dead ? make_float4(0.f, 0.f, 0.f, 0.f)
                     : make_float4(a[4 * g4 + 0] * mul, a[4 * g4 + 1] * mul, a[4 * g4 + 2] * mul, a[4 * g4 + 3] * mul);
          }
      } else {
#pragma unroll
        for (int d = 0; d < kDtPerPass; d++)
#pragma unroll
          for (int g4 = 0; g4 < 4; g4++) {
            const f32x16& a = acc[pass * kDtPerPass + d];
            uint2 u;
            u.x = Tr::pack2(a[4 * g4 + 0] * mul, a[4 * g4 + 1] * mul);
            u.y = Tr::pack2(a[4 * g4 + 2] * mul, a[4 * g4 + 3] * mul);
            if (dead) u = make_uint2(0, 0);
            const int chunk = 4 * d + g4;
            *reinterpret_cast<uint2*>(mine + ((chunk ^ (c & (chunks - 1))) * 16) + 8 * h) = u;
          }
      }
      // 32 rows x `chunks` 16-byte pieces, 64 per instruction
      const int per_iter = 64 / chunks;  // rows per instruction: 8, 4 or 2
      for (int r0 = 0; r0 < 32; r0 += per_iter) {
        const int row = r0 + lane / chunks, chunk = lane % chunks;
        const uint4 v = *reinterpret_cast<const uint4*>(stage + row * row_bytes + ((chunk ^ (row & (chunks - 1))) * 16));
        if (k0 + pair * 32 + row < p.kv_len)
          *reinterpret_cast<uint4*>(base + (tile_off + (int64_t)row * ss) * esize + pass * row_bytes + chunk * 16) = v;
      }
    }
  }
  }  // the item has work
  } else if (tid == 0) {
    ticket = work.draw();
  }
  if (tid == 0) *next_item = work.resolve(ticket);
  __syncthreads();
  }  // items of this XCD
}

template <class K>
int reserve_lds(K kernel, int need, int bytes, LdsReservation* reservation, const char* what) {
  if (need > bytes)
    return fail(KVAX_EUNSUPPORTED, "%s needs %d bytes of LDS for tile bitmaps (limit %d): sequence too long",
                what, need, bytes);
  return reservation->ensure(kernel, bytes, what);
}

// dQ launch: NW wavefronts (32 query rows each) per work-group, WPS per SIMD.
template <class Tr, int D, int NW, int STAGES, int WPS = 2>
int launch_dq(BwdParams p, hipStream_t stream) {
  auto kernel = fa_bwd_dq_kernel<Tr, D, NW, WPS, STAGES>;
  static LdsReservation done;
  constexpr int kLimit = kLdsPerCu / (4 * WPS / NW);  // work-groups per compute unit share the LDS
  const int smem = DqSmem<D, STAGES>::kTotal + live_tiles_bytes(NW, p.n_kv_tiles);
  if (int rc = reserve_lds(kernel, smem, kLimit, &done, "the dQ kernel")) return rc;
  p.num_tiles = cdiv(p.q_len, NW * 32);
  p.total_items = ItemMap{p.batch * p.num_kv_heads, p.num_tiles, p.group}.grid();
  hipLaunchKernelGGL(kernel, dim3(p.total_items), dim3(NW * 64), smem, stream, p);
  return check_launch("fa_bwd_dq_kernel");
}

template <class Tr, int D>
int launch_bwd(BwdParams p, hipStream_t stream) {
  // a key sequence too long for the dQ kernel's largest configuration is refused before anything
  // is enqueued (the dK/dV kernel has no such limit)
  if (p.q_len > 0 && !(p.flags & KVAX_FA_SKIP_DQ)) {
    const int need = D > 128 ? DqSmem<D, 2>::kTotal + live_tiles_bytes(4, p.n_kv_tiles)
                             : DqSmem<D, 3>::kTotal + live_tiles_bytes(8, p.n_kv_tiles);
    if (need > kLdsPerCu)
      return fail(KVAX_EUNSUPPORTED, "the dQ kernel needs %d bytes of LDS for tile bitmaps (limit %d): "
                  "sequence too long", need, kLdsPerCu);
  }
  // tile summaries of both sequences (a few microseconds; needed by dQ and dK/dV)
  {
    TileSummaryJob jobs[2] = {{p.kv_pos, p.kv_seg, (void*)p.kv_tiles, p.kv_len},
                              {p.q_pos, p.q_seg, (void*)p.q_tiles, p.q_len}};
    int32_t* counters = tile_order_counters(p.order_ws, p.batch, cdiv(p.kv_len, DkdvCfg<D>::kKvRows));
    if (int rc = launch_tile_summaries(jobs, 2, p.batch, stream, counters)) return rc;
  }
  // dQ: two work-groups of four wavefronts per compute unit (each hides the other's prologue,
  // barriers and final stores) when the tile bitmaps fit beside the smaller ring, else one of eight;
  // at head_dim 256 (128 accumulator registers for dQ alone) one work-group of four, one per SIMD
  constexpr int kStagesSmall = D == 64 ? 3 : 2;
  using Cfg = DkdvCfg<D>;
  const bool run_dq = p.q_len > 0 && !(p.flags & KVAX_FA_SKIP_DQ);
  const bool run_dkdv = p.kv_len > 0 && !(p.flags & KVAX_FA_SKIP_DKDV);
  const bool dq_small =
      DqSmem<D, kStagesSmall>::kTotal + live_tiles_bytes(4, p.n_kv_tiles) <= kLdsHalfCu;
  // dK/dV runs one long work-group per compute unit: its light work items are dispatched last, by
  // decreasing number of live tiles, so that the launch does not end on a few long ones
  {
    const int items = cdiv(p.kv_len, Cfg::kKvRows);
    if (run_dkdv && items >= kMinOrderedItems && items <= kMaxOrderedItems &&
        (int64_t)items * (p.n_q_tiles + 2) < 0x7fffffff) {
      const TileOrderJob job{p.kv_tiles, p.q_tiles, p.order_ws, p.n_kv_tiles, p.n_q_tiles,
                             Cfg::kKvRows / kTileRows, items, 0};
      if (int rc = launch_tile_order(job, p.batch, stream)) return rc;
      p.dkdv_order = p.order_ws;
    }
  }
  if (run_dq) {
    if constexpr (D > 128) {
      if (int rc = launch_dq<Tr, D, 4, 2, 1>(p, stream)) return rc;
    } else {
      if (dq_small) {
        if (int rc = launch_dq<Tr, D, 4, kStagesSmall>(p, stream)) return rc;
      } else {
        if (int rc = launch_dq<Tr, D, 8, 3>(p, stream)) return rc;
      }
    }
  }
  // dK/dV: wavefronts in role pairs (see DkdvCfg)
  if (run_dkdv) {
    constexpr int NW = Cfg::kWaves;
    auto kernel = fa_bwd_dkdv_kernel<Tr, D>;
    static LdsReservation done;
    // live-tile bookkeeping for as many query tiles as the remaining LDS holds (a multiple of 64)
    constexpr int kLdsLimit = kLdsPerCu;
    int chunk = 64;
    while (chunk < p.n_q_tiles && DkdvSmem<D>::kTotal + live_tiles_bytes(NW, chunk * 2) <= kLdsLimit) chunk *= 2;
    p.list_tiles = min(chunk, max(p.n_q_tiles, 1));
    const int smem = DkdvSmem<D>::kTotal + live_tiles_bytes(NW, p.list_tiles);
    if (int rc = reserve_lds(kernel, smem, kLdsLimit, &done, "the dK/dV kernel")) return rc;
    p.num_tiles = cdiv(p.kv_len, Cfg::kKvRows);
    p.total_items = ItemMap{p.batch * p.num_kv_heads, p.num_tiles, 1}.grid();
    p.dkdv_queue = tile_order_counters(p.order_ws, p.batch, p.num_tiles) + p.batch;
    hipLaunchKernelGGL(kernel, dim3(min(p.total_items, kNumCus)), dim3(NW * 64), smem, stream, p);
    if (int rc = check_launch("fa_bwd_dkdv_kernel")) return rc;
  }
  return KVAX_OK;
}

}  // namespace
}  // namespace kvax

using namespace kvax;

static size_t delta_bytes(const kvax_fa_args* a) {
  return ((size_t)a->batch * a->num_heads * a->q_len * sizeof(float) + 15) / 16 * 16;
}

extern "C" size_t kvax_fa_bwd_workspace_bytes(const kvax_fa_args* a) {
  if (!a || a->batch < 0 || a->q_len < 0 || a->kv_len < 0 || a->num_heads < 0) return 0;
  // delta [batch, heads, q_len] fp32, the tile summaries of the kv and query sequences, and the
  // dispatch order of the dK/dV work items
  return delta_bytes(a) + tile_summary_bytes(a->batch, a->kv_len) + tile_summary_bytes(a->batch, a->q_len) +
         tile_order_bytes(a->batch, cdiv(a->kv_len, a->head_dim > 128 ? 64 : 128));
}

extern "C" int kvax_fa_bwd(const kvax_fa_args* a, void* workspace, size_t workspace_bytes,
                           kvax_stream_t stream_) {
  if (int rc = validate_fa_common(a)) return rc;
  // empty tensors (and the masks over an empty outer axis) may come with null pointers
  const bool has_q = a->batch > 0 && a->q_len > 0, has_kv = a->batch > 0 && a->kv_len > 0;
  if ((has_q && (!a->dout || !a->dq)) || (has_kv && (!a->dk || !a->dv)))
    return fail(KVAX_EINVAL, "null gradient pointer");
  if (a->bwd_query_block <= 0 || a->bwd_kv_block <= 0)
    return fail(KVAX_EINVAL, "backward block sizes must be positive");
  for (int i = 0; i < 4; i++)
    if ((has_q && !a->dq_mask[i]) || (has_kv && !a->dkdv_mask[i]))
      return fail(KVAX_EINVAL, "backward masks are missing");
  const int64_t* strides[] = {a->do_strides, a->dq_strides, a->dk_strides, a->dv_strides};
  for (auto s : strides)
    for (int i = 0; i < 3; i++)
      if (s[i] % 8) return fail(KVAX_EINVAL, "strides must be multiples of 8 elements (16 bytes)");
  for (auto s : strides)
    if (s[1] < 0 || s[1] >= (1 << 24))
      return fail(KVAX_EUNSUPPORTED, "sequence stride of %lld elements is outside [0, 2^24)", (long long)s[1]);
  const void* ptrs[] = {a->dout, a->dq, a->dk, a->dv};
  for (auto ptr : ptrs)
    if ((uintptr_t)ptr % 16) return fail(KVAX_EINVAL, "tensor pointers must be 16-byte aligned");
  const size_t need = kvax_fa_bwd_workspace_bytes(a);
  if (need > workspace_bytes || (need && !workspace))
    return fail(KVAX_EWORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if ((uintptr_t)workspace % 16) return fail(KVAX_EINVAL, "workspace must be 16-byte aligned");
  if (a->batch == 0) return KVAX_OK;

  BwdParams p{};
  p.q = (const char*)a->q, p.k = (const char*)a->k, p.v = (const char*)a->v;
  p.out = (const char*)a->out, p.dout = (const char*)a->dout;
  p.dq = (char*)a->dq, p.dk = (char*)a->dk, p.dv = (char*)a->dv;
  p.lse = a->lse;
  p.delta = (float*)workspace;
  p.kv_tiles = (const int4*)((char*)workspace + delta_bytes(a));
  p.q_tiles = (const int4*)((char*)workspace + delta_bytes(a) + tile_summary_bytes(a->batch, a->kv_len));
  p.n_kv_tiles = cdiv(a->kv_len, kTileRows);
  p.n_q_tiles = cdiv(a->q_len, kTileRows);
  p.order_ws = (int32_t*)((char*)p.q_tiles + tile_summary_bytes(a->batch, a->q_len));
  p.q_pos = a->q_pos, p.q_seg = a->q_seg, p.kv_pos = a->kv_pos, p.kv_seg = a->kv_seg;
  for (int i = 0; i < 4; i++) p.dq_mask[i] = a->dq_mask[i], p.dkdv_mask[i] = a->dkdv_mask[i];
  p.q_sb = a->q_strides[0], p.q_ss = a->q_strides[1], p.q_sh = a->q_strides[2];
  p.k_sb = a->k_strides[0], p.k_ss = a->k_strides[1], p.k_sh = a->k_strides[2];
  p.v_sb = a->v_strides[0], p.v_ss = a->v_strides[1], p.v_sh = a->v_strides[2];
  p.o_sb = a->o_strides[0], p.o_ss = a->o_strides[1], p.o_sh = a->o_strides[2];
  p.do_sb = a->do_strides[0], p.do_ss = a->do_strides[1], p.do_sh = a->do_strides[2];
  p.dq_sb = a->dq_strides[0], p.dq_ss = a->dq_strides[1], p.dq_sh = a->dq_strides[2];
  p.dk_sb = a->dk_strides[0], p.dk_ss = a->dk_strides[1], p.dk_sh = a->dk_strides[2];
  p.dv_sb = a->dv_strides[0], p.dv_ss = a->dv_strides[1], p.dv_sh = a->dv_strides[2];
  p.batch = a->batch, p.q_len = a->q_len, p.kv_len = a->kv_len;
  p.num_heads = a->num_heads, p.num_kv_heads = a->num_kv_heads;
  p.group = a->num_heads / a->num_kv_heads;
  p.bq = a->bwd_query_block, p.bk = a->bwd_kv_block;
  p.n_dq_blocks = cdiv(a->q_len, a->bwd_kv_block);
  p.n_kv_blocks = cdiv(a->kv_len, a->bwd_kv_block);
  p.dkdv_f32 = (a->flags & KVAX_FA_DKDV_F32) != 0;
  p.flags = a->flags;
  p.scale = a->scale;
  p.scale_log2 = a->scale * 1.4426950408889634f;
  p.scale_log2_abs = fmaxf(fabsf(a->scale), 1e-30f) * 1.4426950408889634f;
  p.k_sign = a->scale < 0.f ? 0x80008000u : 0u;
  hipStream_t stream = (hipStream_t)stream_;
  const bool bf16 = a->dtype == KVAX_BF16;
  if (a->head_dim == 256)
    return bf16 ? launch_bwd<Bf16, 256>(p, stream) : launch_bwd<F16, 256>(p, stream);
  if (a->head_dim == 128)
    return bf16 ? launch_bwd<Bf16, 128>(p, stream) : launch_bwd<F16, 128>(p, stream);
  return bf16 ? launch_bwd<Bf16, 64>(p, stream) : launch_bwd<F16, 64>(p, stream);
}
