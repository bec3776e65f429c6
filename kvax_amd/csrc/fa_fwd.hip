// Flash-attention forward for gfx950 (FA2 online softmax, block-sparse document mask, GQA).
//
// Semantics: reference kvax/ops/flash_attention_triton.py:57-370 (three kv ranges per query
// block taken from the block mask: [lower, lower_full) and [upper_full, upper) apply the element
// mask, [lower_full, upper_full) is mask-free; base-2 online softmax with scale*log2(e) folded
// in; P rounded to the input dtype before P.V; lse = m + log2(l)).  Differences, all inside
// what the reference's tests treat as don't-care: padding tokens (segment id -1) attend to
// nothing and rows without any attendable key produce exact zeros (and lse 0).
//
// Design (not the reference's): the wavefront computes S^T = K Q^T so that each lane owns one
// query column of the 32x32 MFMA result.  Row max / row sum are then in-lane reductions plus a
// single exchange between the two half-waves, and the exponentiated tile is already in the
// B-operand layout of the second contraction O^T += V^T P^T -- P never goes through LDS.  V^T
// operands are gathered from the row-major V tile with transposing LDS reads.  K/V tiles reach
// LDS by asynchronous global->LDS copies (no registers involved) into a ring of swizzled stages,
// one or two tiles ahead of the one being consumed, and are shared by the work-group's 4 or 8
// wavefronts (128 or 256 query rows); the query heads of one GQA group run as neighbouring
// work-groups on one XCD so K/V tiles are served from that XCD's L2.  Tiles of the block-mask range
// in which no (query, key) pair can pass the element mask are dropped up front (fa_tiles.hip).
// Short query sequences (decoding) run in a split mode that divides the key sequence over
// work-groups and merges their partial results (see fa_fwd_kernel).
#include <type_traits>

#include "common.h"
#include "fa_common.h"

namespace kvax {
namespace {

constexpr int kTK = kTileRows;  // kv rows per LDS tile

constexpr float kRescaleStep = 8.f;  // log2 units

struct FwdParams {
  const char* q;
  const char* k;
  const char* v;
  char* out;
  float* lse;
  const int32_t* q_pos;
  const int32_t* q_seg;
  const int32_t* kv_pos;
  const int32_t* kv_seg;
  const int32_t* lower;
  const int32_t* upper;
  const int32_t* lower_full;
  const int32_t* upper_full;
  int64_t q_sb, q_ss, q_sh;
  int64_t k_sb, k_ss, k_sh;
  int64_t v_sb, v_ss, v_sh;
  int64_t o_sb, o_ss, o_sh;
  int batch, q_len, kv_len, num_heads, num_kv_heads, group;
  bool split_mode;
  int qbs, kbs, n_qblocks;
  int num_q_tiles, total_items;
  const int4* kv_tiles;  // tile summaries [batch, n_kv_tiles]
  int n_kv_tiles;
  const uint32_t* lists;  // wide kernel: live-tile lists of its query tiles (see TileListJob)
  int list_stride;        // words between two lists
  uint32_t q_sign;       // 0x80008000 when the scale is negative: Q is negated on load
  float scale_log2;      // |scale| * log2(e), > 0
  // split mode (short query sequences, see fa_fwd_kernel): rows are (query, head of the group)
  // pairs; work-group `split` of an item takes the kv tiles [split, split + 1) * split_tiles of the
  // item's range and leaves a partial result
  int num_splits, split_tiles;
  int num_parts;              // partial results per item: num_splits, or twice that in narrow mode
  int part_rows;              // rows per tile that have a partial (<= TQ)
  float* part_o;              // [items, num_parts, part_rows, D] unnormalised O
  float* part_ml;             // [items, num_parts, part_rows, 2] running max (base 2) and sum
};

template <int D, int STAGES>
struct FwdSmem {
  static constexpr int kTileBytes = kTK * D * 2;  // swizzled, unpadded
  static constexpr int kIdBytes = 2 * kTK * 4;    // seg + pos
  static constexpr int kStage = 2 * kTileBytes + kIdBytes;
  static constexpr int kTotal = STAGES * kStage;
};

// One work-group: NW wavefronts x (32 * MQ) query rows of one (batch, head); streams the live kv
// tiles through a STAGES-deep ring of LDS stages filled by asynchronous copies.
//
// SPLIT (short query sequences, e.g. decoding one token against a long key sequence, where one
// work-group per (batch, head) would leave most of the chip idle and read the keys serially): the
// rows of a work-group are (query, query head) pairs of one (batch, kv head) - all heads of a GQA
// group share the key tiles they stream - and the kv range of the block mask is cut into windows of
// split_tiles tiles, one work-group each (those beyond the end of the range have nothing to do), each
// leaving an unnormalised partial result that fa_fwd_combine_kernel merges.  Windows of one size
// for all rows of the batch keep the work-groups equally long when the rows are not.
// NARROW: split mode with at most 32 rows (decoding), where the four wavefronts share the arithmetic
// of every tile instead of the rows (see the constants below).
template <class Tr, int D, int MQ, int NW, int WPS, int STAGES, bool SPLIT, bool NARROW>
__global__ __launch_bounds__(NW * 64, WPS) void fa_fwd_kernel(const FwdParams p) {
  using vec8 = typename Tr::vec8;
  using Smem = FwdSmem<D, STAGES>;
  constexpr int TQ = NW * 32 * MQ;
  constexpr int KSTEPS = D / 16;  // contraction steps of S^T = K Q^T
  constexpr int DT = D / 32;      // 32-row tiles of O^T
  constexpr int RB = D * 2;       // bytes per tile row
  constexpr int kCopies = 2 * async_tile_copies_per_wave<kTK, D, NW>() + 1;  // per wave and tile
  static_assert(STAGES >= 2 && STAGES <= 4, "the loop below keeps STAGES - 1 tiles in flight");
  // NARROW (split mode with at most 32 rows, i.e. decoding): every wavefront takes the same rows and
  // a quarter of the arithmetic of a tile - wavefront w the key rows [32 (w & 1), +32) and, of
  // O^T += V^T P^T, the head-dim slices of half w >> 1 - instead of one wavefront working while three
  // wait.  The two key halves keep separate running maxima and leave separate partial results.
  static_assert(!NARROW || (SPLIT && NW == 4 && MQ == 1 && DT % 2 == 0), "narrow mode splits a tile four ways");
  constexpr int KT = NARROW ? 1 : 2;         // 32-key halves of a tile per wavefront
  constexpr int DTO = NARROW ? DT / 2 : DT;  // 32-row slices of O^T per wavefront
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;  // wave-uniform on purpose
  const int c = lane % 32, h = lane / 32;
  const int kt0 = NARROW ? (wave & 1) : 0, dt0 = NARROW ? (wave >> 1) * DTO : 0;

  // ---- work item: heads of a GQA group adjacent, long (late) query tiles first -------------
  int group, rank, g = 0, split = 0, item = 0;
  if (SPLIT) {
    static_assert(!SPLIT || MQ == 1, "split mode maps one row per lane");
    // kv heads vary fastest: in the usual [batch, seq, heads, dim] layout the work-groups dispatched
    // together then read neighbouring 2 * D bytes of the same key rows at about the same time
    int r = blockIdx.x;
    const int kvh = r % p.num_kv_heads;
    r /= p.num_kv_heads;
    split = r % p.num_splits;
    r /= p.num_splits;
    const int tile = r % p.num_q_tiles;
    group = (r / p.num_q_tiles) * p.num_kv_heads + kvh;
    item = group * p.num_q_tiles + tile;
    rank = p.num_q_tiles - 1 - tile;
  } else {
    const ItemMap items{p.batch * p.num_kv_heads, p.num_q_tiles, p.group};
    if (!items.decode(blockIdx.x, group, rank, g)) return;
  }
  const int q_tile = p.num_q_tiles - 1 - rank;
  const int kv_head = group % p.num_kv_heads;
  const int b = group / p.num_kv_heads;
  const int head = kv_head * p.group + g;  // split mode: first head of the group
  const int q0 = q_tile * TQ;              // split mode: in (query, head) pairs
  const int rows_total = SPLIT ? p.q_len * p.group : p.q_len;

  const int32_t* q_seg = p.q_seg + (int64_t)b * p.q_len;
  const int32_t* q_pos = p.q_pos + (int64_t)b * p.q_len;
  const int32_t* kv_seg = p.kv_seg + (int64_t)b * p.kv_len;
  const int32_t* kv_pos = p.kv_pos + (int64_t)b * p.kv_len;
  const char* qbase = p.q + ((int64_t)b * p.q_sb + (int64_t)head * p.q_sh) * 2;
  const char* kbase = p.k + ((int64_t)b * p.k_sb + (int64_t)kv_head * p.k_sh) * 2;
  const char* vbase = p.v + ((int64_t)b * p.v_sb + (int64_t)kv_head * p.v_sh) * 2;
  char* obase = p.out + ((int64_t)b * p.o_sb + (int64_t)head * p.o_sh) * 2;
  float* lse = p.lse + ((int64_t)b * p.num_heads + head) * p.q_len;

  // ---- kv range of the work-group from the block mask: union of [lower, upper) over the mask's
  // query blocks it covers, intersection of the full ranges (element units) ---------------------
  int lo = 0x7fffffff, hi = 0, flo = 0, fhi = 0x7fffffff;
  {
    const int qb0 = (SPLIT ? q0 / p.group : q0) / p.qbs;
    const int qb1 = min((SPLIT ? (q0 + TQ - 1) / p.group : q0 + TQ - 1) / p.qbs, p.n_qblocks - 1);
    for (int qb = qb0; qb <= qb1; qb++) {
      const int64_t mi = (int64_t)b * p.n_qblocks + qb;
      const int l_ = p.lower[mi] * p.kbs, u_ = p.upper[mi] * p.kbs;
      flo = max(flo, p.lower_full[mi] * p.kbs);
      fhi = min(fhi, p.upper_full[mi] * p.kbs);
      if (u_ > l_) {
        lo = min(lo, l_);
        hi = max(hi, u_);
      }
    }
  }
  hi = min(hi, p.kv_len);
  int t_lo = lo / kTK;
  int t_hi = hi > lo ? (hi + kTK - 1) / kTK : t_lo;
  if (SPLIT) {  // this work-group's window of the range
    t_lo = min(t_lo + split * p.split_tiles, t_hi);
    t_hi = min(t_lo + p.split_tiles, t_hi);
  }
  const int tf_lo = (flo + kTK - 1) / kTK, tf_hi = fhi / kTK;

  if (!SPLIT && t_hi <= t_lo) {
    // No row of the tile can attend to anything (padding queries): zeros for O and lse, and nothing
    // is read.  Whole rows, 16 bytes per lane.
    constexpr int kChunks = D * 2 / 16;
    const int rows = min(TQ, p.q_len - q0);
    for (int i = tid; i < rows * kChunks; i += NW * 64)
      *reinterpret_cast<uint4*>(obase + (int64_t)(q0 + i / kChunks) * p.o_ss * 2 + (i % kChunks) * 16) =
          make_uint4(0, 0, 0, 0);
    for (int i = tid; i < rows; i += NW * 64) lse[q0 + i] = 0.f;
    return;
  }

  // ---- per-lane query columns ------------------------------------------------------------
  // qrow: the lane's query index; lane_head: its query head (split mode: per lane).
  // Everything the prologue reads from memory that does not depend on another read - the lane's
  // ids, its row of the block mask, its Q fragments and the first 64 tile summaries - is requested
  // here in one go, before any of it is used: the reads then cost one trip to memory instead of
  // one after another (the prologue is a sixth of the forward's time on the 32k document workload).
  int qrow[MQ], lane_head[MQ], qseg[MQ], qpos[MQ], col_lo[MQ];
  bool row_in[MQ];
  unsigned col_width[MQ];
  TileParts mine[MQ];
  int lower_raw[MQ], upper_raw[MQ];
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    const int row = q0 + (NARROW ? qt : wave * MQ + qt) * 32 + c;
    row_in[qt] = row < rows_total;
    qrow[qt] = SPLIT ? row / p.group : row;
    lane_head[qt] = SPLIT ? head + row % p.group : head;
    const int qi = row_in[qt] ? qrow[qt] : 0;
    qseg[qt] = q_seg[qi];
    qpos[qt] = q_pos[qi];
    const int64_t mi = (int64_t)b * p.n_qblocks + qi / p.qbs;
    lower_raw[qt] = p.lower[mi];
    upper_raw[qt] = p.upper[mi];
  }

  // Q fragments (B operand of S^T = K Q^T): lane holds 8 consecutive head-dim elements per step.
  // A negative scale is folded into Q so that the softmax below can assume scale_log2 > 0.
  vec8 qf[MQ][KSTEPS];
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    const bool in = row_in[qt] && t_hi > t_lo;  // nothing to attend to: no reads
    const char* row = (SPLIT ? p.q + ((int64_t)b * p.q_sb + (int64_t)lane_head[qt] * p.q_sh) * 2 : qbase) +
                      (int64_t)(in ? qrow[qt] : 0) * p.q_ss * 2;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      uint4 u = make_uint4(0, 0, 0, 0);
      if (in) u = *reinterpret_cast<const uint4*>(row + (16 * ks + 8 * h) * 2);
      u.x ^= p.q_sign, u.y ^= p.q_sign, u.z ^= p.q_sign, u.w ^= p.q_sign;
      qf[qt][ks] = __builtin_bit_cast(vec8, u);
    }
  }
  const int4* kv_summaries = p.kv_tiles + 2 * (int64_t)b * p.n_kv_tiles;
  // (narrow mode walks every tile of its window: see below)
  const WordSummaries first_word =
      load_word_summaries(kv_summaries, t_lo >> 6, t_lo, NARROW ? t_lo : t_hi, lane);

#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    const bool in = row_in[qt];
    qseg[qt] = in ? qseg[qt] : -1;
    qpos[qt] = in ? qpos[qt] : 0;
    col_lo[qt] = 0;
    col_width[qt] = 0;  // padding / out-of-range rows attend to nothing
    const bool valid = in && qseg[qt] != -1;
    if (valid) {
      col_lo[qt] = lower_raw[qt] * p.kbs;
      // keys at or beyond kv_len are never attendable (their LDS rows hold a copy of the last row)
      col_width[qt] = (unsigned)max(min(upper_raw[qt] * p.kbs, p.kv_len) - col_lo[qt], 0);
    }
    mine[qt] = wave_parts(valid && col_width[qt] > 0, qseg[qt], qpos[qt]);
  }

  // ---- live tiles: each wave marks the kv tiles of [t_lo, t_hi) its rows can interact with; the
  // union is compacted into a list the work-group then walks -------------------------------------
  int* live_count = reinterpret_cast<int*>(smem + Smem::kTotal);
  unsigned long long* live_bits = reinterpret_cast<unsigned long long*>(smem + Smem::kTotal + 16);
  const int word0 = t_lo >> 6;
  const int words = t_hi > t_lo ? ((t_hi - 1) >> 6) - word0 + 1 : 0;
  const uint32_t* live_list = reinterpret_cast<const uint32_t*>(live_bits + NW * (cdiv_dev(p.n_kv_tiles, 64) + 1));
  // Narrow mode (decoding) skips the bookkeeping: a window of the key cache has few dead tiles - the
  // block mask already ends where the cache's padding begins - and the 4 us the list costs are a
  // tenth of such a work-group's time; every tile of the window is walked by all four wavefronts,
  // the element mask settles the rest, and the call needs no tile summaries at all.
  if (!NARROW) {
    mark_live_tiles<true, MQ>(kv_summaries, mine, t_lo, t_hi, live_bits + wave * words, word0, lane, first_word);
    __syncthreads();
    if (wave == 0)
      compact_live_tiles<NW>(live_bits, words, word0, const_cast<uint32_t*>(live_list), live_count, lane);
    __syncthreads();
  }
  const int n_live = NARROW ? max(t_hi - t_lo, 0) : *live_count;
  // entry j of the list: tile index | mask of the wavefronts it is live for << 24
  auto list_entry = [&](int j) -> uint32_t {
    return NARROW ? (uint32_t)(t_lo + j) | (0xFu << 24) : live_list[j];
  };
  const int i_lo = 0, i_hi = n_live;

  f32x16 o[DTO][MQ];
  float m_run[MQ], l_run[MQ];
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    m_run[qt] = -1e30f;
    l_run[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DTO; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) o[dt][qt][i] = 0.f;
  }

  if (i_hi > i_lo) {
    const float cs = p.scale_log2;  // > 0

    // per-lane LDS addresses of the operand reads in stage 0 (K rows / V rows of key half kt0): the
    // rest of an address - stage, key half, 16-row step - is a constant of the instruction
    const uint32_t smem_addr = (uint32_t)(uintptr_t)smem;
    // two copies of the loop body, one per stage of a two-stage ring (they do not fit the registers at
    // head_dim 256)
    constexpr bool kStaticStages = STAGES == 2 && D <= 128;
    // at head_dim 64 reads through the generic pointer measured 2 % faster: there the registers hold
    // offsets from the start of the LDS block, not addresses
    constexpr bool kAddresses = D >= 128;
    const uint32_t addr0 = kAddresses ? smem_addr : 0u;
    uint32_t nat_addr[KSTEPS], tr_addr[DTO][2];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      nat_addr[ks] = addr0 + 32 * kt0 * RB + nat_offset<D>(c, ks, h);
      // opaque to the optimiser, which would otherwise keep the summands and add them again per read
      // (only where the loop below exists once per stage: elsewhere a scalar stage offset is added per
      // read anyway, and the optimiser's own choice measured better)
      if constexpr (kStaticStages) asm volatile("" : "+v"(nat_addr[ks]));
    }
#pragma unroll
    for (int dt = 0; dt < DTO; dt++) {
      tr_addr[dt][0] = addr0 + Smem::kTileBytes + 32 * kt0 * RB + tr_offset<D>(lane, dt0 + dt, 0);
      tr_addr[dt][1] = addr0 + Smem::kTileBytes + 32 * kt0 * RB + tr_offset<D>(lane, dt0 + dt, 1);
      if constexpr (kStaticStages) asm volatile("" : "+v"(tr_addr[dt][0]), "+v"(tr_addr[dt][1]));
    }

    const int32_t* id_src = (wave & 1) ? kv_pos : kv_seg;
    const AsyncTileCopy<kTK, D, NW> copy_k(p.k_ss * 2, wave, lane), copy_v(p.v_ss * 2, wave, lane);
    auto issue = [&](int tile, int stage) {
      const uint32_t base = smem_addr + stage * Smem::kStage;
      copy_k(kbase, tile * kTK, p.kv_len, base);
      copy_v(vbase, tile * kTK, p.kv_len, base + Smem::kTileBytes);
      async_copy_b32(id_src + min(tile * kTK + lane, p.kv_len - 1),
                     __builtin_amdgcn_readfirstlane(base + 2 * Smem::kTileBytes + (wave & 1) * (kTK * 4)));
    };

    {
    // entries of the live list for iterations i ... i + kAhead (read ahead of their use); the ring
    // holds the tile being worked on and the kAhead tiles requested after it
    constexpr int kAhead = STAGES - 1;
    static_assert(kAhead >= 1 && kAhead <= 3 && kAhead * kCopies < 64, "prefetch distance");
    uint32_t e[kAhead + 1];
#pragma unroll
    for (int k = 0; k <= kAhead; k++) e[k] = i_lo + k < i_hi ? list_entry(i_lo + k) : 0;
#pragma unroll
    for (int k = 0; k < kAhead; k++)
      if (k == 0 || i_lo + k < i_hi) issue(e[k] & 0xffffff, k);

    // One iteration: tile i of the list, held in ring stage `stage_c`.  With a two-stage ring the
    // driver below alternates two copies of it with the stage as a compile-time constant, so that the
    // stage's LDS base goes into the immediate offsets of the operand reads instead of costing a
    // vector add per read (16 of the ~150 vector instructions of a tile).
    auto iteration = [&](int i, auto stage_c) {
      const int stage = stage_c;
      // tile i has landed once at most the copies of the tiles requested after it are outstanding
      const int later = min(kAhead - 1, i_hi - 1 - i);
      if (kAhead >= 3 && later >= 2) wait_vmcnt<(kAhead >= 3 ? 2 : 0) * kCopies>();
      else if (kAhead >= 2 && later >= 1) wait_vmcnt<(kAhead >= 2 ? 1 : 0) * kCopies>();
      else wait_vmcnt<0>();
      __syncthreads();
      const uint32_t e_next = i + kAhead + 1 < i_hi ? list_entry(i + kAhead + 1) : 0;
      // into the stage of tile i - 1, which every wavefront has left
      if (i + kAhead < i_hi) issue(e[kAhead] & 0xffffff, stage >= 1 ? stage - 1 : STAGES - 1);
      const uint32_t e0 = e[0];
      const int t = e0 & 0xffffff;

      if ((e0 >> (24 + wave)) & 1) {
        const int kv0 = t * kTK;
        const char* ktile = smem + stage * Smem::kStage;
        const int32_t* ids = reinterpret_cast<const int32_t*>(ktile + 2 * Smem::kTileBytes);

        // ---- S^T = K Q^T -----------------------------------------------------------------
        f32x16 s[KT][MQ];  // key half kt0 + kt
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
          for (int qt = 0; qt < MQ; qt++)
#pragma unroll
            for (int i = 0; i < 16; i++) s[kt][qt][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
          vec8 a[KT];
#pragma unroll
          for (int kt = 0; kt < KT; kt++)
            a[kt] = kAddresses ? lds_load<vec8>(nat_addr[ks] + stage * Smem::kStage + 32 * kt * RB)
                               : *reinterpret_cast<const vec8*>(ktile + 32 * kt * RB + nat_addr[ks]);
#pragma unroll
          for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int qt = 0; qt < MQ; qt++) s[kt][qt] = Tr::mfma(a[kt], qf[qt][ks], s[kt][qt]);
        }
        // issue order: operand reads run four ahead of the MFMAs that consume them
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < KT * KSTEPS - 4; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, MQ, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4 * MQ, 0);

        // ---- element mask outside the full range (raw scores; masked -> -inf) -------------
        if (!(t >= tf_lo && t < tf_hi)) {
#pragma unroll
          for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int qt = 0; qt < MQ; qt++)
              mask_c_tile<true>(s[kt][qt], ids, ids + kTK, 32 * (kt0 + kt), kv0, h, qseg[qt], qpos[qt],
                                col_lo[qt], col_width[qt], -INFINITY);
        }

        vec8 pb[KT][2][MQ];
        // ---- online softmax (per query column = per lane, halves combined once) ------------
#pragma unroll
        for (int qt = 0; qt < MQ; qt++) {
          float mx = s[0][qt][0];
#pragma unroll
          for (int kt = 0; kt < KT; kt++)
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[kt][qt][i]);
#ifdef KVAX_FWD_BPERMUTE
          mx = fmaxf(mx, xor32(mx));
#else
          mx = max_xor32(mx);
#endif
          // The running maximum only has to bound the scores loosely: it is raised (and O, l
          // rescaled: 64 multiplies per lane) only when some row's maximum has grown by more than
          // kRescaleStep, i.e. the exponentials below may reach 2^kRescaleStep instead of 1 - exact
          // in the final O = acc / l and lse = m + log2(l), and no loss for a floating-point P.
          // With a plain running maximum some of a wavefront's 32 rows raise it in most tiles.
          if (__any(mx * cs > m_run[qt] + kRescaleStep)) {
            const float m_new = fmaxf(m_run[qt], mx * cs);
            const float alpha = fast_exp2(m_run[qt] - m_new);
            l_run[qt] *= alpha;
#pragma unroll
            for (int dt = 0; dt < DTO; dt++)
#pragma unroll
              for (int i = 0; i < 16; i++) o[dt][qt][i] *= alpha;
            m_run[qt] = m_new;
          }
          const float m_use = m_run[qt];
          float sum = 0.f;
#pragma unroll
          for (int kt = 0; kt < KT; kt++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[kt][qt][i] = fast_exp2(__builtin_fmaf(s[kt][qt][i], cs, -m_use));
#pragma unroll
            for (int st = 0; st < 2; st++) {
              uint32_t w[4];
#pragma unroll
              for (int j = 0; j < 4; j++) {
                w[j] = Tr::pack2(s[kt][qt][8 * st + 2 * j], s[kt][qt][8 * st + 2 * j + 1]);
                sum += s[kt][qt][8 * st + 2 * j] + s[kt][qt][8 * st + 2 * j + 1];
              }
              pb[kt][st][qt] = __builtin_bit_cast(vec8, make_uint4(w[0], w[1], w[2], w[3]));
            }
          }
          l_run[qt] += sum;  // per half-wave partial; halves are added in the epilogue
        }

        // ---- O^T += V^T P^T ---------------------------------------------------------------
#pragma unroll
        for (int kt = 0; kt < KT; kt++)
#pragma unroll
          for (int st = 0; st < 2; st++)
#pragma unroll
            for (int dt = 0; dt < DTO; dt++) {
              const uint32_t at = stage * Smem::kStage + (32 * kt + 16 * st) * RB;
              const vec8 a = kAddresses ? tr_read_a_at<Tr>(tr_addr[dt][0] + at, tr_addr[dt][1] + at)
                                        : tr_read_a_swz<Tr>(smem + at, tr_addr[dt][0], tr_addr[dt][1]);
#pragma unroll
              for (int qt = 0; qt < MQ; qt++) o[dt][qt] = Tr::mfma(a, pb[kt][st][qt], o[dt][qt]);
            }
      }
#pragma unroll
      for (int k = 0; k < kAhead; k++) e[k] = e[k + 1];
      e[kAhead] = e_next;
    };
    if constexpr (kStaticStages) {
      for (int i = i_lo; i < i_hi; i += 2) {
        iteration(i, std::integral_constant<int, 0>{});
        if (i + 1 < i_hi) iteration(i + 1, std::integral_constant<int, 1>{});
      }
    } else {
      int stage = 0;
      for (int i = i_lo; i < i_hi; i++) {
        iteration(i, stage);
        stage = stage == STAGES - 1 ? 0 : stage + 1;
      }
    }
    }
  }

  // ---- split mode with several parts per item: leave the unnormalised partial result (narrow
  // mode: one per key half of every window, its head-dim slices written by two wavefronts) --------
  if (SPLIT && (NARROW || p.num_splits > 1)) {
    const int prow = (NARROW ? 0 : wave) * 32 + c;  // MQ == 1
    const float l_row = l_run[0] + xor32(l_run[0]);  // cross-lane: outside the divergent branch
    if (row_in[0] && prow < p.part_rows) {
      const int64_t part = ((int64_t)item * p.num_splits + split) * (NARROW ? 2 : 1) + kt0;
      const int64_t slot = part * p.part_rows + prow;
      float* po = p.part_o + slot * D + 32 * dt0;
#pragma unroll
      for (int dt = 0; dt < DTO; dt++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++)
          *reinterpret_cast<float4*>(po + 32 * dt + 8 * g4 + 4 * h) =
              make_float4(o[dt][0][4 * g4 + 0], o[dt][0][4 * g4 + 1], o[dt][0][4 * g4 + 2], o[dt][0][4 * g4 + 3]);
      // a row that may attend to nothing (padding) leaves an empty partial: its accumulator is not zero
      // when the block mask declares padding-against-padding blocks mask-free (masks built without
      // skipping padding), where the element mask, which is what excludes such rows, is not applied
      if (h == 0 && dt0 == 0)
        *reinterpret_cast<float2*>(p.part_ml + slot * 2) = make_float2(m_run[0], col_width[0] > 0 ? l_row : 0.f);
    }
    return;
  }

  // ---- epilogue: normalise, write O (query dtype) and lse --------------------------------
  if constexpr (!SPLIT && MQ == 1) {
    // A lane holds 4 consecutive head-dim elements of its query row per register group, so storing
    // from the registers would touch 32 rows with 8 bytes each per instruction.  Each wavefront
    // passes its 32 x D tile through its own part of the LDS (the tiles are done with) and writes
    // whole rows, 16 bytes per lane; rows are swizzled by the row index against bank conflicts.
    const float l = l_run[0] + xor32(l_run[0]);
    const bool alive = l > 0.f && col_width[0] > 0;  // padding / out-of-range rows stay zero
    const float inv = alive ? 1.f / l : 0.f;
    if (row_in[0] && h == 0) lse[qrow[0]] = alive ? m_run[0] + fast_log2(l) : 0.f;
    __syncthreads();  // every wavefront has read its last tile
    constexpr int kRowBytes = D * 2, kChunks = kRowBytes / 16, kRowsPerStore = 64 / kChunks;
    char* stage = smem + wave * (32 * kRowBytes);
    char* mine = stage + c * kRowBytes;
#pragma unroll
    for (int dt = 0; dt < DTO; dt++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        uint2 u;
        u.x = Tr::pack2(o[dt][0][4 * g4 + 0] * inv, o[dt][0][4 * g4 + 1] * inv);
        u.y = Tr::pack2(o[dt][0][4 * g4 + 2] * inv, o[dt][0][4 * g4 + 3] * inv);
        *reinterpret_cast<uint2*>(mine + (((4 * dt + g4) ^ (c & (kChunks - 1))) * 16) + 8 * h) = u;
      }
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += kRowsPerStore) {
      const int row = r0 + lane / kChunks, chunk = lane % kChunks;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + row * kRowBytes + ((chunk ^ (row & (kChunks - 1))) * 16));
      const int qr = q0 + wave * 32 + row;
      if (qr < p.q_len) *reinterpret_cast<uint4*>(obase + (int64_t)qr * p.o_ss * 2 + chunk * 16) = v;
    }
    return;
  }
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    const float l = l_run[qt] + xor32(l_run[qt]);
    const bool alive = l > 0.f && col_width[qt] > 0;  // padding / out-of-range rows stay zero
    const float inv = alive ? 1.f / l : 0.f;
    if (row_in[qt]) {
      char* row = (SPLIT ? p.out + ((int64_t)b * p.o_sb + (int64_t)lane_head[qt] * p.o_sh) * 2 : obase) +
                  (int64_t)qrow[qt] * p.o_ss * 2;
#pragma unroll
      for (int dt = 0; dt < DTO; dt++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          uint2 u;
          u.x = Tr::pack2(o[dt][qt][4 * g4 + 0] * inv, o[dt][qt][4 * g4 + 1] * inv);
          u.y = Tr::pack2(o[dt][qt][4 * g4 + 2] * inv, o[dt][qt][4 * g4 + 3] * inv);
          *reinterpret_cast<uint2*>(row + (32 * dt + 8 * g4 + 4 * h) * 2) = u;
        }
      if (h == 0)
        (SPLIT ? p.lse + ((int64_t)b * p.num_heads + lane_head[qt]) * p.q_len : lse)[qrow[qt]] =
            alive ? m_run[qt] + fast_log2(l) : 0.f;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Wide forward kernel: four wavefronts, one per SIMD, each with 64 query rows (two 32-row
// sub-tiles) of one (batch, head), i.e. 256 query rows per work-group and one work-group per
// compute unit.  Every K / V operand read from LDS feeds two MFMAs (one per sub-tile): reading 1 KiB
// of LDS per MFMA, as the 32-row kernels do, caps the matrix pipeline at about 70 % whatever else
// the wavefronts do, because the LDS delivers about 100 bytes per clock and compute unit.  With one
// wavefront per SIMD nobody else fills the gaps in a wavefront's instruction stream, so the loop
// is software-pipelined over half tiles of 32 keys and the order is written out: while the vector
// unit does the softmax of half j (scores computed one half step earlier), the matrix pipeline
// computes the scores of half j + 1 and, as the exponentials arrive, O^T += V^T P^T of half j -
// chunks of one MFMA, its share of the operand reads and four vector instructions, kept in place
// by scheduling fences (and, for instructions without side effects, by empty asm statements that
// use their results).
// Ring protocol (one barrier per tile, two stages): iteration i works on the second half of K(i),
// the first half of K(i + 1) and all of V(i); after the barrier at its top the copies of the second
// half of K(i + 1), of V(i + 1) with its ids and of the first half of K(i + 2) are issued into the
// rows nobody reads any more.  One loop body serves both stages: the registers that hold the operand
// addresses are moved to the other stage once per tile, everything else is an immediate offset.
// Every wavefront works on every tile of the work-group's list (built by launch_tile_lists for
// items of 256 rows): a tile that is live for another wavefront only lies outside the mask-free
// range, so the element mask turns all of its scores into -inf and P into zeros.
// ---------------------------------------------------------------------------------------------
template <class Tr, int D>
__global__ __launch_bounds__(256, 1) void fa_fwd_wide_kernel(const FwdParams p) {
  using vec8 = typename Tr::vec8;
  constexpr int NW = 4, MQ = 2, STAGES = 2;
  using Smem = FwdSmem<D, STAGES>;
  constexpr int TQ = NW * 32 * MQ;
  constexpr int KSTEPS = D / 16, DT = D / 32, RB = D * 2;
  constexpr int kCopies = 2 * async_tile_copies_per_wave<kTK, D, NW>() + 1;
  static_assert(KSTEPS == 8 && DT == 4, "the chunk plan below is laid out for head_dim 128");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int c = lane % 32, h = lane / 32;
  int group, rank, g;
  const ItemMap items{p.batch * p.num_kv_heads, p.num_q_tiles, p.group};
  if (!items.decode(blockIdx.x, group, rank, g)) return;
  const int q_tile = p.num_q_tiles - 1 - rank;
  const int kv_head = group % p.num_kv_heads, b = group / p.num_kv_heads;
  const int head = kv_head * p.group + g;
  const int q0 = q_tile * TQ;

  const int32_t* kv_seg = p.kv_seg + (int64_t)b * p.kv_len;
  const int32_t* kv_pos = p.kv_pos + (int64_t)b * p.kv_len;
  const char* qbase = p.q + ((int64_t)b * p.q_sb + (int64_t)head * p.q_sh) * 2;
  const char* kbase = p.k + ((int64_t)b * p.k_sb + (int64_t)kv_head * p.k_sh) * 2;
  const char* vbase = p.v + ((int64_t)b * p.v_sb + (int64_t)kv_head * p.v_sh) * 2;
  char* obase = p.out + ((int64_t)b * p.o_sb + (int64_t)head * p.o_sh) * 2;
  float* lse = p.lse + ((int64_t)b * p.num_heads + head) * p.q_len;

  const uint32_t* list = p.lists + ((int64_t)b * p.num_q_tiles + q_tile) * p.list_stride;
  const int n_live = (int)list[0], tf_lo = (int)list[1], tf_hi = (int)list[2];

  // ---- per-lane query columns (sub-tile qt: rows q0 + 64 * wave + 32 * qt + c) -----------------
  int qrow[MQ], qseg[MQ], qpos[MQ], col_lo[MQ];
  bool row_in[MQ];
  unsigned col_width[MQ];
  vec8 qf[MQ][KSTEPS];
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    qrow[qt] = q0 + (wave * MQ + qt) * 32 + c;
    row_in[qt] = qrow[qt] < p.q_len;
    const int qi = row_in[qt] ? qrow[qt] : 0;
    const int seg = p.q_seg[(int64_t)b * p.q_len + qi], pos = p.q_pos[(int64_t)b * p.q_len + qi];
    const int64_t mi = (int64_t)b * p.n_qblocks + qi / p.qbs;
    const int lower_raw = p.lower[mi], upper_raw = p.upper[mi];
    const char* row = qbase + (int64_t)qi * p.q_ss * 2;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      uint4 u = make_uint4(0, 0, 0, 0);
      if (row_in[qt]) u = *reinterpret_cast<const uint4*>(row + (16 * ks + 8 * h) * 2);
      u.x ^= p.q_sign, u.y ^= p.q_sign, u.z ^= p.q_sign, u.w ^= p.q_sign;
      // The fragments are only ever MFMA operands, which may come from the accumulation registers: put
      // them there for good (the vector registers are needed for the scores; left to itself the
      // register allocator parks the fragments in accumulation registers anyway, but copies them back
      // in front of every use).
      uint32_t a0, a1, a2, a3;
      asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a0) : "v"(u.x));
      asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a1) : "v"(u.y));
      asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a2) : "v"(u.z));
      asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a3) : "v"(u.w));
      qf[qt][ks] = __builtin_bit_cast(vec8, make_uint4(a0, a1, a2, a3));
    }
    qseg[qt] = row_in[qt] ? seg : -1;
    qpos[qt] = row_in[qt] ? pos : 0;
    col_lo[qt] = 0;
    col_width[qt] = 0;
    if (row_in[qt] && seg != -1) {
      col_lo[qt] = lower_raw * p.kbs;
      col_width[qt] = (unsigned)max(min(upper_raw * p.kbs, p.kv_len) - col_lo[qt], 0);
    }
  }

  f32x16 o[DT][MQ];
  float m_run[MQ], l_run[MQ];
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    m_run[qt] = -1e30f;
    l_run[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) o[dt][qt][i] = 0.f;
  }

  if (n_live > 0) {
    const float cs = p.scale_log2;  // > 0
    const uint32_t smem_addr = (uint32_t)(uintptr_t)smem;
    uint32_t nat_addr[KSTEPS], tr_addr[DT][2];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) nat_addr[ks] = smem_addr + nat_offset<D>(c, ks, h);
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      tr_addr[dt][0] = smem_addr + Smem::kTileBytes + tr_offset<D>(lane, dt, 0);
      tr_addr[dt][1] = smem_addr + Smem::kTileBytes + tr_offset<D>(lane, dt, 1);
    }
    const int32_t* id_src = (wave & 1) ? kv_pos : kv_seg;
    const AsyncTileCopy<kTK, D, NW> copy_k(p.k_ss * 2, wave, lane), copy_v(p.v_ss * 2, wave, lane);
    constexpr uint32_t kHalf = 32 * RB;  // bytes of 32 rows of a tile
    auto k_read = [&](int ks, uint32_t off) { return lds_load<vec8>(nat_addr[ks] + off); };
    auto v_read = [&](int dt, uint32_t off) { return tr_read_a_at<Tr>(tr_addr[dt][0] + off, tr_addr[dt][1] + off); };
#define KVAX_FENCE() __builtin_amdgcn_sched_barrier(0)
#define KVAX_ANCHOR(x) asm volatile("" : "+v"(x))

    // scores of 32 keys on their own (the first half of the first tile)
    auto scores_only = [&](f32x16 (&nxt)[MQ]) __attribute__((always_inline)) {
      f32x16 z;
#pragma unroll
      for (int i = 0; i < 16; i++) z[i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        const vec8 a = k_read(ks, 0);
#pragma unroll
        for (int qt = 0; qt < MQ; qt++) nxt[qt] = Tr::mfma(a, qf[qt][ks], ks == 0 ? z : nxt[qt]);
      }
    };

    // One half step.  cur: scores of this half (in), nxt: scores of the next half (out); voff: byte
    // offset of this half's V rows from where the V address registers point (the K address registers
    // point at the next half's rows).
    auto half_step = [&](f32x16 (&cur)[MQ], f32x16 (&nxt)[MQ], auto voff_c) __attribute__((always_inline)) {
      constexpr uint32_t voff = decltype(voff_c)::value;
      vec8 kop[KSTEPS], vop[2 * DT];
      uint32_t w[MQ][8];
      float sum0[MQ], sum1[MQ];
      // operand r of the half step's MFMA pairs: K rows of the next half (r < 8), then V^T of this
      // half (16-key step (r - 8) / 4, head-dim block (r - 8) % 4); read kAheadOps pairs ahead
      constexpr int kAheadOps = 3;
      auto read_operand = [&](auto r_c) __attribute__((always_inline)) {
        constexpr int r = decltype(r_c)::value;
        if constexpr (r < KSTEPS) kop[r] = k_read(r, 0);
        else if constexpr (r < KSTEPS + 2 * DT)
          vop[r - KSTEPS] = v_read((r - KSTEPS) % DT, voff + ((r - KSTEPS) / DT) * 16 * RB);
      };
      static_for<kAheadOps>([&](auto r_c) __attribute__((always_inline)) { read_operand(r_c); });
      KVAX_FENCE();
      // ---- row maxima of both sub-tiles, with the first score MFMAs of the next half behind them
      float mx[MQ];
      f32x16 z;
#pragma unroll
      for (int i = 0; i < 16; i++) z[i] = 0.f;
#pragma unroll
      for (int qt = 0; qt < MQ; qt++) {
        mx[qt] = __builtin_fmaxf(cur[qt][0], cur[qt][1]);
#pragma unroll
        for (int i = 2; i < 8; i += 2) mx[qt] = __builtin_fmaxf(__builtin_fmaxf(mx[qt], cur[qt][i]), cur[qt][i + 1]);
        nxt[qt] = Tr::mfma(kop[0], qf[qt][0], z);
        KVAX_ANCHOR(nxt[qt]);
        if (qt == 1) read_operand(std::integral_constant<int, kAheadOps>{});
        KVAX_FENCE();
      }
#pragma unroll
      for (int qt = 0; qt < MQ; qt++) {
#pragma unroll
        for (int i = 8; i < 16; i += 2) mx[qt] = __builtin_fmaxf(__builtin_fmaxf(mx[qt], cur[qt][i]), cur[qt][i + 1]);
        nxt[qt] = Tr::mfma(kop[1], qf[qt][1], nxt[qt]);
        KVAX_ANCHOR(nxt[qt]);
        if (qt == 1) read_operand(std::integral_constant<int, kAheadOps + 1>{});
        KVAX_FENCE();
      }
#pragma unroll
      for (int qt = 0; qt < MQ; qt++) mx[qt] = max_xor32(mx[qt]) * cs;
      // lazy running maxima (see fa_fwd_kernel): one test for both sub-tiles
      if (__any(mx[0] > m_run[0] + kRescaleStep || mx[1] > m_run[1] + kRescaleStep)) {
#pragma unroll
        for (int qt = 0; qt < MQ; qt++) {
          const float m_new = fmaxf(m_run[qt], mx[qt]);
          const float alpha = fast_exp2(m_run[qt] - m_new);
          l_run[qt] *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[dt][qt][i] *= alpha;
          m_run[qt] = m_new;
        }
      }
      const float m_use[MQ] = {m_run[0], m_run[1]};
      // vector instruction I of the 112 that turn the 2 x 16 scores into P (packed in w) and its row
      // sums: per group of 8 elements and sub-tile 4 x (fma, fma, exp, exp) then 4 packs - group 0 of
      // both sub-tiles, then group 1 -, and the 2 x 14 additions last
      auto valu_op = [&](auto i_c) __attribute__((always_inline)) {
        constexpr int I = decltype(i_c)::value;
        if constexpr (I < 80) {
          constexpr int grp = I / 40, qt = (I % 40) / 20, k = I % 20;
          if constexpr (k < 16) {
            constexpr int e = 8 * grp + 2 * (k / 4) + k % 2;
            if constexpr (k % 4 < 2) cur[qt][e] = __builtin_fmaf(cur[qt][e], cs, -m_use[qt]);
            else cur[qt][e] = fast_exp2(cur[qt][e]);
          } else {
            constexpr int j = 4 * grp + (k - 16);
            w[qt][j] = Tr::pack2(cur[qt][2 * j], cur[qt][2 * j + 1]);
          }
        } else if constexpr (I < 108) {
          constexpr int qt = (I - 80) / 14, e = (I - 80) % 14 + 2;
          if constexpr (e == 2) sum0[qt] = cur[qt][0] + cur[qt][2];
          else if constexpr (e == 3) sum1[qt] = cur[qt][1] + cur[qt][3];
          else if constexpr (e % 2 == 0) sum0[qt] += cur[qt][e];
          else sum1[qt] += cur[qt][e];
          if constexpr (I % 4 == 3) asm volatile("" : "+v"(sum0[qt]), "+v"(sum1[qt]));  // stay in this chunk
        }
      };
      // ---- chunks: MFMA pair index m = 2 .. 15 (scores of the next half up to 7, then O^T += V^T P^T
      // of this half), two chunks (one per sub-tile) each
      static_for<28>([&](auto c_c) __attribute__((always_inline)) {
        constexpr int ch = decltype(c_c)::value;
        constexpr int m = ch / 2 + 2, qt = ch % 2;
        if constexpr (m < KSTEPS) {
          nxt[qt] = Tr::mfma(kop[m], qf[qt][m], nxt[qt]);
          KVAX_ANCHOR(nxt[qt]);
        } else {
          constexpr int st = (m - 8) / DT, dt = (m - 8) % DT;
          const vec8 pb = __builtin_bit_cast(vec8, make_uint4(w[qt][4 * st], w[qt][4 * st + 1], w[qt][4 * st + 2], w[qt][4 * st + 3]));
          o[dt][qt] = Tr::mfma(vop[m - 8], pb, o[dt][qt]);
        }
        if constexpr (qt == 1) read_operand(std::integral_constant<int, m + kAheadOps>{});
        static_for<4>([&](auto j_c) __attribute__((always_inline)) {
          valu_op(std::integral_constant<int, 4 * ch + decltype(j_c)::value>{});
        });
        KVAX_FENCE();
      });
#pragma unroll
      for (int qt = 0; qt < MQ; qt++) l_run[qt] += sum0[qt] + sum1[qt];  // per half-wave partial
    };

    f32x16 sa[MQ], sb[MQ];  // scores of the first / second 32 keys of a tile
#pragma unroll
    for (int qt = 0; qt < MQ; qt++)
#pragma unroll
      for (int i = 0; i < 16; i++) sb[qt][i] = 0.f;
    uint32_t e0 = list[4], e1 = 1 < n_live ? list[5] : 0, e2 = 2 < n_live ? list[6] : 0;
    // prologue: first half of K(0), scores of the first 32 keys
    copy_k.template half<0>(kbase, (int)(e0 & 0xffffff) * kTK, p.kv_len, smem_addr);
    {
      const int tile = e0 & 0xffffff;
      copy_k.template half<1>(kbase, tile * kTK, p.kv_len, smem_addr);
      copy_v(vbase, tile * kTK, p.kv_len, smem_addr + Smem::kTileBytes);
      async_copy_b32(id_src + min(tile * kTK + lane, p.kv_len - 1),
                     __builtin_amdgcn_readfirstlane(smem_addr + 2 * Smem::kTileBytes + (wave & 1) * (kTK * 4)));
      if (1 < n_live) copy_k.template half<0>(kbase, (int)(e1 & 0xffffff) * kTK, p.kv_len, smem_addr + Smem::kStage);
    }
    // the first copies issued have landed: first half of K(0)
    if (1 < n_live) wait_vmcnt<kCopies>(); else wait_vmcnt<kCopies - async_tile_copies_per_wave<kTK, D, NW>() / 2>();
    __syncthreads();
    scores_only(sa);
    // The K address registers point at the second half of the iteration's own stage in its first half
    // step and at the first half of the other stage in its second; the V address registers at the
    // iteration's stage.  The updates are made opaque to the optimiser, which would otherwise keep the
    // first values and add the running offset again in front of every read.
    int to_other = Smem::kStage;  // from the stage of this iteration to the other one
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      nat_addr[ks] += kHalf;
      asm volatile("" : "+v"(nat_addr[ks]));
    }
    using Z = std::integral_constant<uint32_t, 0>;
    using H = std::integral_constant<uint32_t, kHalf>;

#pragma unroll 1
    for (int i = 0; i < n_live; i++) {
      // K(i), the first half of K(i + 1), V(i) have landed; everybody is done with iteration i - 1
      wait_vmcnt<0>();
      __syncthreads();
      const uint32_t e3 = i + 3 < n_live ? list[4 + i + 3] : 0;
      {
        const uint32_t mine = smem_addr + (to_other < 0 ? Smem::kStage : 0), other = mine + to_other;
        if (i + 1 < n_live) {
          const int tile = e1 & 0xffffff;
          copy_k.template half<1>(kbase, tile * kTK, p.kv_len, other);
          copy_v(vbase, tile * kTK, p.kv_len, other + Smem::kTileBytes);
          async_copy_b32(id_src + min(tile * kTK + lane, p.kv_len - 1),
                         __builtin_amdgcn_readfirstlane(other + 2 * Smem::kTileBytes + (wave & 1) * (kTK * 4)));
        }
        if (i + 2 < n_live) copy_k.template half<0>(kbase, (int)(e2 & 0xffffff) * kTK, p.kv_len, mine);
      }
      const int t = e0 & 0xffffff;
      const int kv0 = t * kTK;
      const int32_t* ids = reinterpret_cast<const int32_t*>(smem + (to_other < 0 ? Smem::kStage : 0) + 2 * Smem::kTileBytes);
      const bool full = t >= tf_lo && t < tf_hi;
      if (!full) {
#pragma unroll
        for (int qt = 0; qt < MQ; qt++)
          mask_c_tile<true>(sa[qt], ids, ids + kTK, 0, kv0, h, qseg[qt], qpos[qt], col_lo[qt], col_width[qt], -INFINITY);
      }
      half_step(sa, sb, Z{});  // K: second half of this stage
      // K addresses: to the first half of the other stage
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        nat_addr[ks] += to_other - (int)kHalf;
        asm volatile("" : "+v"(nat_addr[ks]));
      }
      if (!full) {
#pragma unroll
        for (int qt = 0; qt < MQ; qt++)
          mask_c_tile<true>(sb[qt], ids, ids + kTK, 32, kv0, h, qseg[qt], qpos[qt], col_lo[qt], col_width[qt], -INFINITY);
      }
      half_step(sb, sa, H{});  // (the scores computed here are not used after the last tile)
      // ... to its second half, and the V addresses to the other stage, for the next iteration
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        nat_addr[ks] += kHalf;
        asm volatile("" : "+v"(nat_addr[ks]));
      }
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
        tr_addr[dt][0] += to_other, tr_addr[dt][1] += to_other;
        asm volatile("" : "+v"(tr_addr[dt][0]), "+v"(tr_addr[dt][1]));
      }
      to_other = -to_other;
      e0 = e1, e1 = e2, e2 = e3;
    }
#undef KVAX_FENCE
#undef KVAX_ANCHOR
  }

  // ---- epilogue: normalise, write O (query dtype) and lse ----------------------------------------
#pragma unroll
  for (int qt = 0; qt < MQ; qt++) {
    const float l = sum_xor32(l_run[qt]);
    const bool alive = l > 0.f && col_width[qt] > 0;  // padding / out-of-range rows stay zero
    const float inv = alive ? 1.f / l : 0.f;
    if (row_in[qt]) {
      char* row = obase + (int64_t)qrow[qt] * p.o_ss * 2;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          uint2 u;
          u.x = Tr::pack2(o[dt][qt][4 * g4 + 0] * inv, o[dt][qt][4 * g4 + 1] * inv);
          u.y = Tr::pack2(o[dt][qt][4 * g4 + 2] * inv, o[dt][qt][4 * g4 + 3] * inv);
          *reinterpret_cast<uint2*>(row + (32 * dt + 8 * g4 + 4 * h) * 2) = u;
        }
      if (h == 0) lse[qrow[qt]] = alive ? m_run[qt] + fast_log2(l) : 0.f;
    }
  }
}

// Merges the partial results of the split mode: one work-group per (item, row), one thread per
// head-dim element.  M = max m_s, L = sum l_s 2^(m_s - M), O = sum O_s 2^(m_s - M) / L,
// lse = M + log2 L; rows no split found a key for give zeros (and lse 0).
template <class Tr, int D>
__global__ __launch_bounds__(D) void fa_fwd_combine_kernel(const FwdParams p, int tile_rows) {
  const int prow = blockIdx.x % p.part_rows;
  const int item = blockIdx.x / p.part_rows;
  const int q_tile = item % p.num_q_tiles;
  const int group = item / p.num_q_tiles;
  const int row = q_tile * tile_rows + prow;
  if (row >= p.q_len * p.group) return;
  const int kv_head = group % p.num_kv_heads, b = group / p.num_kv_heads;
  const int qi = row / p.group, head = kv_head * p.group + row % p.group;
  const int d = threadIdx.x;
  const int64_t slot0 = (int64_t)item * p.num_parts * p.part_rows + prow;
  float m = -1e30f;
#pragma unroll 8
  for (int s = 0; s < p.num_parts; s++) m = fmaxf(m, p.part_ml[(slot0 + (int64_t)s * p.part_rows) * 2]);
  float l = 0.f, acc = 0.f;
#pragma unroll 8
  for (int s = 0; s < p.num_parts; s++) {
    const int64_t slot = slot0 + (int64_t)s * p.part_rows;
    const float2 ml = *reinterpret_cast<const float2*>(p.part_ml + slot * 2);
    const float w = ml.y > 0.f ? fast_exp2(ml.x - m) : 0.f;
    l += ml.y * w;
    acc += p.part_o[slot * D + d] * w;
  }
  const bool alive = l > 0.f;
  const float value = alive ? acc / l : 0.f;
  // 16-bit stores: pairs of neighbouring threads would need a shuffle to store 32 bits; the tensor
  // is tiny in this mode
  uint16_t* out = reinterpret_cast<uint16_t*>(p.out + ((int64_t)b * p.o_sb + (int64_t)head * p.o_sh + (int64_t)qi * p.o_ss) * 2);
  out[d] = (uint16_t)(Tr::pack2(value, 0.f) & 0xffff);
  if (d == 0) p.lse[((int64_t)b * p.num_heads + head) * p.q_len + qi] = alive ? m + fast_log2(l) : 0.f;
}

// How a forward call is run: in split mode (see fa_fwd_kernel) when the query sequence is shorter
// than a work-group's 128 rows - the heads of a GQA group then fill the rows and share the key
// tiles - or when one work-group per 128 query rows and head would occupy less than the chip's
// 256 compute units.  The key sequence is cut into equal windows of at least four tiles, as many as
// make one resident set of work-groups if every range were full (two work-groups per compute unit,
// one at head_dim 256) and never more: work-groups beyond the resident set would start when the
// first ones end and double the time of the call (measured on 8 rows x 32k keys: 408 live
// work-groups of 64 tiles 0.162 ms, 792 of 32 tiles 0.171, 594 of 43 tiles 0.192).  Depends on the
// shapes only, so that the workspace can be sized up front.
constexpr int kSplitTileRows = 128;  // (query, head) rows per work-group in split mode
constexpr int kWideTileRows = 256;   // query rows per work-group of fa_fwd_wide_kernel
struct FwdPlan {
  bool split_mode = false;
  int num_splits = 1, split_tiles = 0;
  int num_parts = 1;  // partial results per item: twice num_splits in narrow mode (at most 32 rows)
  int part_rows = 0;
  size_t part_o_bytes = 0, part_ml_bytes = 0;
  // workspace layout: tile summaries of the kv sequence (not in narrow mode, which walks every tile
  // of its windows), the partial results of the split mode, the live-tile lists of the wide kernel
  bool narrow() const { return num_parts > num_splits; }
  bool wide = false;  // regular mode with fa_fwd_wide_kernel (on request): lists for items of 256 query rows
  size_t summary_bytes = 0, list_bytes = 0;
  size_t total_bytes() const { return summary_bytes + part_o_bytes + part_ml_bytes + list_bytes; }
};
FwdPlan plan_forward(int batch, int q_len, int kv_len, int num_heads, int num_kv_heads, int head_dim,
                     bool want_wide) {
  FwdPlan plan;
  if (batch <= 0 || q_len <= 0 || kv_len <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return plan;
  const int n_kv_tiles = cdiv(kv_len, kTileRows);
  plan.summary_bytes = tile_summary_bytes(batch, kv_len);
  if (want_wide && head_dim == 128) {  // lists of live tiles per 256 query rows, shared by the heads
    const size_t bytes = tile_list_bytes(batch, q_len, kWideTileRows, kv_len);
    if (bytes > 0 && bytes <= kMaxTileListBytes && live_tiles_bytes(8, n_kv_tiles) <= kLdsPerCu) {
      plan.wide = true;
      plan.list_bytes = bytes;
    }
  }
  const int64_t regular = (int64_t)batch * num_heads * cdiv(q_len, kSplitTileRows);
  // the ring of the four-wavefront configuration (see launch_fwd_auto) and its share of the LDS
  const int ring_bytes = (2 * kTK * head_dim * 2 + 2 * kTK * 4) * (head_dim == 64 ? 3 : 2);
  if (ring_bytes + live_tiles_bytes(4, n_kv_tiles) > (head_dim == 256 ? kLdsPerCu : kLdsHalfCu)) return plan;
  if (q_len >= kSplitTileRows && regular >= 256) return plan;
  plan.split_mode = true;
  plan.list_bytes = 0;
  plan.wide = false;
  const int64_t rows = (int64_t)q_len * (num_heads / num_kv_heads);
  const int64_t items = (int64_t)batch * num_kv_heads * ((rows + kSplitTileRows - 1) / kSplitTileRows);
  // windows of one size for every item, at most 64 per item
  const int64_t resident = (head_dim == 256 ? 1 : 2) * kNumCus;
  int64_t max_splits = items >= resident ? 1 : resident / items;
  max_splits = max_splits < 64 ? max_splits : 64;
  int window = cdiv(n_kv_tiles, (int)max_splits);
  window = window > 4 ? window : 4;
  plan.split_tiles = window;
  plan.num_splits = cdiv(n_kv_tiles, window);
  // narrow mode (see fa_fwd_kernel) where the key sequence is divided anyway: with a single window it
  // would only add the launch that merges the partial results
  plan.num_parts = plan.num_splits * (rows <= 32 && plan.num_splits > 1 ? 2 : 1);
  if (plan.num_parts > 1) {
    plan.part_rows = (int)(rows < kSplitTileRows ? rows : kSplitTileRows);
    const size_t slots = (size_t)items * plan.num_parts * plan.part_rows;
    plan.part_o_bytes = (slots * head_dim * sizeof(float) + 15) / 16 * 16;
    plan.part_ml_bytes = (slots * 2 * sizeof(float) + 15) / 16 * 16;
  }
  if (plan.narrow()) plan.summary_bytes = 0;
  return plan;
}

template <class Tr, int D, int MQ, int NW, int WPS, int STAGES = 3, bool SPLIT = false, bool NARROW = false>
int launch_fwd(const FwdParams& p0, hipStream_t stream) {
  FwdParams p = p0;
  constexpr int TQ = NW * 32 * MQ;
  static_assert(!SPLIT || TQ == kSplitTileRows, "plan_forward() sizes the partial results for this tile");
  if (SPLIT) {
    p.num_q_tiles = cdiv(p.q_len * p.group, TQ);
    p.total_items = p.batch * p.num_kv_heads * p.num_q_tiles * p.num_splits;
  } else {
    p.num_splits = p.num_parts = 1;
    p.num_q_tiles = cdiv(p.q_len, TQ);
    p.total_items = ItemMap{p.batch * p.num_kv_heads, p.num_q_tiles, p.group}.grid();
  }
  if (p.batch * p.num_heads * p.num_q_tiles == 0) return KVAX_OK;
  auto kernel = fa_fwd_kernel<Tr, D, MQ, NW, WPS, STAGES, SPLIT, NARROW>;
  const int smem = FwdSmem<D, STAGES>::kTotal + live_tiles_bytes(NW, p.n_kv_tiles);
  constexpr int kWgPerCu = (WPS * 4 / NW) > 0 ? (WPS * 4 / NW) : 1;
  constexpr int kMaxSmem = kLdsPerCu / kWgPerCu;
  if (smem > kMaxSmem)
    return fail(KVAX_EUNSUPPORTED, "kv_len %d needs %d bytes of LDS for tile bitmaps (limit %d)",
                p.kv_len, smem, kMaxSmem);
  static LdsReservation reservation;  // one per instantiation of this function template
  if (int rc = reservation.ensure(kernel, kMaxSmem, "the forward kernel")) return rc;
  hipLaunchKernelGGL(kernel, dim3(p.total_items), dim3(NW * 64), smem, stream, p);
  if (int rc = check_launch("fa_fwd_kernel")) return rc;
  if (SPLIT && p.num_parts > 1) {
    const int blocks = p.batch * p.num_kv_heads * p.num_q_tiles * p.part_rows;
    hipLaunchKernelGGL((fa_fwd_combine_kernel<Tr, D>), dim3(blocks), dim3(D), 0, stream, p, TQ);
    return check_launch("fa_fwd_combine_kernel");
  }
  return KVAX_OK;
}

template <class Tr, int D>
int launch_fwd_wide(const FwdParams& p0, hipStream_t stream) {
  FwdParams p = p0;
  p.num_splits = p.num_parts = 1;
  p.num_q_tiles = cdiv(p.q_len, kWideTileRows);
  p.total_items = ItemMap{p.batch * p.num_kv_heads, p.num_q_tiles, p.group}.grid();
  if (p.batch * p.num_heads * p.num_q_tiles == 0) return KVAX_OK;
  auto kernel = fa_fwd_wide_kernel<Tr, D>;
  constexpr int smem = FwdSmem<D, 2>::kTotal;
  static LdsReservation reservation;
  if (int rc = reservation.ensure(kernel, kLdsPerCu, "the wide forward kernel")) return rc;
  hipLaunchKernelGGL(kernel, dim3(p.total_items), dim3(256), smem, stream, p);
  return check_launch("fa_fwd_wide_kernel");
}

// Two work-groups of four wavefronts per compute unit (each hides the other's prologue, barriers
// and final stores) whenever the tile bitmaps of the sequence fit beside the smaller ring;
// otherwise one work-group of eight wavefronts.
template <class Tr, int D>
int launch_fwd_auto(const FwdParams& p, hipStream_t stream) {
  if constexpr (D == 256) {
    // 128 accumulator registers for O and 64 for the Q fragments: one wavefront per SIMD, one
    // work-group of four per compute unit, two 64.5 KB stages
    if (p.split_mode && p.num_parts > p.num_splits) return launch_fwd<Tr, D, 1, 4, 1, 2, true, true>(p, stream);
    if (p.split_mode) return launch_fwd<Tr, D, 1, 4, 1, 2, true>(p, stream);
    return launch_fwd<Tr, D, 1, 4, 1, 2>(p, stream);
  } else {
    constexpr int kStagesSmall = D == 128 ? 2 : 3;
    if (p.split_mode && p.num_parts > p.num_splits) return launch_fwd<Tr, D, 1, 4, 2, kStagesSmall, true, true>(p, stream);
    if (p.split_mode) return launch_fwd<Tr, D, 1, 4, 2, kStagesSmall, true>(p, stream);
    const int small = FwdSmem<D, kStagesSmall>::kTotal + live_tiles_bytes(4, p.n_kv_tiles);
    if (small <= kLdsHalfCu) return launch_fwd<Tr, D, 1, 4, 2, kStagesSmall>(p, stream);
    return launch_fwd<Tr, D, 1, 8, 2, 3>(p, stream);
  }
}

}  // namespace

int validate_fa_common(const kvax_fa_args* a) {
  if (!a) return fail(KVAX_EINVAL, "args is null");
  if (a->batch < 0 || a->q_len < 0 || a->kv_len < 0 || a->num_heads <= 0 || a->num_kv_heads <= 0)
    return fail(KVAX_EINVAL, "bad batch/length/head counts");
  if (a->num_heads % a->num_kv_heads)
    return fail(KVAX_EINVAL, "num_heads %d is not a multiple of num_kv_heads %d", a->num_heads,
                a->num_kv_heads);
  if (a->head_dim != 64 && a->head_dim != 128 && a->head_dim != 256)
    return fail(KVAX_EUNSUPPORTED, "head_dim %d is not built (64, 128 and 256 are)", a->head_dim);
  if (a->dtype != KVAX_BF16 && a->dtype != KVAX_F16)
    return fail(KVAX_EUNSUPPORTED, "dtype %d is not supported (bf16 and f16 are)", a->dtype);
  if (a->flags & ~(KVAX_FA_DKDV_F32 | KVAX_FA_SKIP_DELTA | KVAX_FA_SKIP_DQ | KVAX_FA_SKIP_DKDV | KVAX_FA_FWD_WIDE))
    return fail(KVAX_EINVAL, "unknown bits in flags");
  // empty tensors may come with null pointers
  const bool has_q = a->batch > 0 && a->q_len > 0, has_kv = a->batch > 0 && a->kv_len > 0;
  if ((has_q && (!a->q || !a->out || !a->lse || !a->q_pos || !a->q_seg)) ||
      (has_kv && (!a->k || !a->v || !a->kv_pos || !a->kv_seg)))
    return fail(KVAX_EINVAL, "null tensor pointer");
  const int64_t* strides[] = {a->q_strides, a->k_strides, a->v_strides, a->o_strides};
  for (auto s : strides)
    for (int i = 0; i < 3; i++)
      if (s[i] % 8) return fail(KVAX_EINVAL, "strides must be multiples of 8 elements (16 bytes)");
  for (auto s : strides)
    if (s[1] < 0 || s[1] >= (1 << 24))
      return fail(KVAX_EUNSUPPORTED, "sequence stride of %lld elements is outside [0, 2^24)", (long long)s[1]);
  const void* ptrs[] = {a->q, a->k, a->v, a->out};
  for (auto ptr : ptrs)
    if ((uintptr_t)ptr % 16) return fail(KVAX_EINVAL, "tensor pointers must be 16-byte aligned");
  return KVAX_OK;
}

}  // namespace kvax

using namespace kvax;

extern "C" size_t kvax_fa_fwd_workspace_bytes(const kvax_fa_args* a) {
  if (!a || a->batch < 0 || a->kv_len < 0) return 0;
  // see FwdPlan
  return plan_forward(a->batch, a->q_len, a->kv_len, a->num_heads, a->num_kv_heads, a->head_dim,
                                    (a->flags & KVAX_FA_FWD_WIDE) != 0).total_bytes();
}

// Scratch memory of kvax_fa_fwd_static: one copy per GPU the library runs on, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress(); the device
// address it yields is what kernels and memory operations are given.
constexpr size_t kStaticScratchBytes = KVAX_FA_FWD_STATIC_MAX_WORKSPACE;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** ptr) {
  constexpr int kMaxDevices = 64;
  static std::mutex mutex;
  static void* address[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(KVAX_ELAUNCH, "cannot identify the current device");
  std::lock_guard<std::mutex> lock(mutex);
  if (!address[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(KVAX_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    address[dev] = p;
  }
  *ptr = address[dev];
  return KVAX_OK;
}

int fa_fwd_impl(const kvax_fa_args* a, void* workspace, kvax_stream_t stream_);

}  // namespace

extern "C" int kvax_fa_fwd(const kvax_fa_args* a, void* workspace, size_t workspace_bytes,
                           kvax_stream_t stream_) {
  if (int rc = validate_fa_common(a)) return rc;
  const size_t need = kvax_fa_fwd_workspace_bytes(a);
  if (need > workspace_bytes || (need && !workspace))
    return fail(KVAX_EWORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  return fa_fwd_impl(a, workspace, stream_);
}

extern "C" int kvax_fa_fwd_static(const kvax_fa_args* a, kvax_stream_t stream_) {
  if (int rc = validate_fa_common(a)) return rc;
  const size_t need = kvax_fa_fwd_workspace_bytes(a);
  if (need > kStaticScratchBytes)
    return fail(KVAX_EWORKSPACE, "this call needs %zu bytes of scratch memory, the library's static "
                "buffer holds %zu: use kvax_fa_fwd with a caller-provided workspace", need,
                kStaticScratchBytes);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // Nothing in the buffer has to start at zero: the tile summaries, the lists and, in split mode,
  // every partial result that is read are written by this call's own kernels first.
  return fa_fwd_impl(a, ws, stream_);
}

namespace {
int fa_fwd_impl(const kvax_fa_args* a, void* workspace, kvax_stream_t stream_) {
  if ((uintptr_t)workspace % 16) return fail(KVAX_EINVAL, "workspace must be 16-byte aligned");
  if (a->fwd_query_block <= 0 || a->fwd_kv_block <= 0)
    return fail(KVAX_EINVAL, "forward block sizes must be positive");
  if (a->q_len == 0 || a->batch == 0) return KVAX_OK;
  for (int i = 0; i < 4; i++)
    if (!a->fwd_mask[i]) return fail(KVAX_EINVAL, "forward mask is missing");
  FwdParams p{};
  p.q = (const char*)a->q;
  p.k = (const char*)a->k;
  p.v = (const char*)a->v;
  p.out = (char*)a->out;
  p.lse = a->lse;
  p.q_pos = a->q_pos;
  p.q_seg = a->q_seg;
  p.kv_pos = a->kv_pos;
  p.kv_seg = a->kv_seg;
  p.lower = a->fwd_mask[0];
  p.upper = a->fwd_mask[1];
  p.lower_full = a->fwd_mask[2];
  p.upper_full = a->fwd_mask[3];
  p.q_sb = a->q_strides[0], p.q_ss = a->q_strides[1], p.q_sh = a->q_strides[2];
  p.k_sb = a->k_strides[0], p.k_ss = a->k_strides[1], p.k_sh = a->k_strides[2];
  p.v_sb = a->v_strides[0], p.v_ss = a->v_strides[1], p.v_sh = a->v_strides[2];
  p.o_sb = a->o_strides[0], p.o_ss = a->o_strides[1], p.o_sh = a->o_strides[2];
  p.batch = a->batch, p.q_len = a->q_len, p.kv_len = a->kv_len;
  p.num_heads = a->num_heads, p.num_kv_heads = a->num_kv_heads;
  p.group = a->num_heads / a->num_kv_heads;
  p.qbs = a->fwd_query_block, p.kbs = a->fwd_kv_block;
  p.n_qblocks = cdiv(a->q_len, a->fwd_query_block);
  p.q_sign = a->scale < 0.f ? 0x80008000u : 0u;
  p.scale_log2 = fmaxf(fabsf(a->scale), 1e-30f) * 1.4426950408889634f;
  p.kv_tiles = (const int4*)workspace;
  p.n_kv_tiles = cdiv(a->kv_len, kTileRows);
  const FwdPlan plan = plan_forward(a->batch, a->q_len, a->kv_len, a->num_heads, a->num_kv_heads, a->head_dim,
                                    (a->flags & KVAX_FA_FWD_WIDE) != 0);
  p.split_mode = plan.split_mode;
  p.num_splits = plan.num_splits;
  p.num_parts = plan.num_parts;
  p.split_tiles = plan.split_tiles;
  p.part_rows = plan.part_rows;
  p.part_o = (float*)((char*)workspace + plan.summary_bytes);
  p.part_ml = (float*)((char*)p.part_o + plan.part_o_bytes);
  uint32_t* lists = plan.wide ? (uint32_t*)((char*)p.part_ml + plan.part_ml_bytes) : nullptr;
  p.lists = lists;
  p.list_stride = (int)tile_list_stride(p.n_kv_tiles);
  hipStream_t stream = (hipStream_t)stream_;
  if (!plan.wide) {  // too long for the largest configuration: refuse before anything is enqueued
    const int ring = (2 * kTK * a->head_dim * 2 + 2 * kTK * 4) * (a->head_dim == 256 ? 2 : 3);
    const int need = ring + live_tiles_bytes(a->head_dim == 256 ? 4 : 8, p.n_kv_tiles);
    if (need > kLdsPerCu)
      return fail(KVAX_EUNSUPPORTED, "kv_len %d needs %d bytes of LDS for tile bitmaps (limit %d)",
                  a->kv_len, need, kLdsPerCu);
  }
  if (!plan.narrow()) {  // the narrow mode does not read them
    TileSummaryJob job{a->kv_pos, a->kv_seg, workspace, a->kv_len};
    if (int rc = launch_tile_summaries(&job, 1, a->batch, stream)) return rc;
  }
  if (lists) {
    TileListJob job{a->q_pos, a->q_seg, {a->fwd_mask[0], a->fwd_mask[1], a->fwd_mask[2], a->fwd_mask[3]},
                    workspace, lists, a->q_len, a->kv_len, a->fwd_query_block, a->fwd_kv_block,
                    p.n_qblocks, p.n_kv_tiles, kWideTileRows / 32};
    if (int rc = launch_tile_lists(job, a->batch, stream)) return rc;
  }
  if (plan.wide)
    return a->dtype == KVAX_BF16 ? launch_fwd_wide<Bf16, 128>(p, stream) : launch_fwd_wide<F16, 128>(p, stream);
  const bool bf16 = a->dtype == KVAX_BF16;
  if (a->head_dim == 256)
    return bf16 ? launch_fwd_auto<Bf16, 256>(p, stream) : launch_fwd_auto<F16, 256>(p, stream);
  if (a->head_dim == 128)
    return bf16 ? launch_fwd_auto<Bf16, 128>(p, stream) : launch_fwd_auto<F16, 128>(p, stream);
  return bf16 ? launch_fwd_auto<Bf16, 64>(p, stream) : launch_fwd_auto<F16, 64>(p, stream);
}
}  // namespace
