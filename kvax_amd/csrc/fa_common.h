// Device-side building blocks shared by the flash-attention kernels (gfx950 only).
//
// MFMA operand layouts used throughout (wave64, v_mfma_f32_32x32x16_{bf16,f16}):
//   A (32 x 16):  lane l holds row  l % 32, k = 8 * (l / 32) + [0, 8)
//   B (16 x 32):  lane l holds col  l % 32, k = 8 * (l / 32) + [0, 8)
//   C (32 x 32):  lane l holds col  l % 32, rows 8 * (i / 4) + 4 * (l / 32) + i % 4, i in [0, 16)
// A C tile can therefore be fed back as a B operand whose contraction index is the C row
// index: k-slot e of half h in step s (s = 0, 1) is C register 8 * s + e, i.e. row
// 16 * s + 8 * (e / 4) + 4 * h + e % 4.  The matching A operand gathers those rows with two
// transposing LDS reads (ds_read_b64_tr_b16), see tr_read_a_swz().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

namespace kvax {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define KVAX_LDS(ptr, T) ((__attribute__((address_space(3))) T*)(ptr))

struct Bf16 {
  using vec8 = bf16x8;
  __device__ static __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static __forceinline__ float to_float(uint16_t bits) {
    return __builtin_bit_cast(float, (uint32_t)bits << 16);
  }
};

struct F16 {
  using vec8 = f16x8;
  __device__ static __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static __forceinline__ float to_float(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
  }
};

// Eight consecutive fp32 values -> one 8 x 16-bit MFMA operand.
template <class Tr>
__device__ __forceinline__ typename Tr::vec8 pack8(float a0, float a1, float a2, float a3,
                                                   float a4, float a5, float a6, float a7) {
  uint4 u = make_uint4(Tr::pack2(a0, a1), Tr::pack2(a2, a3), Tr::pack2(a4, a5), Tr::pack2(a6, a7));
  return __builtin_bit_cast(typename Tr::vec8, u);
}

// Transposing LDS read.  Within each group of 16 lanes, lane i passes the address of 4
// consecutive 16-bit elements; the 16 x 64-bit chunks form a 4 x 16 matrix (row = i / 4, columns
// 4 * (i % 4) + [0, 4)) and lane i receives column i of it.
__device__ __forceinline__ s16x4 ds_read_tr16(const void* lds_ptr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(KVAX_LDS(lds_ptr, s16x4));
}

// LDS reads through a 32-bit LDS address held in a register: with `addr` = per-lane part + compile-time
// constant the constant lands in the instruction's immediate offset and costs no vector add.
template <class T>
__device__ __forceinline__ T lds_load(uint32_t addr) {
  return *reinterpret_cast<__attribute__((address_space(3))) const T*>(addr);
}
__device__ __forceinline__ s16x4 ds_read_tr16_at(uint32_t addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<__attribute__((address_space(3))) s16x4*>(addr));
}

// v_exp_f32 / v_log_f32 without the denormal-range fix-ups of exp2f / log2f.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ int cdiv_dev(int a, int b) { return (a + b - 1) / b; }

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32); }

// max / sum of a value with the one held by lane ^ 32, through v_permlane32_swap_b32 (exchanges
// the upper half of one register with the lower half of another): one vector instruction where
// __shfl_xor goes through the LDS crossbar and makes the wave wait for its answer.
__device__ __forceinline__ void swap_halves(float x, float& a, float& b) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];  // [x.lo, x.lo] and [x.hi, x.hi]
  a = __builtin_bit_cast(float, r0);
  b = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float max_xor32(float x) {
  float a, b;
  swap_halves(x, a, b);
  return __builtin_fmaxf(a, b);
}
__device__ __forceinline__ float sum_xor32(float x) {
  float a, b;
  swap_halves(x, a, b);
  return a + b;
}

// Compile-time loop: f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N - 1>).
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Work distribution.  Work-groups are dealt round-robin to the 8 XCDs (work-group L runs on XCD
// L % 8, each XCD has its own L2), so the map from L to a work item decides both L2 sharing and
// balance.  Items are (group, tile rank, member): a group is one (batch, kv head) -- everything
// that reads the same K/V -- with `tiles` tiles ranked heaviest first and `members` query heads
// per tile.  With at least 8 groups each XCD owns whole groups (visited in an order that rotates
// from rank to rank, see decode()); with fewer (and 8 divisible by
// the count) the tiles of a group are dealt round-robin to the XCDs that share it, so that every
// XCD gets the same mix of heavy and light tiles; otherwise items are cut into 8 contiguous runs.
struct ItemMap {
  int groups, tiles, members;
  __host__ __device__ int mode() const { return groups >= 8 ? 0 : (8 % groups == 0 ? 1 : 2); }
  __host__ __device__ int grid() const {
    if (mode() == 0) return 8 * members * ((groups + 7) / 8) * tiles;
    if (mode() == 1) return 8 * members * ((tiles + 8 / groups - 1) / (8 / groups));
    return groups * tiles * members;
  }
  // false when work-group L has nothing to do
  __device__ __forceinline__ bool decode(int L, int& group, int& rank, int& member) const {
    const int x = L % 8, j = L / 8;
    if (mode() == 0) {
      const int per_xcd = (groups + 7) / 8;
      const int jm = j / members;
      member = j % members;
      rank = jm / per_xcd;
      // The work-groups of an XCD go to its four shader engines in turn (work-group j to engine
      // j % 4, measured), and an engine that is full holds back the ones behind it.  With a number
      // of items per rank that shares a factor with 4, an engine would get the same groups (batch
      // rows) at every rank, and rows differ in work: the groups are rotated from rank to rank so
      // that every engine sees all of them.
      const int per_rank = per_xcd * members;
      const int every = per_rank % 4 == 0 ? 1 : (per_rank % 2 == 0 ? 2 : 4);  // 4 / gcd(per_rank, 4)
      group = x + 8 * ((jm + rank / every) % per_xcd);
      return group < groups && rank < tiles;
    }
    if (mode() == 1) {
      const int share = 8 / groups;
      member = j % members;
      group = x / share;
      rank = x % share + share * (j / members);
      return rank < tiles;
    }
    const int total = groups * tiles * members;
    const int per = total / 8, rem = total % 8;
    int item = x * per + (x < rem ? x : rem) + j;
    member = item % members;
    item /= members;
    rank = item % tiles;
    group = item / tiles;
    return true;
  }
};


// Item queues of a launch whose work-groups stay on their compute units and take work items until
// none is left, instead of one work-group per item: the dK/dV kernel, whose items are long and take
// a whole compute unit.  (Within an XCD the hardware hands the work-groups of a launch to the four
// shader engines in strict rotation and in order, so a compute unit that becomes free waits until
// the rotation comes round to its engine, which it does not while an earlier work-group waits for
// room on another engine: measured, 6 to 12 % of that kernel's compute-unit time idle between
// work-groups.  The forward and dQ kernels, two short work-groups per compute unit, lose less to
// this - a compute unit holds one work-group instead of two for 9 % of a launch - and more to the
// registers such a loop keeps live: dQ 6 % slower with queues.)  One counter per XCD, zero at launch:
// ticket j of queue x stands for item 8 j + x, which is what work-group 8 j + x of a launch with one
// work-group per item would take, so the items of a group still meet in one L2.  A work-group whose
// queue has run out goes on with the next XCD's (XCDs differ by 5-10 % in speed within a launch):
// that gives up L2 sharing, but only at the end of the launch.  Used by one thread per work-group;
// every work-group ends when resolve() returns -1, and none waits for another.
struct ItemQueue {
  int32_t* counters;
  int total;  // items of the launch
  int queue;  // the queue this work-group currently draws from
  __device__ __forceinline__ int draw() const { return atomicAdd(counters + queue, 1); }
  // the item a ticket of the current queue stands for, moving on while that queue is exhausted
  __device__ __forceinline__ int resolve(int ticket) {
    for (int tries = 0;; tries++) {
      const int id = 8 * ticket + queue;
      if (id < total) return id;
      if (tries == 7) return -1;
      queue = (queue + 1) % 8;
      ticket = draw();
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Tile summaries {seg_min, seg_max, pos_min, pos_max} over non-padding rows (fa_tiles.hip).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int4 empty_summary() {
  return make_int4(0x7fffffff, -0x7fffffff - 1, 0x7fffffff, -0x7fffffff - 1);
}

// Summary of the rows held one per lane (valid == false lanes are ignored), reduced over the wave.
__device__ __forceinline__ int4 wave_summary(bool valid, int seg, int pos) {
  int4 s = empty_summary();
  if (valid) s = make_int4(seg, seg, pos, pos);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s.x = min(s.x, __shfl_xor(s.x, off));
    s.y = max(s.y, __shfl_xor(s.y, off));
    s.z = min(s.z, __shfl_xor(s.z, off));
    s.w = max(s.w, __shfl_xor(s.w, off));
  }
  return s;
}

// True when no query of summary `q` can attend any key of summary `k`: segment ranges are
// disjoint or every key position exceeds every query position.  Empty summaries never attend.
__device__ __forceinline__ bool cannot_attend(const int4& q, const int4& k) {
  return (k.y < q.x) | (k.x > q.y) | (k.z > q.w);
}

// A tile (or a wavefront's own rows) summarised in two parts: rows sharing the segment id of the
// first non-padding row, and all other non-padding rows.
struct TileParts {
  int4 a, b;
};

__device__ __forceinline__ TileParts wave_parts(bool valid, int seg, int pos) {
  const unsigned long long vm = __ballot(valid);
  const int first = vm ? (int)__ffsll((long long)vm) - 1 : 0;
  const int fseg = __shfl(seg, first);
  TileParts t;
  t.a = wave_summary(valid && seg == fseg, seg, pos);
  t.b = wave_summary(valid && seg != fseg, seg, pos);
  return t;
}

__device__ __forceinline__ bool parts_cannot_attend(const TileParts& q, const TileParts& k) {
  return cannot_attend(q.a, k.a) & cannot_attend(q.a, k.b) & cannot_attend(q.b, k.a) &
         cannot_attend(q.b, k.b);
}

// Summaries of the 64 tiles of bitmap word w, one per lane (those outside [t_lo, t_hi) are not read).
struct WordSummaries {
  TileParts parts;
  bool have;
};
__device__ __forceinline__ WordSummaries load_word_summaries(const int4* tiles, int w, int t_lo, int t_hi, int lane) {
  WordSummaries s;
  const int t = w * 64 + lane;
  s.have = t >= t_lo && t < t_hi;
  s.parts.a = s.parts.b = empty_summary();
  if (s.have) {
    s.parts.a = tiles[2 * t];
    s.parts.b = tiles[2 * t + 1];
  }
  return s;
}

// Live-tile bitmaps.  Each wavefront marks, for the tiles [t_lo, t_hi) of the streamed axis, the
// ones its own rows (NP parts sets) can interact with; bit t % 64 of word t / 64 - word0.
// `bits` points at this wave's words in LDS.  `first`: the summaries of word word0, which callers
// request early, together with the other loads of their prologue.
template <bool MINE_IS_QUERY, int NP>
__device__ __forceinline__ void mark_live_tiles(const int4* tiles, const TileParts (&mine)[NP],
                                                int t_lo, int t_hi, unsigned long long* bits,
                                                int word0, int lane, const WordSummaries& first) {
  for (int w = word0; w * 64 < t_hi; w++) {
    const WordSummaries other = w == word0 ? first : load_word_summaries(tiles, w, t_lo, t_hi, lane);
    bool live = false;
    if (other.have) {
#pragma unroll
      for (int i = 0; i < NP; i++)
        live |= MINE_IS_QUERY ? !parts_cannot_attend(mine[i], other.parts) : !parts_cannot_attend(other.parts, mine[i]);
    }
    const unsigned long long m = __ballot(live);
    if (lane == 0) bits[w - word0] = m;
  }
}

// Compacts the NW per-wave bitmaps into a list of the tiles that are live for at least one
// wavefront: entry = tile index | (mask of the waves it is live for) << 24, in ascending tile order
// (DESCENDING: highest tile first).  Executed by one wavefront; the number of entries is written
// to *count.
template <int NW, bool DESCENDING = false>
__device__ __forceinline__ void compact_live_tiles(const unsigned long long* bits, int words, int word0,
                                                   uint32_t* list, int* count, int lane) {
  static_assert(NW <= 8, "the wave mask is stored in the top byte of an entry");
  int n = 0;
  for (int k = 0; k < words; k++) {
    const int w = DESCENDING ? words - 1 - k : k;
    unsigned long long any = 0;
    uint32_t waves = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) {
      const unsigned long long m = bits[i * words + w];
      any |= m;
      waves |= (uint32_t)((m >> lane) & 1) << i;
    }
    // entries of this word before the lane's own: set bits below it (ascending) or above it
    const unsigned long long before = DESCENDING ? (any >> lane) >> 1 : any & ((1ull << lane) - 1);
    if ((any >> lane) & 1)
      list[n + __popcll(before)] = (uint32_t)((word0 + w) * 64 + lane) | (waves << 24);
    n += __popcll(any);
  }
  if (lane == 0) *count = n;
}

// LDS of a gfx950 compute unit, and the share of each work-group when two run per compute unit.
constexpr int kNumCus = 256;  // compute units of the part this library is built for
constexpr int kLdsPerCu = 160 * 1024;
constexpr int kLdsHalfCu = kLdsPerCu / 2;

// LDS bytes for the live-tile bookkeeping of a range of at most `tiles` tiles.
__host__ __device__ constexpr int live_tiles_bytes(int nw, int tiles) {
  return 16 + nw * ((tiles + 63) / 64 + 1) * 8 + tiles * 4;
}

// Element mask of one 32 x 32 C tile whose columns are per-lane (the wave's own rows) and whose
// rows are 16 ids of the streamed tile (4 groups of 4 consecutive rows, row_ids = seg[], pos[]).
// ok = same segment & causal & streamed index inside the column's [c_lo, c_lo + c_width).
// COL_IS_QUERY: columns are queries (forward, dQ) or keys (dK/dV).  Branch-free.
template <bool COL_IS_QUERY>
__device__ __forceinline__ void mask_c_tile(f32x16& s, const int32_t* row_seg, const int32_t* row_pos,
                                            int row0, int row_global0, int h, int cseg, int cpos,
                                            int c_lo, unsigned c_width, float fill) {
#pragma unroll
  for (int g4 = 0; g4 < 4; g4++) {
    const int r = row0 + 8 * g4 + 4 * h;
    const int4 sg = *reinterpret_cast<const int4*>(row_seg + r);
    const int4 ps = *reinterpret_cast<const int4*>(row_pos + r);
    const int sgv[4] = {sg.x, sg.y, sg.z, sg.w};
    const int psv[4] = {ps.x, ps.y, ps.z, ps.w};
    const int rel = row_global0 + r - c_lo;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const bool causal = COL_IS_QUERY ? (cpos >= psv[j]) : (psv[j] >= cpos);
      const bool ok = (sgv[j] == cseg) & causal & ((unsigned)(rel + j) < c_width);
      s[4 * g4 + j] = ok ? s[4 * g4 + j] : fill;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Swizzled LDS tiles filled by asynchronous global -> LDS copies.
//
// A tile is ROWS rows of D 16-bit elements, unpadded (D * 2 bytes per row).  The 16-byte chunk c
// of row r lives at chunk position c ^ swz<D>(r).  With this permutation both access patterns
// of the kernels are bank-conflict free on the same tile: row reads (16 lanes = 16 consecutive
// rows, one chunk each) and 4-row transposing reads (ds_read_b64_tr_b16).  Unpadded rows also
// make each 1 KiB of the tile contiguous, which is what a wave-wide global_load_lds_dwordx4
// writes (lane i -> LDS base + 16 * i), so tiles are copied without passing through registers.
// ---------------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ int swz(int r) {
  // D == 128, 256: rows are one or two full turns of the 64 banks apart, so the chunk position
  // modulo 16 decides the banks and one 4-bit pattern serves both (at 256 it permutes the chunks
  // within each half of the row)
  if (D >= 128) return ((r & 3) << 2) | ((r >> 2) & 3);
  return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);  // D == 64: 8 chunks per row
}

// One asynchronous 16-byte-per-lane copy: the wave writes 1 KiB at LDS address `lds_addr`
// (wave-uniform), lane i providing its own global source address.  Completion is tracked by
// vmcnt; the data is visible to other waves after an s_waitcnt vmcnt + barrier.  Issued through
// inline assembly so that the compiler does not serialise later LDS reads against it.
// The statements write M0 without naming it as a clobber: M0 is a reserved register for this
// target (clang rejects it in a clobber list with a warning and ignores it), the compiler never
// keeps a value live in it and loads it immediately before each use of its own (indirect register
// indexing, s_sendmsg, its LDS-DMA builtins) - none of which these kernels contain.
__device__ __forceinline__ void async_copy_b128(const void* gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr)
               : "memory");
}
// Same for 4 bytes per lane (256 B per wave).
__device__ __forceinline__ void async_copy_b32(const void* gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(gptr)
               : "memory");
}

// s_waitcnt vmcnt(N) leaving the other counters alone (gfx9 encoding: vmcnt = bits 3:0 and
// 15:14, expcnt = 6:4, lgkmcnt = 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// Same with a wave-uniform 64-bit base address (held in SGPRs) plus a 32-bit per-lane byte offset:
// no vector ALU work per copy.
__device__ __forceinline__ void async_copy_b128(const char* sbase, uint32_t lane_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off),
               "s"(sbase)
               : "memory");
}

// Copies rows [row0, row0 + ROWS) of a row-major global matrix (16-bit elements, D per row,
// `row_stride_bytes` between rows) into a swizzled LDS tile at LDS address `tile_addr`.  Rows at
// or beyond `limit` (>= 1) are replaced by row limit - 1: callers mask them out by index.
// Every wave issues ROWS * D * 2 / 1024 / NW copies; the per-lane part of the source address is
// computed once (in the constructor) and only one scalar base changes from tile to tile: scalar
// address arithmetic per copy is serial work of the issuing wave and showed up as a fifth of the
// kernels' time before it was reduced to one multiply per tile.
template <int ROWS, int D, int NW>
struct AsyncTileCopy {
  static constexpr int kRowsPerCopy = 1024 / (D * 2);  // 4 (D = 128) or 8 (D = 64)
  static constexpr int kCopies = ROWS / kRowsPerCopy;
  static constexpr int kPerWave = kCopies / NW;
  static constexpr int kChunks = D / 8;
  static_assert(kCopies % NW == 0, "copies must split evenly over the waves");
  // Copy j of a wave covers the rows (j * NW + wave) * kRowsPerCopy + [0, kRowsPerCopy).  Up to
  // head_dim 128 and with a multiple of four waves the swizzle term of a lane is the same in all of
  // them, so one per-lane offset serves every copy and the scalar base moves on instead (vector
  // registers are what the kernels run out of first).
  static constexpr bool kCompact = D <= 128 && NW % 4 == 0;
  static constexpr int kOffsets = kCompact ? 1 : kPerWave;
  uint32_t lane_off[kOffsets];  // (row of the lane within the tile) * stride + chunk * 16, per copy
  int64_t stride;
  int wave_u, lane_;

  // The whole tile must span less than 4 GiB (ROWS * row_stride_bytes < 2^32; the entry points
  // check it), so that one scalar base per tile plus 32-bit lane offsets address every copy.
  __device__ __forceinline__ AsyncTileCopy(int64_t row_stride_bytes, int wave, int lane)
      : stride(row_stride_bytes), wave_u(__builtin_amdgcn_readfirstlane(wave)), lane_(lane) {
    const int rin = lane / kChunks, pos = lane % kChunks;
#pragma unroll
    for (int j = 0; j < kOffsets; j++) {
      const int r = (j * NW + wave_u) * kRowsPerCopy + rin;
      lane_off[j] = (uint32_t)(r * row_stride_bytes) + (uint32_t)((pos ^ swz<D>(r)) * 16);
    }
  }

  __device__ __forceinline__ void operator()(const char* gbase, int row0, int limit, uint32_t tile_addr) const {
    part<0, kPerWave>(gbase, row0, limit, tile_addr);
  }
  // Rows [row0 + HF * ROWS / 2, + ROWS / 2) of the tile only, into their place in the tile at
  // `tile_addr` (the copies of a wave alternate over groups of rows, the first half of them lies in
  // the first half of the tile).
  template <int HF>
  __device__ __forceinline__ void half(const char* gbase, int row0, int limit, uint32_t tile_addr) const {
    static_assert(kPerWave % 2 == 0, "a wave's copies must split over the two halves of a tile");
    part<HF * (kPerWave / 2), (HF + 1) * (kPerWave / 2)>(gbase, row0, limit, tile_addr);
  }
  // row0 < limit
  template <int J0, int J1>
  __device__ __forceinline__ void part(const char* gbase, int row0, int limit, uint32_t tile_addr) const {
    const char* tile_base = gbase + (int64_t)row0 * stride;
    if (row0 + ROWS <= limit) {  // whole tile in range (uniform): scalar bases + fixed lane offsets
      const uint32_t lds = tile_addr + wave_u * 1024;
#pragma unroll
      for (int j = J0; j < J1; j++) {
        if constexpr (kCompact)
          async_copy_b128(tile_base + j * (NW * kRowsPerCopy) * stride, lane_off[0], lds + j * NW * 1024);
        else
          async_copy_b128(tile_base, lane_off[j], lds + j * NW * 1024);
      }
    } else {  // ragged tail: clamp each lane's row (32-bit offsets from the tile's base)
      int l = lane_;
      asm volatile("" : "+v"(l));  // keeps what follows from being computed ahead of a loop around the call
      const int rin = l / kChunks, pos = l % kChunks;
      const int last = limit - 1 - row0;
#pragma unroll
      for (int j = J0; j < J1; j++) {
        const int grp = j * NW + wave_u;
        const int r = grp * kRowsPerCopy + rin;
        const uint32_t off = (uint32_t)min(r, last) * (uint32_t)stride + (uint32_t)((pos ^ swz<D>(r)) * 16);
        async_copy_b128(tile_base, off, tile_addr + grp * 1024);
      }
    }
  }
};
template <int ROWS, int D, int NW>
constexpr int async_tile_copies_per_wave() {
  return ROWS / (1024 / (D * 2)) / NW;
}

// Per-lane byte offsets into a swizzled tile.
// Row read (natural MFMA operand): lane (c, h) reads elements [16 * ks + 8 * h, +8) of row
// `row_in_16 + 32 * kt`; nat_offset gives the offset for kt = 0, add 32 * kt * D * 2.
template <int D>
__device__ __forceinline__ int nat_offset(int row, int ks, int h) {
  return row * (D * 2) + ((((2 * ks) | h) ^ swz<D>(row)) << 4);
}
// Transposed operand gather (see tr_read_a): lane (g, i) of step `half` (0: first 4-row read,
// 1: second) for the 32-column block dt; add row0 * D * 2 for the row block (row0 % 16 == 0).
template <int D>
__device__ __forceinline__ int tr_offset(int lane, int dt, int half) {
  const int g = lane >> 4, i = lane & 15;
  const int row = 4 * (g >> 1) + (i >> 2) + 8 * half;
  const int chunk = 4 * dt + 2 * (g & 1) + ((i & 3) >> 1);
  return row * (D * 2) + ((chunk ^ swz<D>(row)) << 4) + (i & 1) * 8;
}
template <class Tr>
__device__ __forceinline__ typename Tr::vec8 tr_read_a_at(uint32_t addr_lo, uint32_t addr_hi) {
  s16x4 lo = ds_read_tr16_at(addr_lo);
  s16x4 hi = ds_read_tr16_at(addr_hi);
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(typename Tr::vec8, v);
}
template <class Tr>
__device__ __forceinline__ typename Tr::vec8 tr_read_a_swz(const char* tile_row0, int off_lo, int off_hi) {
  s16x4 lo = ds_read_tr16(tile_row0 + off_lo);
  s16x4 hi = ds_read_tr16(tile_row0 + off_hi);
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(typename Tr::vec8, v);
}

}  // namespace kvax
