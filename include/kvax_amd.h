/* C ABI of the MI355X (gfx950) kvax attention hot path.
 *
 * The reference reaches its device kernels through jax_triton's `jt.triton_call`; these entry
 * points are what a host binding (jax.ffi custom call, ctypes, cgo ...) would call instead.
 * All pointers are device pointers unless stated otherwise.  No entry point allocates, frees or
 * synchronises: work is enqueued on `stream` and scratch memory comes in through a workspace
 * argument whose size the matching *_workspace_bytes function reports.
 *
 * Every function returns 0 on success and a negative KVAX_E* code on failure; the message of the
 * last failure on the calling thread is available from kvax_last_error().
 */
#ifndef KVAX_AMD_H_
#define KVAX_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* kvax_stream_t; /* a hipStream_t (NULL = the null stream) */

enum {
  KVAX_OK = 0,
  KVAX_EINVAL = -1,       /* bad shape / flag / null pointer */
  KVAX_EUNSUPPORTED = -2, /* valid request that the kernels do not cover (e.g. head_dim 96) */
  KVAX_EWORKSPACE = -3,   /* workspace missing or too small */
  KVAX_ELAUNCH = -4       /* HIP reported a launch error */
};

enum { KVAX_BF16 = 0, KVAX_F16 = 1 };

/* Version of this ABI (bumped on any incompatible change) and last error text. */
int kvax_abi_version(void);
const char* kvax_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Block-mask builder.
 * Replaces the `jt.triton_call` launches of compute_attention_mask_kernel
 * (reference kvax/ops/mask_creator.py:280 and :296) together with the host pre/post-processing
 * around them (:212-259 padding and padding-id remap, :317-333 sentinel fix-ups), for up to
 * KVAX_MAX_MASKS masks over the same id arrays in one call -- create_attention_mask
 * (:377-490) needs three: forward, dQ (swapped block sizes) and dK/dV (kv-outer).
 * ------------------------------------------------------------------------------------------ */
#define KVAX_MAX_MASKS 4

typedef struct kvax_mask_desc {
  int32_t query_block_size;
  int32_t kv_block_size;
  int32_t kv_outer; /* 0: one entry per query block (forward, dQ); 1: per kv block (dK/dV) */
  int32_t reserved;
  /* Outputs, int32.  kv_outer == 0: [batch, 1, ceil(q_len / query_block_size)].
   * kv_outer == 1: [batch, num_q_shards, ceil(kv_len / kv_block_size)], bounds are query-block
   * indices local to the shard. */
  int32_t* lower;
  int32_t* upper;
  int32_t* lower_full;
  int32_t* upper_full;
} kvax_mask_desc;

/* q_pos/q_seg: int32 [batch, q_len]; kv_pos/kv_seg: int32 [batch, kv_len], contiguous.
 * num_q_shards > 1 describes context parallelism: the query axis is `num_q_shards` contiguous
 * shards (q_len and every query block size must divide evenly); it only changes kv-outer masks. */
size_t kvax_mask_workspace_bytes(int batch, int q_len, int kv_len, const kvax_mask_desc* masks,
                                 int num_masks);
int kvax_mask_build(const int32_t* q_pos, const int32_t* q_seg, const int32_t* kv_pos,
                    const int32_t* kv_seg, int batch, int q_len, int kv_len, int num_q_shards,
                    int skip_pad_tokens, const kvax_mask_desc* masks, int num_masks,
                    void* workspace, size_t workspace_bytes, kvax_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Flash attention, forward and backward.
 * kvax_fa_fwd replaces the `jt.triton_call` of flash_attention_forward_kernel
 * (reference kvax/ops/flash_attention_triton.py:1517-1540) and the padding / un-padding around it
 * (:1457-1472, :1543-1544); kvax_fa_bwd replaces the launches of attn_bwd_preprocess (:1692),
 * flash_attention_backward_kernel_dquery (:1740), flash_attention_backward_kernel_dkdv (:1778)
 * or the fused flash_attention_backward_kernel (:1819), and the reduction of dK/dV over the
 * query heads of a group (:1855-1868).
 *
 * Tensors are consumed in the public [batch, seq, heads, head_dim] layout through element
 * strides {batch, seq, head}; the head_dim axis must be contiguous and head_dim is 64, 128 or 256
 * (the reference's other sizes, :1397-1403, are zero-padded to these by the caller).  Sequence lengths need not
 * be multiples of the block sizes: tails are handled inside the kernels.  The reference's
 * assume_sequential_positions mode (causal test on token indices plus a per-shard offset,
 * :1421-1451) needs no kernel support: the caller passes those indices as q_pos / kv_pos.
 * ------------------------------------------------------------------------------------------ */
enum {
  KVAX_FA_DKDV_F32 = 1,  /* backward writes dk / dv as fp32 (the reference kernels' output type,
                            flash_attention_triton.py:1729-1730) instead of the dtype of q */
  /* Backward phase selection, for profiling one kernel at a time.  The reference's
   * context-parallel path has three launches (:1692 delta, :1740 dQ, :1778 dK/dV); here the dQ
   * kernel also produces delta (rowsum(O * dO), kept in the workspace for the dK/dV kernel), so
   * KVAX_FA_SKIP_DELTA is accepted and changes nothing.  Skipping a phase leaves its outputs
   * untouched; dK/dV alone reuses the delta a previous call left in the same workspace. */
  KVAX_FA_SKIP_DELTA = 16,
  KVAX_FA_SKIP_DQ = 32,
  KVAX_FA_SKIP_DKDV = 64,
  /* Forward only, a request that is ignored where it does not apply (head_dim other than 128, short
   * query sequences): run the forward as one work-group of four wavefronts per compute unit, each
   * wavefront with 64 query rows, so that every K / V operand read from LDS feeds two MFMAs, with
   * the matrix and vector instructions of the loop interleaved by hand.  Same results to rounding
   * (the running maximum is raised per 32 keys instead of per 64).  It is as fast as the default at
   * long dense sequences and slower on document masks (its wavefronts do not skip tiles one by
   * one); it exists to measure what halving the LDS traffic buys.  No counterpart in the reference. */
  KVAX_FA_FWD_WIDE = 128
};

typedef struct kvax_fa_args {
  const void* q;   /* [batch, q_len, num_heads, head_dim]     */
  const void* k;   /* [batch, kv_len, num_kv_heads, head_dim] */
  const void* v;   /* [batch, kv_len, num_kv_heads, head_dim] */
  void* out;       /* forward: output, like q.  backward: input (forward result) */
  float* lse;      /* [batch, num_heads, q_len] fp32, base-2 log-sum-exp of scale*log2(e)*logits;
                      forward output / backward input; 0 for rows that attend to nothing */
  const void* dout; /* backward only: like out */
  void* dq;         /* backward only: like q, dtype of q */
  void* dk;         /* backward only: like k; dtype of q, or fp32 with KVAX_FA_DKDV_F32 */
  void* dv;         /* backward only: like v; dtype of q, or fp32 with KVAX_FA_DKDV_F32 */
  const int32_t* q_pos;  /* [batch, q_len]  */
  const int32_t* q_seg;  /* [batch, q_len]  */
  const int32_t* kv_pos; /* [batch, kv_len] */
  const int32_t* kv_seg; /* [batch, kv_len] */
  /* block masks as produced by kvax_mask_build: {lower, upper, lower_full, upper_full} */
  const int32_t* fwd_mask[4];  /* [batch, ceil(q_len / fwd_query_block)], kv blocks of fwd_kv_block */
  const int32_t* dq_mask[4];   /* [batch, ceil(q_len / bwd_kv_block)], kv blocks of bwd_query_block */
  const int32_t* dkdv_mask[4]; /* [batch, ceil(kv_len / bwd_kv_block)], query blocks of bwd_query_block */
  int64_t q_strides[3];
  int64_t k_strides[3];
  int64_t v_strides[3];
  int64_t o_strides[3];
  int64_t do_strides[3];
  int64_t dq_strides[3];
  int64_t dk_strides[3];
  int64_t dv_strides[3];
  int32_t batch, q_len, kv_len, num_heads, num_kv_heads, head_dim;
  int32_t fwd_query_block, fwd_kv_block; /* granularity of fwd_mask */
  int32_t bwd_query_block, bwd_kv_block; /* granularity of dq_mask (swapped) and dkdv_mask */
  int32_t dtype;                         /* KVAX_BF16 or KVAX_F16 */
  int32_t flags;                         /* KVAX_FA_* bits */
  float scale;
  int32_t reserved;
} kvax_fa_args;

/* Workspaces (16-byte aligned device memory, contents undefined on entry, reusable right after the
 * call's work on `stream`):
 *   forward:  32 bytes per 64-row kv tile and batch row (tile summaries used to skip dead tiles),
 *             plus, for short query sequences, the fp32 partial results of the work-groups that
 *             share one key sequence (a function of the shapes only), plus, with KVAX_FA_FWD_WIDE,
 *             the lists of live kv tiles per 256 query rows;
 *   backward: delta [batch, num_heads, q_len] fp32, the tile summaries of the kv and the query
 *             sequence, the order in which the dK/dV kernel takes its work items and the counters of
 *             the queues it takes them from (cleared by the call itself). */
size_t kvax_fa_fwd_workspace_bytes(const kvax_fa_args* args);
size_t kvax_fa_bwd_workspace_bytes(const kvax_fa_args* args);
int kvax_fa_fwd(const kvax_fa_args* args, void* workspace, size_t workspace_bytes,
                kvax_stream_t stream);
int kvax_fa_bwd(const kvax_fa_args* args, void* workspace, size_t workspace_bytes,
                kvax_stream_t stream);

/* kvax_fa_fwd without a workspace argument, for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (there XLA owns every buffer).  Same arguments, kernels and results
 * as kvax_fa_fwd; the scratch memory is a buffer of KVAX_FA_FWD_STATIC_MAX_WORKSPACE bytes that the
 * library holds in device memory on every GPU it runs on until the process ends.  A call whose
 * kvax_fa_fwd_workspace_bytes() exceeds that size fails with KVAX_EWORKSPACE and enqueues nothing
 * (long key sequences in split mode are the only such case: 8 MiB cover 32 rows x 32 query heads
 * decoding against 128k keys).  The call allocates and frees nothing and does not synchronise.
 * The first call of each kernel variant (head_dim, dtype, regular / split / decoding shape class) on
 * a device makes the HIP runtime load that kernel and look up the scratch buffer's address: make one
 * call per variant outside stream capture first, as for any kernel that is to be captured.
 * All calls on one GPU share the buffer: calls that overlap in time on one GPU (different streams
 * or host threads) race; serialise them or use kvax_fa_fwd with separate workspaces. */
#define KVAX_FA_FWD_STATIC_MAX_WORKSPACE (8u << 20)
int kvax_fa_fwd_static(const kvax_fa_args* args, kvax_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KVAX_AMD_H_ */
