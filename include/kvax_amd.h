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
  KVAX_EUNSUPPORTED = -2, /* valid request that the kernels do not cover (e.g. head_dim) */
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

#ifdef __cplusplus
}
#endif
#endif /* KVAX_AMD_H_ */
