/* CPU restatement of the reference block-mask builder.  TEST INFRASTRUCTURE ONLY: the product
 * library never links or loads this file.
 *
 * Follows the reference element by element, including its O(n_outer * inner_len) re-scan of the
 * inner sequence for every outer block:
 *   - padding of ragged tails and the remap of segment id -1 to (padded kv length + 1):
 *     kvax/ops/mask_creator.py:212-225 and :247-259 (done on the fly by elem_pos/elem_seg);
 *   - per-outer-block loop: kvax/ops/mask_creator.py:61-152;
 *   - sentinel post-processing: kvax/ops/mask_creator.py:317-333.
 *
 * Parity status: pinned by tests/test_oracle_mask.py (agreement with the numpy restatements, the
 * dense any/all definition on the reference test's input family, closed forms, invariants).
 */
#include <stdint.h>
#include <limits.h>

typedef struct {
    const int32_t* pos;
    const int32_t* seg;
    int len;        /* real length */
    int32_t pos_fill;
    int32_t pad_id; /* value that replaces -1 */
} seq_t;

static inline int32_t elem_pos(const seq_t* s, int i) { return i < s->len ? s->pos[i] : s->pos_fill; }
static inline int32_t elem_seg(const seq_t* s, int i) {
    int32_t v = i < s->len ? s->seg[i] : -1;
    return v == -1 ? s->pad_id : v;
}

static void block_minmax(const seq_t* s, int start, int size, int32_t* smin, int32_t* smax,
                         int32_t* pmin, int32_t* pmax) {
    int32_t a = INT32_MAX, b = INT32_MIN, c = INT32_MAX, d = INT32_MIN;
    for (int i = start; i < start + size; i++) {
        int32_t sg = elem_seg(s, i), ps = elem_pos(s, i);
        if (sg < a) a = sg;
        if (sg > b) b = sg;
        if (ps < c) c = ps;
        if (ps > d) d = ps;
    }
    *smin = a; *smax = b; *pmin = c; *pmax = d;
}

/* Outputs are [batch][n_outer] int32 (the reference's [batch, 1, n_outer]). Returns 0, or -1 on
 * bad arguments. */
int kvax_oracle_block_mask(const int32_t* q_pos, const int32_t* q_seg, const int32_t* kv_pos,
                           const int32_t* kv_seg, int batch, int q_len, int kv_len,
                           int query_block_size, int kv_block_size, int skip_pad_tokens,
                           int calculate_dkdv_mask, int32_t* lower_out, int32_t* upper_out,
                           int32_t* lower_full_out, int32_t* upper_full_out) {
    if (batch < 0 || q_len < 0 || kv_len < 0 || query_block_size <= 0 || kv_block_size <= 0) return -1;
    const int nq = (q_len + query_block_size - 1) / query_block_size;
    const int nk = (kv_len + kv_block_size - 1) / kv_block_size;
    const int32_t pad_id = (int32_t)(nk * kv_block_size + 1);
    const int n_outer = calculate_dkdv_mask ? nk : nq;
    const int n_inner = calculate_dkdv_mask ? nq : nk;
    const int o_bs = calculate_dkdv_mask ? kv_block_size : query_block_size;
    const int i_bs = calculate_dkdv_mask ? query_block_size : kv_block_size;
    for (int b = 0; b < batch; b++) {
        seq_t q = {q_pos + (long)b * q_len, q_seg + (long)b * q_len, q_len, -1, pad_id};
        seq_t kv = {kv_pos + (long)b * kv_len, kv_seg + (long)b * kv_len, kv_len, INT32_MAX, pad_id};
        const seq_t* outer = calculate_dkdv_mask ? &kv : &q;
        const seq_t* inner = calculate_dkdv_mask ? &q : &kv;
        for (int o = 0; o < n_outer; o++) {
            int32_t os_min, os_max, op_min, op_max;
            block_minmax(outer, o * o_bs, o_bs, &os_min, &os_max, &op_min, &op_max);
            const int osame = os_min == os_max;
            int32_t lower = n_inner, upper = 0, lower_full = n_inner, upper_full = 0;
            if (skip_pad_tokens && osame && os_min == pad_id) {
                lower = upper = lower_full = upper_full = 0;
            } else {
                for (int i = 0; i < n_inner; i++) {
                    int32_t is_min, is_max, ip_min, ip_max;
                    block_minmax(inner, i * i_bs, i_bs, &is_min, &is_max, &ip_min, &ip_max);
                    const int isame = is_min == is_max;
                    const int seg_overlap = is_min <= os_max && os_min <= is_max;
                    int attend_pos, full_pos;
                    if (!calculate_dkdv_mask) {
                        attend_pos = op_max >= ip_min;
                        full_pos = op_min >= ip_max;
                    } else {
                        attend_pos = ip_max >= op_min;
                        full_pos = ip_min >= op_max;
                    }
                    int attend = attend_pos && seg_overlap;
                    if (skip_pad_tokens && is_min == pad_id) attend = 0;
                    if (attend) {
                        if (i + 1 > upper) upper = i + 1;
                        if (i < lower) lower = i;
                    }
                    if (osame && isame && full_pos && attend) {
                        if (i + 1 > upper_full) upper_full = i + 1;
                        if (i < lower_full) lower_full = i;
                    }
                }
            }
            /* post-processing */
            if (lower == n_inner) lower = upper;
            if (lower_full == n_inner) lower_full = calculate_dkdv_mask ? upper : lower;
            if (upper_full < lower_full) upper_full = lower_full;
            const long idx = (long)b * n_outer + o;
            lower_out[idx] = lower;
            upper_out[idx] = upper;
            lower_full_out[idx] = lower_full;
            upper_full_out[idx] = upper_full;
        }
    }
    return 0;
}
