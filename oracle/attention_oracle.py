"""Dense masked attention and its VJP on the CPU.  TEST INFRASTRUCTURE ONLY.

Textbook ``softmax(mask(Q K^T * scale)) V`` with the element mask of the reference kernels
(kvax/ops/flash_attention_triton.py:31-54: same segment id AND ``q_pos >= kv_pos``) evaluated
densely, one (batch, head) at a time, in float64 by default.  Grouped-query attention maps query
head ``h`` to kv head ``h // (Hq // Hkv)`` (flash_attention_triton.py:196-197).  The backward is
the closed-form softmax-attention VJP (what flash_attention_triton.py:473-516 and :583-612
accumulate blockwise): ``dV = P^T dO``, ``dP = dO V^T``, ``dS = P * (dP - rowsum(dO*O))``,
``dQ = scale * dS K``, ``dK = scale * dS^T Q``.

Deliberate differences from the reference's *device* behaviour (both are don't-care regions for
the reference's own tests, which zero padding rows before comparing,
tests/test_attention.py:144-149,267-283): padding tokens (segment id -1) attend to nothing and are
attended by nothing, and a query row with no attendable key yields an exact zero row (and lse 0).

Parity status: pinned by tests/test_oracle_attention.py -- torch autograd on an independently
written dense graph, finite differences in float64, and closed forms (single key => O = V,
Q = 0 => mean of the allowed V rows, packed documents == per-document runs, GQA == repeated
heads, constant positions == bidirectional).
"""
from __future__ import annotations

import numpy as np

PADDING_SEGMENT_ID = -1


def element_mask(q_pos, q_seg, kv_pos, kv_seg):
    """[Sq, Sk] boolean for one batch row."""
    m = (q_seg[:, None] == kv_seg[None, :]) & (q_pos[:, None] >= kv_pos[None, :])
    m &= (q_seg != PADDING_SEGMENT_ID)[:, None]
    m &= (kv_seg != PADDING_SEGMENT_ID)[None, :]
    return m


def count_unmasked_pairs(q_pos, q_seg, kv_pos, kv_seg, row_block=2048):
    """Number of attendable (batch, q, kv) element pairs, counted exactly."""
    q_pos, q_seg = np.asarray(q_pos), np.asarray(q_seg)
    kv_pos, kv_seg = np.asarray(kv_pos), np.asarray(kv_seg)
    total = 0
    for b in range(q_pos.shape[0]):
        for r0 in range(0, q_pos.shape[1], row_block):
            sl = slice(r0, r0 + row_block)
            total += int(element_mask(q_pos[b, sl], q_seg[b, sl], kv_pos[b], kv_seg[b]).sum())
    return total


def _softmax_rows(s, mask):
    """Row softmax over allowed entries; rows with none allowed give zeros. Returns (p, lse)."""
    s = np.where(mask, s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    dead = ~np.isfinite(m)
    m = np.where(dead, 0.0, m)
    e = np.exp(s - m)
    l = e.sum(axis=-1, keepdims=True)
    p = e / np.where(dead, 1.0, l)
    lse = np.where(dead[:, 0], 0.0, m[:, 0] + np.log(np.where(dead, 1.0, l))[:, 0])
    return p, lse


def attention_forward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, scale, dtype=np.float64,
                      heads=None, row_block=4096):
    """q [B,Sq,Hq,D], k/v [B,Sk,Hkv,D] -> (out [B,Sq,Hq,Dv], lse [B,Hq,Sq]) in ``dtype``.

    ``lse`` is the natural-log sum-exp of the scaled, masked logits.  ``heads`` restricts the
    computation to a subset of query heads (others are left zero) so that long sequences can be
    spot-checked cheaply.
    """
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    B, Sq, Hq, _ = q.shape
    _, Sk, Hkv, Dv = v.shape
    G = Hq // Hkv
    out = np.zeros((B, Sq, Hq, Dv), dtype)
    lse = np.zeros((B, Hq, Sq), dtype)
    hs = range(Hq) if heads is None else heads
    for b in range(B):
        for r0 in range(0, Sq, row_block):
            sl = slice(r0, min(Sq, r0 + row_block))
            mask = element_mask(np.asarray(q_pos[b])[sl], np.asarray(q_seg[b])[sl],
                                np.asarray(kv_pos[b]), np.asarray(kv_seg[b]))
            for h in hs:
                s = (q[b, sl, h] @ k[b, :, h // G].T) * scale
                p, l = _softmax_rows(s, mask)
                out[b, sl, h] = p @ v[b, :, h // G]
                lse[b, h, sl] = l
    return out, lse


def attention_backward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, scale, dout, dtype=np.float64,
                       heads=None, row_block=4096):
    """Returns (dq [B,Sq,Hq,D], dk [B,Sk,Hkv,D], dv [B,Sk,Hkv,Dv]) in ``dtype``.

    With ``heads`` given, dk/dv hold only the contributions of those query heads.
    """
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    dout = np.asarray(dout, dtype)
    B, Sq, Hq, _ = q.shape
    _, Sk, Hkv, _ = v.shape
    G = Hq // Hkv
    dq = np.zeros_like(q); dk = np.zeros_like(k); dv = np.zeros_like(v)
    hs = range(Hq) if heads is None else heads
    for b in range(B):
        for r0 in range(0, Sq, row_block):
            sl = slice(r0, min(Sq, r0 + row_block))
            mask = element_mask(np.asarray(q_pos[b])[sl], np.asarray(q_seg[b])[sl],
                                np.asarray(kv_pos[b]), np.asarray(kv_seg[b]))
            for h in hs:
                kh, vh = k[b, :, h // G], v[b, :, h // G]
                s = (q[b, sl, h] @ kh.T) * scale
                p, _ = _softmax_rows(s, mask)
                do = dout[b, sl, h]
                o = p @ vh
                dv[b, :, h // G] += p.T @ do
                dp = do @ vh.T
                delta = (do * o).sum(-1, keepdims=True)
                ds = p * (dp - delta)
                dq[b, sl, h] = (ds @ kh) * scale
                dk[b, :, h // G] += (ds.T @ q[b, sl, h]) * scale
    return dq, dk, dv
