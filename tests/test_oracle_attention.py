"""Pins the dense attention oracle (no GPU): autograd on an independent graph, finite differences,
closed forms."""
import numpy as np
import pytest
import torch

from oracle import attention_oracle as ao


def _inputs(seed, b=2, sq=40, sk=56, hq=4, hkv=2, d=8, pad=5, docs=(17, 20)):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((b, sq, hq, d))
    k = rng.standard_normal((b, sk, hkv, d))
    v = rng.standard_normal((b, sk, hkv, d))
    kv_seg = np.full((b, sk), -1, np.int32)
    kv_pos = np.zeros((b, sk), np.int32)
    at = 0
    for i, n in enumerate(docs):
        kv_seg[:, at:at + n] = i
        kv_pos[:, at:at + n] = np.arange(n)
        at += n
    q_seg, q_pos = kv_seg[:, :sq].copy(), kv_pos[:, :sq].copy()
    if pad:
        q_seg[:, sq - pad:] = -1
    return q, k, v, q_pos, q_seg, kv_pos, kv_seg


def _torch_dense(q, k, v, q_pos, q_seg, kv_pos, kv_seg, scale):
    """Independent statement: einsum + masked_fill + softmax, K/V heads repeated for GQA."""
    q, k, v = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    g = q.shape[2] // k.shape[2]
    kk, vv = k.repeat_interleave(g, dim=2), v.repeat_interleave(g, dim=2)
    s = torch.einsum("bqhd,bkhd->bhqk", q, kk) * scale
    qs, ks = torch.tensor(q_seg), torch.tensor(kv_seg)
    mask = (qs[:, :, None] == ks[:, None, :]) & (torch.tensor(q_pos)[:, :, None] >= torch.tensor(kv_pos)[:, None, :])
    mask &= (qs != -1)[:, :, None] & (ks != -1)[:, None, :]
    s = s.masked_fill(~mask[:, None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)  # rows with nothing to attend
    return (q, k, v), torch.einsum("bhqk,bkhd->bqhd", p, vv)


def test_forward_and_backward_match_torch_autograd():
    args = _inputs(0)
    scale = 0.3
    (q, k, v), out_t = _torch_dense(*args, scale)
    dout = np.random.default_rng(1).standard_normal(out_t.shape)
    out_t.backward(torch.tensor(dout))
    out, lse = ao.attention_forward(*args, scale)
    dq, dk, dv = ao.attention_backward(*args, scale, dout)
    np.testing.assert_allclose(out, out_t.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(dq, q.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(dk, k.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(dv, v.grad.numpy(), atol=1e-12)
    assert (out[:, -5:] == 0).all() and (lse[:, :, -5:] == 0).all()


def test_backward_matches_finite_differences():
    q, k, v, *ids = _inputs(2, b=1, sq=12, sk=12, hq=2, hkv=1, d=4, pad=2, docs=(5, 5))
    scale = 0.5
    dout = np.random.default_rng(3).standard_normal((1, 12, 2, 4))
    dq, dk, dv = ao.attention_backward(q, k, v, *ids, scale, dout)
    loss = lambda q_, k_, v_: (ao.attention_forward(q_, k_, v_, *ids, scale)[0] * dout).sum()
    eps = 1e-6
    rng = np.random.default_rng(4)
    for arr, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for _ in range(10):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            plus, minus = arr.copy(), arr.copy()
            plus[idx] += eps
            minus[idx] -= eps
            a = [q, k, v]
            a[which] = plus
            lp = loss(*a)
            a[which] = minus
            lm = loss(*a)
            assert abs((lp - lm) / (2 * eps) - grad[idx]) < 1e-6


def test_closed_forms():
    rng = np.random.default_rng(5)
    # single key: O = V for every live query
    q = rng.standard_normal((1, 6, 2, 4)); k = rng.standard_normal((1, 1, 2, 4)); v = rng.standard_normal((1, 1, 2, 4))
    zq, zk = np.zeros((1, 6), np.int32), np.zeros((1, 1), np.int32)
    out, _ = ao.attention_forward(q, k, v, zq + 3, zq, zk, zk, 1.0)
    np.testing.assert_allclose(out, np.broadcast_to(v, out.shape), atol=1e-14)
    # Q = 0: uniform weights => running mean of V under a causal mask
    n = 9
    k = rng.standard_normal((1, n, 1, 4)); v = rng.standard_normal((1, n, 1, 4))
    pos = np.arange(n, dtype=np.int32)[None]
    seg = np.zeros((1, n), np.int32)
    out, lse = ao.attention_forward(np.zeros((1, n, 1, 4)), k, v, pos, seg, pos, seg, 0.7)
    want = np.cumsum(v[0, :, 0], axis=0) / np.arange(1, n + 1)[:, None]
    np.testing.assert_allclose(out[0, :, 0], want, atol=1e-14)
    np.testing.assert_allclose(lse[0, 0], np.log(np.arange(1, n + 1)), atol=1e-14)
    # constant positions: bidirectional == plain softmax attention
    q = rng.standard_normal((1, n, 1, 4))
    out, _ = ao.attention_forward(q, k, v, 0 * pos, seg, 0 * pos, seg, 0.5)
    s = q[0, :, 0] @ k[0, :, 0].T * 0.5
    p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
    np.testing.assert_allclose(out[0, :, 0], p @ v[0, :, 0], atol=1e-13)


def test_packed_documents_equal_separate_runs_and_gqa_equals_repeat():
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = _inputs(6, b=1, sq=37, sk=37, pad=0, docs=(17, 20))
    out, _ = ao.attention_forward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, 0.4)
    for a, n in ((0, 17), (17, 20)):
        sl = slice(a, a + n)
        z = np.zeros((1, n), np.int32)
        part, _ = ao.attention_forward(q[:, sl], k[:, sl], v[:, sl], q_pos[:, sl], z, kv_pos[:, sl], z, 0.4)
        np.testing.assert_allclose(out[:, sl], part, atol=1e-13)
    rep, _ = ao.attention_forward(q, np.repeat(k, 2, axis=2), np.repeat(v, 2, axis=2),
                                  q_pos, q_seg, kv_pos, kv_seg, 0.4)
    np.testing.assert_allclose(out, rep, atol=1e-13)


def test_pair_counters_agree():
    from kvax_amd.utils.benchmarking import count_unmasked_pairs, workload
    for name in ("cpu_plumbing",):
        w = workload(name)
        assert count_unmasked_pairs(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg) == \
            ao.count_unmasked_pairs(w.q_pos, w.q_seg, w.kv_pos, w.kv_seg)
    q, k, v, *ids = _inputs(7)
    assert count_unmasked_pairs(*ids) == ao.count_unmasked_pairs(*ids)
