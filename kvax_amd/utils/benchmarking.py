"""Seeded synthetic inputs for tests and the benchmark, and the comparison tolerances.

Two families:

* ``make_random_attention_inputs`` / ``generate_random_segments_lengths`` regenerate the input
  family of the reference's tests (kvax/utils/benchmarking.py:36-184 and :309-324): global
  ``arange`` positions, documents laid out contiguously with ids 0..n-1, trailing padding with
  id -1.  Segment lengths come from Python's ``random`` seeded with 0, so they are identical to
  the reference's; the N(0,1) tensors come from a torch CPU generator (jax's PRNG is not
  reproduced -- no reference test depends on the tensor values, only on their distribution).
* ``workload(...)`` builds the five measurement configurations (documents with positions that
  restart per document, lognormal / exponential lengths, the CP shard, the bidirectional case).

``check_outputs_fwd`` / ``check_outputs_bwd`` carry the reference's tolerances
(kvax/utils/benchmarking.py:601-629).
"""
from __future__ import annotations

import math
import random
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch

from kvax_amd.utils.common import PADDING_SEGMENT_ID
from kvax_amd.utils.permutation import generate_shard_indices


def generate_random_segments_lengths(seq_len: int, num_segments: int) -> list[int] | None:
    """``num_segments`` positive lengths summing to ``seq_len``; None for a single segment.

    Each of the ``seq_len - num_segments`` spare tokens goes to a segment drawn by
    ``random.randint`` after ``random.seed(0)`` -- the reference's exact recipe.
    """
    if num_segments == 1:
        return None
    random.seed(0)
    lengths = [1] * num_segments
    for _ in range(seq_len - num_segments):
        lengths[random.randint(0, num_segments - 1)] += 1
    return lengths


def make_random_attention_inputs(
    batch_size: int,
    query_seq_len: int,
    kv_seq_len: int,
    num_query_heads: int,
    num_kv_heads: int,
    qk_head_dim: int,
    value_head_dim: int,
    seed: int = 0,
    num_pad_tokens: int | Sequence[int] = 0,
    start_query_position: int | Sequence[int] = 0,
    list_of_segment_lengths: list[int] | None = None,
    dtype: torch.dtype = torch.bfloat16,
    device: str | torch.device = "cpu",
):
    """(query, key, value, q_pos, q_seg, kv_pos, kv_seg), scale -- BSHD tensors, int32 ids.

    ``num_pad_tokens`` may be per batch row.  As in the reference, when the query length is 1
    (decode) the padding is derived from ``start_query_position``: every kv token after the
    query's position is padding.
    """
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((batch_size, query_seq_len, num_query_heads, qk_head_dim), generator=g)
    k = torch.randn((batch_size, kv_seq_len, num_kv_heads, qk_head_dim), generator=g)
    v = torch.randn((batch_size, kv_seq_len, num_kv_heads, value_head_dim), generator=g)
    scale = 1.0 / math.sqrt(qk_head_dim)

    start = np.broadcast_to(np.asarray(start_query_position, np.int32).reshape(-1, 1), (batch_size, 1))
    q_pos = np.broadcast_to(np.arange(query_seq_len, dtype=np.int32), (batch_size, query_seq_len)) + start
    kv_pos = np.broadcast_to(np.arange(kv_seq_len, dtype=np.int32), (batch_size, kv_seq_len)).copy()
    q_seg = np.zeros((batch_size, query_seq_len), np.int32)
    kv_seg = np.zeros((batch_size, kv_seq_len), np.int32)

    decode = query_seq_len == 1
    if decode:
        pads = kv_seq_len - start[:, 0] - 1
    else:
        pads = np.broadcast_to(np.asarray(num_pad_tokens, np.int32), (batch_size,))

    if list_of_segment_lengths:
        lengths = list(list_of_segment_lengths)
        if lengths[-1] == -1:
            lengths[-1] = query_seq_len - sum(lengths[:-1])
            if lengths[-1] < 0:
                raise ValueError("Sum of all sizes in list_of_segment_lengths exceed seq_len.")
        bounds = np.cumsum([0] + lengths)
        if bounds[-1] > kv_seq_len or bounds[-1] > query_seq_len:
            raise ValueError("Sum of all sizes in list_of_segment_lengths exceed seq_len.")
        for i, (a, b) in enumerate(zip(bounds[:-1], bounds[1:])):
            q_seg[:, a:b] = i
            kv_seg[:, a:b] = i

    for b in range(batch_size):
        n = int(pads[b])
        if n > 0:
            if not decode:
                q_seg[b, query_seq_len - n:] = PADDING_SEGMENT_ID
            kv_seg[b, kv_seq_len - n:] = PADDING_SEGMENT_ID

    def dev(x):
        return torch.from_numpy(np.ascontiguousarray(x)).to(device)

    data = (q.to(dtype).to(device), k.to(dtype).to(device), v.to(dtype).to(device),
            dev(q_pos), dev(q_seg), dev(kv_pos), dev(kv_seg))
    return data, scale


# --------------------------------------------------------------------------------------------
# measurement workloads
# --------------------------------------------------------------------------------------------

@dataclass
class Workload:
    """One measurement configuration: id arrays on the CPU (numpy) plus shape metadata.

    Tensors Q/K/V/dO are drawn separately (``draw_tensors``) so that id-only work such as
    FLOP counting and mask building does not have to materialise gigabytes.
    """

    name: str
    batch: int
    q_len: int
    kv_len: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    causal: bool
    fwd_blocks: tuple[int, int]
    bwd_blocks: tuple[int, int]
    backward: bool
    q_pos: np.ndarray
    q_seg: np.ndarray
    kv_pos: np.ndarray
    kv_seg: np.ndarray
    dtype: torch.dtype = torch.bfloat16
    meta: dict = field(default_factory=dict)

    @property
    def scale(self) -> float:
        return 1.0 / math.sqrt(self.head_dim)

    def draw_tensors(self, seed: int, device="cpu", with_dout: bool | None = None):
        g = torch.Generator().manual_seed(seed)
        shapes = [
            (self.batch, self.q_len, self.num_heads, self.head_dim),
            (self.batch, self.kv_len, self.num_kv_heads, self.head_dim),
            (self.batch, self.kv_len, self.num_kv_heads, self.head_dim),
        ]
        if self.backward if with_dout is None else with_dout:
            shapes.append(shapes[0])
        out = []
        for s in shapes:
            # drawn per batch row to bound the fp32 staging buffer
            rows = [torch.randn(s[1:], generator=g).to(self.dtype) for _ in range(s[0])]
            out.append(torch.stack(rows).to(device))
        return out

    def ids(self, device="cpu"):
        return tuple(torch.from_numpy(np.ascontiguousarray(x)).to(device)
                     for x in (self.q_pos, self.q_seg, self.kv_pos, self.kv_seg))

    def unmasked_pairs(self) -> int:
        """Exact count of attendable (b, q, kv) pairs via per-segment position histograms."""
        return count_unmasked_pairs(self.q_pos, self.q_seg, self.kv_pos, self.kv_seg)


def count_unmasked_pairs(q_pos, q_seg, kv_pos, kv_seg) -> int:
    """#{(b,i,j): q_seg == kv_seg != -1 and q_pos >= kv_pos}, in O(S log S) per row."""
    total = 0
    for b in range(q_pos.shape[0]):
        qs, qp, ks, kp = q_seg[b], q_pos[b], kv_seg[b], kv_pos[b]
        keep_k = ks != PADDING_SEGMENT_ID
        ks, kp = ks[keep_k], kp[keep_k]
        keep_q = qs != PADDING_SEGMENT_ID
        qs, qp = qs[keep_q], qp[keep_q]
        order = np.lexsort((kp, ks))
        ks, kp = ks[order], kp[order]
        # composite keys keep everything in one searchsorted; positions fit in 32 bits
        kkey = ks.astype(np.int64) * (1 << 32) + (kp.astype(np.int64) + (1 << 31))
        lo = np.searchsorted(kkey, qs.astype(np.int64) * (1 << 32), side="left")
        hi = np.searchsorted(kkey, qs.astype(np.int64) * (1 << 32) + (qp.astype(np.int64) + (1 << 31)),
                             side="right")
        total += int((hi - lo).sum())
    return total


def _layout_documents(lengths: Sequence[int], seq_len: int, restart_positions: bool,
                      pad_positions: str = "restart"):
    """ids/positions for documents packed left to right then padding (id -1) to ``seq_len``.

    Padding positions follow a fixed rule because the block-mask builder's per-block min/max
    include padding tokens of mixed blocks: ``"restart"`` numbers the padding tail 0,1,2,...
    like one more document, ``"global"`` keeps the global index, ``"zero"`` writes zeros.
    """
    seg = np.full(seq_len, PADDING_SEGMENT_ID, np.int32)
    pos = np.zeros(seq_len, np.int32)
    at = 0
    for i, n in enumerate(lengths):
        seg[at:at + n] = i
        pos[at:at + n] = np.arange(n) if restart_positions else np.arange(at, at + n)
        at += n
    tail = seq_len - at
    if tail:
        if pad_positions == "restart":
            pos[at:] = np.arange(tail)
        elif pad_positions == "global":
            pos[at:] = np.arange(at, seq_len)
        elif pad_positions == "zero":
            pos[at:] = 0
        else:
            raise ValueError(pad_positions)
    return pos, seg


def _fill_lengths(draw, total: int) -> list[int]:
    """Draw document lengths until ``total`` tokens are covered; the last one is truncated."""
    lengths, used = [], 0
    while used < total:
        n = min(int(draw()), total - used)
        lengths.append(n)
        used += n
    return lengths


def workload(name: str, seed: int = 0, restart_positions: bool = True, cp_rank: int = 3,
             block: int = 128) -> Workload:
    """The measurement configurations, by name:

    ``cpu_plumbing``   B1 S2048 Hq8/Hkv2 D64 fp32, 4 documents + 128 padding tokens, causal, block 64
    ``dense_causal``   B1 S8192 32/8 D128 bf16, one document, forward only, block 128
    ``dense64k``       B1 S65536 4/1 D128 bf16, one document, forward only, block 128: the same FLOPs
                       per head as 64 heads at 16k, in few long rows (the loops of the forward kernel
                       with almost nothing else: used to compare kernel variants)
    ``doc32k``         B1 S32768 32/8 D128 bf16, lognormal documents (median 2048, sigma 1,
                       clipped to [128, 16384]) + ~5 % padding, forward + backward, block 128
    ``cp_shard``       queries = chunks (r, 15-r) of a 131072-token sequence cut in 16, keys =
                       all 131072 tokens; lognormal documents (median 4096), forward + backward
    ``block_skip``     B4 S16384 64/8 D128 bf16, exponential documents (mean 512, min 32), 20-30 %
                       padding per row, bidirectional (constant positions), forward + backward
    ``decode32k``      B8, one query per row against a 32768-slot key cache, 32/8 D128 bf16; row i has
                       16384 + i * 2340 keys filled, the rest of the cache is padding; forward only
    """
    rng = np.random.default_rng(seed)
    if name == "cpu_plumbing":
        S, pad = 2048, 128
        cuts = np.sort(rng.choice(np.arange(1, S - pad), size=3, replace=False))
        lengths = np.diff(np.concatenate([[0], cuts, [S - pad]])).tolist()
        pos, seg = _layout_documents(lengths, S, restart_positions=True)
        return Workload(name, 1, S, S, 8, 2, 64, True, (64, 64), (64, 64), False,
                        pos[None], seg[None], pos[None].copy(), seg[None].copy(),
                        dtype=torch.float32, meta=dict(seed=seed, doc_lengths=lengths, pad=pad))
    if name == "dense_causal":
        S = 8192
        pos, seg = _layout_documents([S], S, restart_positions)
        return Workload(name, 1, S, S, 32, 8, 128, True, (128, 128), (128, 128), False,
                        pos[None], seg[None], pos[None].copy(), seg[None].copy(),
                        meta=dict(seed=seed, doc_lengths=[S], pad=0))
    if name == "dense64k":
        S = 65536
        pos, seg = _layout_documents([S], S, restart_positions)
        return Workload(name, 1, S, S, 4, 1, 128, True, (128, 128), (128, 128), False,
                        pos[None], seg[None], pos[None].copy(), seg[None].copy(),
                        meta=dict(seed=seed, doc_lengths=[S], pad=0))
    if name == "doc32k":
        S = 32768
        real = S - int(round(0.05 * S))
        lengths = _fill_lengths(
            lambda: np.clip(rng.lognormal(math.log(2048.0), 1.0), 128, 16384), real)
        pos, seg = _layout_documents(lengths, S, restart_positions)
        return Workload(name, 1, S, S, 32, 8, 128, True, (block, block), (block, block), True,
                        pos[None], seg[None], pos[None].copy(), seg[None].copy(),
                        meta=dict(seed=seed, sigma=1.0, doc_lengths=lengths, pad=S - real,
                                  restart_positions=restart_positions))
    if name == "cp_shard":
        S, cp = 131072, 8
        lengths = _fill_lengths(
            lambda: np.clip(rng.lognormal(math.log(4096.0), 1.0), 128, 65536), S)
        pos, seg = _layout_documents(lengths, S, restart_positions)
        order = generate_shard_indices(2 * cp)
        chunk = S // (2 * cp)
        mine = order[2 * cp_rank:2 * cp_rank + 2]
        idx = np.concatenate([np.arange(c * chunk, (c + 1) * chunk) for c in mine])
        return Workload(name, 1, 2 * chunk, S, 32, 8, 128, True, (block, block), (block, block),
                        True, pos[idx][None], seg[idx][None], pos[None], seg[None],
                        meta=dict(seed=seed, sigma=1.0, doc_lengths=lengths, cp=cp,
                                  cp_rank=cp_rank, chunks=[int(c) for c in mine],
                                  restart_positions=restart_positions))
    if name == "block_skip":
        B, S = 4, 16384
        pos_rows, seg_rows, metas = [], [], []
        for _ in range(B):
            pad = int(round(rng.uniform(0.20, 0.30) * S))
            lengths = _fill_lengths(lambda: max(32, rng.exponential(512.0)), S - pad)
            _, seg = _layout_documents(lengths, S, restart_positions=False)
            pos_rows.append(np.zeros(S, np.int32))  # constant positions => bidirectional
            seg_rows.append(seg)
            metas.append(dict(pad=pad, num_docs=len(lengths)))
        pos, seg = np.stack(pos_rows), np.stack(seg_rows)
        return Workload(name, B, S, S, 64, 8, 128, False, (block, block), (block, block), True,
                        pos, seg, pos.copy(), seg.copy(), meta=dict(seed=seed, rows=metas))
    if name == "decode32k":
        B, S = 8, 32768
        filled = np.array([16384 + i * 2340 for i in range(B)], np.int32)  # 16384 ... 32764
        kv_pos = np.broadcast_to(np.arange(S, dtype=np.int32), (B, S)).copy()
        kv_seg = np.where(kv_pos < filled[:, None], 0, PADDING_SEGMENT_ID).astype(np.int32)
        q_pos = (filled - 1)[:, None].astype(np.int32)
        q_seg = np.zeros((B, 1), np.int32)
        return Workload(name, B, 1, S, 32, 8, 128, True, (block, block), (block, block), False,
                        q_pos, q_seg, kv_pos, kv_seg, meta=dict(seed=seed, filled=filled.tolist()))
    raise ValueError(f"unknown workload {name!r}")


# --------------------------------------------------------------------------------------------
# tolerances
# --------------------------------------------------------------------------------------------

def check_outputs_fwd(results_ref, results, atol: float = 2e-2, rtol: float = 1e-5) -> None:
    results, results_ref = torch.as_tensor(results).float(), torch.as_tensor(results_ref).float()
    assert torch.isfinite(results).all()
    assert torch.isfinite(results_ref).all()
    assert torch.allclose(results, results_ref, atol=atol, rtol=rtol), \
        f"max abs err {(results - results_ref).abs().max().item():.4g}"


def check_outputs_bwd(results_ref, results, query_atol: float = 3e-2, query_rtol: float = 1e-2,
                      kv_atol: float = 3e-2, kv_rtol: float = 3e-2) -> None:
    names = ("dq", "dk", "dv")
    tols = ((query_atol, query_rtol), (kv_atol, kv_rtol), (kv_atol, kv_rtol))
    for n, got, ref, (atol, rtol) in zip(names, results, results_ref, tols):
        got, ref = torch.as_tensor(got).float(), torch.as_tensor(ref).float()
        assert torch.allclose(got, ref, atol=atol, rtol=rtol), \
            f"{n}: max abs err {(got - ref).abs().max().item():.4g}"
