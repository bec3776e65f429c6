"""Forward parity of the HIP flash-attention kernel (through the C ABI) with the dense CPU oracle.

Tolerance: max abs error <= 2e-2 on O over all rows (padding rows must be exactly zero), the
bound the reference's forward tests use (kvax/utils/benchmarking.py:601-609) and the one the
build's target states.
"""
import numpy as np
import pytest
import torch

from kvax_amd import create_attention_mask, flash_attention
from kvax_amd.utils import FlashAttentionParamsConfig, attention_specs
from kvax_amd.utils.benchmarking import (
    generate_random_segments_lengths,
    make_random_attention_inputs,
    workload,
)
from oracle import attention_oracle as ao

pytestmark = pytest.mark.gpu
TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))
ATOL = 2e-2


def run_forward(data, scale, qbs, kbs, calc_bwd=False, bwd=None):
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    params = FlashAttentionParamsConfig(query_block_size=qbs, kv_block_size=kbs)
    with attention_specs(*TP_SPECS):
        mask = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=params,
                                     bwd_params=bwd, calc_bwd_mask=calc_bwd)
        out = flash_attention(q, k, v, q_pos, q_seg, kv_pos, kv_seg, mask, scale=scale,
                              fwd_params=params, bwd_params=bwd)
    return out


def oracle_forward(data, scale, heads=None):
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = [x.cpu() for x in data]
    out, _ = ao.attention_forward(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                  q_pos.numpy(), q_seg.numpy(), kv_pos.numpy(), kv_seg.numpy(),
                                  scale, dtype=np.float64, heads=heads)
    return out


def check(out, ref, q_seg, heads=None):
    out = out.float().cpu().numpy()
    assert np.isfinite(out).all()
    if heads is not None:
        out, ref = out[:, :, heads], ref[:, :, heads]
    err = np.abs(out - ref).max()
    assert err <= ATOL, f"max abs err {err:.4g}"
    pad = q_seg.cpu().numpy() == -1
    assert (out[pad] == 0).all(), "padding query rows must be exactly zero"


# (q_len, kv_len, heads, kv_heads, head_dim, pad, segments, qbs, kbs): the shape families of the
# reference's forward tests (tests/test_attention.py:304-341) at the head dims built here
CASES = [
    (384, 384, 8, 8, 64, 0, 1, 64, 64),
    (400, 400, 8, 8, 64, 0, 1, 64, 64),
    (384, 256, 8, 8, 64, 0, 1, 64, 64),
    (384, 300, 4, 4, 128, 0, 1, 64, 64),
    (400, 256, 4, 4, 128, 0, 1, 128, 128),
    (400, 300, 4, 4, 128, 0, 1, 128, 64),
    (256, 1, 8, 8, 64, 0, 1, 64, 64),
    (300, 1, 4, 4, 128, 0, 1, 64, 64),
    (384, 384, 8, 8, 128, 100, 1, 64, 64),
    (384, 384, 8, 8, 128, 383, 1, 64, 64),
    (384, 384, 16, 8, 128, 0, 1, 128, 128),
    (384, 384, 16, 1, 64, 100, 1, 64, 128),
    (1024, 1024, 8, 2, 128, 77, 5, 128, 128),
    (1024, 1024, 8, 2, 128, 0, 12, 64, 64),
    (2048, 2048, 4, 4, 64, 300, 7, 128, 128),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16])
def test_forward_matches_dense_oracle(device, case, dtype):
    sq, sk, hq, hkv, d, pad, nseg, qbs, kbs = case
    lengths = generate_random_segments_lengths(min(sq, sk), nseg)
    data, scale = make_random_attention_inputs(2, sq, sk, hq, hkv, d, d, seed=sq + sk + d,
                                               num_pad_tokens=min(pad, sk - 1),
                                               list_of_segment_lengths=lengths, dtype=dtype,
                                               device=device)
    out = run_forward(data, scale, qbs, kbs)
    check(out, oracle_forward(data, scale), data[4])


# The reference's own forward cases run at head_dim 16 (tests/test_attention.py:308-340): taken
# through zero padding to the built sizes, as are value head dims that differ from the qk one.
@pytest.mark.parametrize("sq, sk, hq, hkv, d_qk, d_v, pad", [
    (384, 384, 8, 8, 16, 16, 0), (400, 300, 8, 8, 16, 16, 0), (1, 256, 8, 8, 16, 16, 0),
    (256, 1, 8, 8, 16, 16, 0), (1, 3, 8, 8, 16, 16, 0), (384, 384, 16, 8, 16, 16, 383),
    (384, 384, 16, 1, 16, 16, 100), (384, 384, 8, 4, 32, 32, 50), (384, 384, 8, 4, 32, 96, 50),
    (256, 320, 4, 2, 128, 64, 0), (256, 320, 4, 2, 64, 8, 17),
])
def test_forward_small_and_unequal_head_dims(device, sq, sk, hq, hkv, d_qk, d_v, pad):
    data, scale = make_random_attention_inputs(2, sq, sk, hq, hkv, d_qk, d_v, seed=sq + sk + d_qk + d_v,
                                               num_pad_tokens=min(pad, sk - 1), device=device)
    out = run_forward(data, scale, 64, 64)
    assert out.shape == (2, sq, hq, d_v)
    check(out, oracle_forward(data, scale), data[4])


# head_dim 256 runs natively (one wavefront per SIMD), 192 through zero padding to 256; the list of
# sizes is the reference's (flash_attention_triton.py:1397-1403)
@pytest.mark.parametrize("sq, sk, hq, hkv, d_qk, d_v, pad, nseg, block", [
    (384, 384, 4, 4, 256, 256, 0, 1, 64),
    (400, 300, 4, 2, 256, 256, 0, 1, 128),
    (1024, 1024, 8, 2, 256, 256, 77, 5, 128),
    (2048, 2048, 4, 1, 256, 256, 300, 7, 64),
    (512, 512, 4, 2, 192, 192, 50, 3, 64),
    (384, 384, 4, 4, 192, 128, 0, 1, 64),
    (384, 384, 4, 4, 128, 256, 30, 2, 64),
    (1, 4096, 16, 4, 256, 256, 0, 1, 128),      # decode: split mode at head_dim 256
    (8, 3000, 8, 2, 192, 192, 0, 1, 128),
])
def test_forward_large_head_dims(device, sq, sk, hq, hkv, d_qk, d_v, pad, nseg, block):
    lengths = generate_random_segments_lengths(min(sq, sk), nseg) if sq > 8 else None
    start = sk - sq if sq <= 8 else 0
    data, scale = make_random_attention_inputs(2, sq, sk, hq, hkv, d_qk, d_v, seed=sq + sk + d_qk,
                                               num_pad_tokens=pad, start_query_position=start,
                                               list_of_segment_lengths=lengths, device=device)
    out = run_forward(data, scale, block, block)
    assert out.shape == (2, sq, hq, d_v)
    check(out, oracle_forward(data, scale), data[4])


def test_head_dims_that_are_not_taken(device):
    data, scale = make_random_attention_inputs(1, 128, 128, 2, 2, 512, 512, device=device)
    with pytest.raises(ValueError, match="hid_dim"):
        run_forward(data, scale, 64, 64)
    data, scale = make_random_attention_inputs(1, 128, 128, 2, 2, 24, 24, device=device)
    with pytest.raises(ValueError, match="hid_dim"):
        run_forward(data, scale, 64, 64)
    data, scale = make_random_attention_inputs(1, 128, 128, 2, 2, 64, 320, device=device)
    with pytest.raises(ValueError, match="value head_dim"):
        run_forward(data, scale, 64, 64)


def test_forward_fp16(device):
    data, scale = make_random_attention_inputs(1, 512, 512, 4, 2, 128, 128, seed=3,
                                               num_pad_tokens=50, dtype=torch.float16, device=device)
    out = run_forward(data, scale, 128, 128)
    check(out, oracle_forward(data, scale), data[4])


@pytest.mark.parametrize("kv_len, start", [(384, 300), (512, 500), (500, 300), (4096, (1200, 200, 1000, 3500))])
def test_decode_single_query(device, kv_len, start):
    """q_len = 1 with per-row start positions (tests/test_attention.py:1089-1128)."""
    data, scale = make_random_attention_inputs(4, 1, kv_len, 16, 8, 128, 128, seed=kv_len,
                                               start_query_position=start, device=device)
    out = run_forward(data, scale, 64, 64)
    check(out, oracle_forward(data, scale), data[4])


def test_positions_restart_per_document(device):
    """cpu_plumbing layout (positions restart, padding tail) in bf16 on the GPU."""
    w = workload("cpu_plumbing")
    w.dtype = torch.bfloat16
    q, k, v = w.draw_tensors(0, device, with_dout=False)
    data = (q, k, v) + w.ids(device)
    out = run_forward(data, w.scale, 64, 64)
    check(out, oracle_forward(data, w.scale), data[4])


def test_packed_documents_equal_separate_runs(device):
    """Document masking == block-diagonal concatenation of independent causal attentions."""
    lengths = [200, 56, 312, 200]
    data, scale = make_random_attention_inputs(1, 768, 768, 4, 2, 128, 128, seed=11,
                                               list_of_segment_lengths=lengths, device=device)
    packed = run_forward(data, scale, 64, 64)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    at = 0
    for n in lengths:
        sl = slice(at, at + n)
        part = (q[:, sl].contiguous(), k[:, sl].contiguous(), v[:, sl].contiguous(),
                q_pos[:, sl] - at, torch.zeros_like(q_seg[:, sl]), kv_pos[:, sl] - at,
                torch.zeros_like(kv_seg[:, sl]))
        single = run_forward(part, scale, 64, 64)
        # tiles align differently in the two runs, so sums round differently: allow one bf16
        # ulp of an O(1) value
        assert (packed[:, sl].float() - single.float()).abs().max().item() <= 1.6e-2
        at += n


def test_constant_positions_are_bidirectional(device):
    data, scale = make_random_attention_inputs(1, 256, 256, 2, 2, 64, 64, seed=5, device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    data = (q, k, v, torch.zeros_like(q_pos), q_seg, torch.zeros_like(kv_pos), kv_seg)
    out = run_forward(data, scale, 64, 64).float().cpu()
    s = torch.einsum("bqhd,bkhd->bhqk", q.float().cpu(), k.float().cpu()) * scale
    ref = torch.einsum("bhqk,bkhd->bqhd", s.softmax(-1), v.float().cpu())
    assert (out - ref).abs().max().item() <= ATOL


_HEADS_ORACLE = {}


def _sampled_heads_oracle(name, heads, row=0):
    """Oracle output of a few heads of one batch row of a full-size workload, computed once per
    process: it does not depend on the mask block size."""
    key = (name, tuple(heads), row)
    if key not in _HEADS_ORACLE:
        w = workload(name)
        q, k, v = w.draw_tensors(0, "cpu", with_dout=False)
        r = slice(row, row + 1)
        ref, _ = ao.attention_forward(q[r].float().numpy(), k[r].float().numpy(), v[r].float().numpy(),
                                      w.q_pos[r], w.q_seg[r], w.kv_pos[r], w.kv_seg[r],
                                      w.scale, dtype=np.float32, heads=heads, row_block=2048)
        _HEADS_ORACLE[key] = ref
    return _HEADS_ORACLE[key]


# heads from different kv groups; for the four-row block_skip workload also the last batch row (its
# byte offsets are the largest of all configurations)
@pytest.mark.parametrize("name, block, heads, row", [
    ("dense_causal", 128, [0, 13], 0), ("doc32k", 128, [5, 26], 0),
    ("block_skip", 128, [0, 63], 0), ("block_skip", 64, [0, 63], 0),
    ("block_skip", 128, [0, 63], 3), ("block_skip", 64, [0, 63], 3)])
def test_measurement_workloads_sampled_heads(device, name, block, heads, row):
    """Full-size configurations at every mask block size they are specified for; the dense oracle is
    evaluated for a sample of heads of one batch row."""
    w = workload(name, block=block)
    q, k, v = w.draw_tensors(0, device, with_dout=False)
    data = (q, k, v) + w.ids(device)
    assert w.fwd_blocks == (block, block)
    out = run_forward(data, w.scale, *w.fwd_blocks)
    r = slice(row, row + 1)
    err = np.abs(out[r].float().cpu().numpy()[:, :, heads] - _sampled_heads_oracle(name, heads, row)[:, :, heads]).max()
    print(f"{name} block {block} row {row} heads {heads}: max abs err {err:.3e}")
    check(out[r], _sampled_heads_oracle(name, heads, row), data[4][r], heads=heads)


def test_unsorted_document_ids(device):
    """Documents laid out one after another whose ids are neither sorted nor dense (9, 2, 5 ...):
    allowed; only an id that comes back after another one is outside the contract."""
    data, scale = make_random_attention_inputs(2, 1024, 1024, 4, 2, 128, 128, seed=17, num_pad_tokens=120,
                                               list_of_segment_lengths=[200, 130, 300, 64, -1],
                                               device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    relabel = torch.tensor([9, 2, 5, 1000000, 3], dtype=torch.int32, device=device)
    q_seg = torch.where(q_seg == -1, q_seg, relabel[q_seg.clamp(min=0).long()])
    kv_seg = torch.where(kv_seg == -1, kv_seg, relabel[kv_seg.clamp(min=0).long()])
    data = (q, k, v, q_pos, q_seg, kv_pos, kv_seg)
    for block in (64, 128):
        out = run_forward(data, scale, block, block)
        check(out, oracle_forward(data, scale), q_seg)


def test_debug_flag_checks_the_document_layout(device):
    """``debug=True`` verifies that no segment id returns after another one has followed it."""
    data, scale = make_random_attention_inputs(1, 256, 256, 2, 2, 64, 64, num_pad_tokens=20,
                                               list_of_segment_lengths=[100, 60, -1], device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    with attention_specs(*TP_SPECS):
        mask = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg)
        flash_attention(q, k, v, q_pos, q_seg, kv_pos, kv_seg, mask, scale=scale, debug=True)  # fine
        bad = kv_seg.clone()
        bad[:, 200:210] = 0  # document 0 comes back inside document 2
        with pytest.raises(ValueError, match="comes back"):
            flash_attention(q, k, v, q_pos, q_seg, kv_pos, bad, mask, scale=scale, debug=True)
        ok = kv_seg.clone()
        ok[:, 120:125] = -1  # padding in the middle of a document does not split it
        flash_attention(q, k, v, q_pos, q_seg, kv_pos, ok, mask, scale=scale, debug=True)


def test_errors(device):
    data, scale = make_random_attention_inputs(1, 128, 128, 2, 2, 64, 64, device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    with attention_specs(*TP_SPECS):
        mask = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg)
        with pytest.raises(NotImplementedError):
            flash_attention(*data, mask, bias=torch.zeros(1, device=device))
        with pytest.raises(ValueError):
            flash_attention(*data, ())
        with pytest.raises(ValueError):
            flash_attention(q[..., :48], k[..., :48], v[..., :48], q_pos, q_seg, kv_pos, kv_seg, mask)


# Short query sequences run in the split mode: rows are (query, head) pairs of a GQA group and the
# key sequence is divided over several work-groups whose partial results are merged.
@pytest.mark.parametrize("sq, sk, hq, hkv, d, batch, pad, nseg", [
    (1, 8192, 16, 4, 128, 2, 0, 1),       # decode, one row group per kv head
    (1, 16384, 32, 8, 128, 4, 0, 1),      # decode at the benchmark's head layout
    (1, 5000, 8, 8, 64, 3, 0, 1),         # decode, ragged key length, head_dim 64
    (8, 4096, 32, 8, 128, 1, 0, 1),       # a few new tokens (32 rows per kv head)
    (48, 2048, 16, 4, 128, 2, 0, 1),      # 192 rows per kv head: two row tiles
    (200, 3000, 6, 2, 64, 1, 37, 3),      # ragged prefill chunk with documents and padding
    (128, 1024, 4, 1, 128, 1, 100, 2),    # multi-query attention
    (1, 4096, 16, 4, 256, 2, 0, 1),       # decode at head_dim 256
    (3, 2500, 8, 1, 256, 1, 0, 2),        # 24 rows per kv head, documents, head_dim 256
    (2, 3000, 32, 2, 64, 2, 5, 2),        # exactly 32 rows per kv head, padding, head_dim 64
    (9, 3000, 8, 2, 128, 2, 0, 1),        # 36 rows per kv head: just beyond the 32-row case
    (1, 300, 16, 16, 128, 40, 0, 1),      # 640 (batch, kv head) items: more than one resident set, no windows
    (1, 700, 32, 16, 256, 20, 0, 1),      # head_dim 256: 320 items against 256 resident work-groups
    (2, 9000, 8, 8, 64, 9, 3, 2),         # 72 items: 7 windows each
])
def test_split_mode_matches_dense_oracle(device, sq, sk, hq, hkv, d, batch, pad, nseg):
    lengths = generate_random_segments_lengths(sk, nseg)
    start = sk - sq - pad
    data, scale = make_random_attention_inputs(batch, sq, sk, hq, hkv, d, d, seed=sq + sk,
                                               num_pad_tokens=pad, start_query_position=start,
                                               device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    if lengths is not None:  # documents over the keys; each query takes the document of its position
        bounds = np.cumsum([0] + lengths)
        seg_of = np.searchsorted(bounds, np.arange(sk), side="right") - 1
        kv_seg = torch.where(kv_seg == -1, kv_seg, torch.from_numpy(seg_of).to(torch.int32).to(device)[None])
        q_seg = torch.where(q_seg == -1, q_seg,
                            torch.from_numpy(seg_of).to(torch.int32).to(device)[q_pos.clamp(max=sk - 1).long()])
        data = (q, k, v, q_pos, q_seg, kv_pos, kv_seg)
    out = run_forward(data, scale, 128, 128)
    check(out, oracle_forward(data, scale), data[4])


@pytest.mark.parametrize("sq, hq, hkv, d", [(1, 16, 4, 128), (24, 8, 2, 64)])
def test_split_mode_fp16(device, sq, hq, hkv, d):
    """fp16 through the split mode: one query per row (the narrow decoding path, 4 rows per kv head)
    and a chunk of 24 new tokens (96 rows per kv head: windows with live-tile lists), with documents
    over the key cache."""
    sk = 6000
    data, scale = make_random_attention_inputs(2, sq, sk, hq, hkv, d, d, seed=sq + d, num_pad_tokens=0,
                                               start_query_position=sk - sq, dtype=torch.float16,
                                               device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    assert q.dtype == torch.float16
    bounds = np.cumsum([0, 1500, 2500, 2000])
    seg_of = torch.from_numpy(np.searchsorted(bounds, np.arange(sk), side="right") - 1).to(torch.int32).to(device)
    kv_seg = seg_of[None].expand_as(kv_seg).contiguous()
    q_seg = seg_of[q_pos.clamp(max=sk - 1).long()]
    data = (q, k, v, q_pos, q_seg, kv_pos, kv_seg)
    out = run_forward(data, scale, 128, 128)
    assert out.dtype == torch.float16
    check(out, oracle_forward(data, scale), q_seg)


def test_decode_workload_all_rows(device):
    """The decode measurement workload (one query per row, key caches filled to different lengths)
    against the oracle, every batch row and head."""
    w = workload("decode32k")
    q, k, v = w.draw_tensors(0, device, with_dout=False)
    data = (q, k, v, *w.ids(device))
    out = run_forward(data, w.scale, *w.fwd_blocks)
    check(out, oracle_forward(data, w.scale), data[4])


def _short_query_case(seed):
    """Seeded random decoding / chunked-prefill inputs: the queries are the last tokens of a key
    cache filled to a random length (the rest is padding), documents with monotone ids over the
    cache, positions global or restarting per document, some trailing query padding."""
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.choice([64, 128]))
    hkv = int(rng.choice([1, 2, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 8, 16]))
    batch = int(rng.integers(1, 5))
    sq = int(rng.choice([1, 1, 2, 5, 8, 17, 64, 100, 200]))
    sk = int(rng.integers(max(sq, 65), 7000))
    block = int(rng.choice([64, 128]))
    restart = bool(rng.random() < 0.5)
    kv_seg = np.zeros((batch, sk), np.int32); kv_pos = np.zeros((batch, sk), np.int32)
    q_seg = np.zeros((batch, sq), np.int32); q_pos = np.zeros((batch, sq), np.int32)
    for b in range(batch):
        filled = int(rng.integers(sq, sk + 1))
        ndoc = int(rng.integers(1, 6))
        cuts = (np.sort(rng.choice(np.arange(1, filled), size=min(ndoc - 1, filled - 1), replace=False))
                if ndoc > 1 and filled > 1 else np.array([], int))
        seg = np.searchsorted(cuts, np.arange(filled), side="right").astype(np.int32)
        pos = np.arange(filled, dtype=np.int32)
        if restart:
            pos = pos - np.r_[0, cuts][seg].astype(np.int32)
        kv_seg[b, :filled], kv_seg[b, filled:] = seg, -1
        kv_pos[b, :filled], kv_pos[b, filled:] = pos, np.arange(sk - filled)
        q_seg[b], q_pos[b] = seg[filled - sq:], pos[filled - sq:]
        if rng.random() < 0.3 and sq > 2:
            q_seg[b, sq - int(rng.integers(1, sq)):] = -1
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, sq, hq, d, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, sk, hkv, d, generator=g).to(torch.bfloat16)
    v = torch.randn(batch, sk, hkv, d, generator=g).to(torch.bfloat16)
    ids = tuple(torch.from_numpy(x) for x in (q_pos, q_seg, kv_pos, kv_seg))
    return (q, k, v, *ids), d ** -0.5, block


@pytest.mark.parametrize("seed", range(12))
def test_randomized_short_query_shapes(device, seed):
    data, scale, block = _short_query_case(seed)
    out = run_forward(tuple(x.to(device) for x in data), scale, block, block)
    check(out, oracle_forward(data, scale), data[4])


@pytest.mark.parametrize("sq, qbs", [(1, 1), (64, 32)])
def test_split_mode_padding_queries_with_masks_that_keep_padding(device, sq, qbs):
    """Split mode with masks built with ``skip_pad_tokens=False``, which declare blocks of padding
    queries against padding keys mask-free: work-groups whose rows are all padding (an inactive slot
    of a decoding batch: the narrow path; the padded half of a chunk of 64 new tokens: windows with
    live-tile lists) accumulate over those blocks without the element mask and must still write
    exact zeros."""
    sk, hq, hkv, batch = 4096, 8, 2, 3
    g = torch.Generator().manual_seed(sq)
    q = torch.randn((batch, sq, hq, 128), generator=g).to(torch.bfloat16).to(device)
    k = torch.randn((batch, sk, hkv, 128), generator=g).to(torch.bfloat16).to(device)
    v = torch.randn((batch, sk, hkv, 128), generator=g).to(torch.bfloat16).to(device)
    filled = sk - 1500  # key cache: `filled` tokens, then padding
    kv_pos = torch.arange(sk, dtype=torch.int32)[None].repeat(batch, 1)
    kv_seg = torch.zeros((batch, sk), dtype=torch.int32)
    kv_seg[:, filled:] = -1
    q_pos = kv_pos[:, filled - sq:filled].clone()
    q_seg = torch.zeros((batch, sq), dtype=torch.int32)
    if sq == 1:  # batch row 1 is an inactive slot
        q_seg[1, :], q_pos[1, :] = -1, sk + 10
    else:        # the second half of every chunk is padding
        q_seg[:, sq // 2:], q_pos[:, sq // 2:] = -1, sk + 10
    ids = tuple(x.to(device) for x in (q_pos, q_seg, kv_pos, kv_seg))
    params = FlashAttentionParamsConfig(qbs, 128)
    with attention_specs(*TP_SPECS):
        mask = create_attention_mask(*ids, fwd_params=params, skip_pad_tokens=False)
        out = flash_attention(q, k, v, *ids, mask, scale=128 ** -0.5, fwd_params=params)
    # the case is the intended one: some query block sees the padding keys as a mask-free range
    m = mask[0]
    assert ((m.upper_full_bounds - m.lower_full_bounds) * 128 >= 1024).any()
    data = (q, k, v) + ids
    check(out, oracle_forward(data, 128 ** -0.5), ids[1])


def _forward_with_flags(data, scale, block, flags):
    from kvax_amd import _native
    from kvax_amd.ops.flash_attention import flash_attention_forward
    q, k, v, *ids = data
    params = FlashAttentionParamsConfig(block, block)
    with attention_specs(*TP_SPECS):
        mask = create_attention_mask(*ids, fwd_params=params)
    out, lse = flash_attention_forward(q, k, v, *ids, mask[0], scale, params, params,
                                       flags=_native.KVAX_FA_FWD_WIDE if flags else 0)
    return out, lse


@pytest.mark.parametrize("sq, sk, hq, hkv, pad, nseg, block", [
    (2048, 2048, 8, 2, 77, 5, 128),     # documents and padding
    (2000, 1900, 8, 8, 0, 1, 64),       # ragged lengths, one document
    (4096, 4096, 4, 1, 600, 12, 128),   # many documents, multi-query
])
def test_wide_forward_kernel(device, sq, sk, hq, hkv, pad, nseg, block):
    """KVAX_FA_FWD_WIDE (64 query rows per wavefront, one wavefront per SIMD) against the oracle and
    against the default kernel (same values up to the rounding of a different summation order)."""
    lengths = generate_random_segments_lengths(min(sq, sk), nseg)
    data, scale = make_random_attention_inputs(2, sq, sk, hq, hkv, 128, 128, seed=sq + nseg,
                                               num_pad_tokens=pad, list_of_segment_lengths=lengths,
                                               device=device)
    wide, lse_w = _forward_with_flags(data, scale, block, True)
    plain, lse_p = _forward_with_flags(data, scale, block, False)
    check(wide, oracle_forward(data, scale), data[4])
    assert (wide.float() - plain.float()).abs().max().item() <= 1.6e-2
    assert (lse_w - lse_p).abs().max().item() <= 1e-3


def test_wide_forward_kernel_restarting_positions(device):
    """The wide kernel on the 32k document workload (positions restart per document, padding tail):
    two heads against the dense oracle."""
    w = workload("doc32k")
    q, k, v = w.draw_tensors(0, device, with_dout=False)
    data = (q, k, v) + w.ids(device)
    out, _ = _forward_with_flags(data, w.scale, 128, True)
    check(out[:1], _sampled_heads_oracle("doc32k", [5, 26]), data[4][:1], heads=[5, 26])
