"""Edge cases and size-independent properties of the HIP path (no oracle needed at full size).

Properties used: attention is linear in V (forward) and the backward is linear in dO; an
all-padding batch row gives exact zeros; a sequence of one token attends to itself; empty inputs
are accepted and launch nothing.
"""
import numpy as np
import pytest
import torch

from kvax_amd import (
    FlashAttentionParamsConfig,
    attention_specs,
    create_attention_mask,
    flash_attention,
)
from kvax_amd.ops.flash_attention import flash_attention_backward, flash_attention_forward
from kvax_amd.utils.benchmarking import make_random_attention_inputs, workload

pytestmark = pytest.mark.gpu
TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))


def _doc32k(device):
    w = workload("doc32k")
    q, k, v, dout = w.draw_tensors(0, device, with_dout=True)
    ids = w.ids(device)
    fp, bp = FlashAttentionParamsConfig(*w.fwd_blocks), FlashAttentionParamsConfig(*w.bwd_blocks)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=fp, bwd_params=bp, calc_bwd_mask=True)
    return w, (q, k, v, dout), ids, masks, fp, bp


def test_full_size_forward_is_linear_in_v(device):
    """out(V1 + V2) = out(V1) + out(V2) up to the bf16 rounding of the three outputs (32k tokens)."""
    w, (q, k, v, _), ids, masks, fp, bp = _doc32k(device)
    v2 = torch.randn(v.shape, generator=torch.Generator().manual_seed(11)).to(v.dtype).to(device)
    f = lambda vv: flash_attention_forward(q, k, vv, *ids, masks[0], w.scale, fp, bp)[0].float()
    both = f((v.float() + v2.float()).to(v.dtype))
    parts = f(v) + f(v2)
    # V1 + V2 is itself rounded to bf16 before the kernel sees it: compare against that input
    err = (both - parts).abs().max().item()
    assert err <= 4e-2, err
    live = torch.from_numpy(w.q_seg != -1).to(device)
    assert (both[~live] == 0).all() and (parts[~live] == 0).all()


def test_full_size_backward_is_linear_in_dout(device):
    """Gradients for 2 * dO are exactly twice those for dO (power-of-two scaling commutes with every
    rounding in the path), and padding rows stay exactly zero (32k tokens)."""
    w, (q, k, v, dout), ids, masks, fp, bp = _doc32k(device)
    out, lse = flash_attention_forward(q, k, v, *ids, masks[0], w.scale, fp, bp)
    g1 = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, w.scale, fp, bp)
    g2 = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout * 2, w.scale, fp, bp)
    for name, a, b in zip(("dq", "dk", "dv"), g1, g2):
        assert torch.isfinite(a).all(), name
        assert torch.equal(a * 2, b), name
    qpad = torch.from_numpy(w.q_seg == -1).to(device)
    kpad = torch.from_numpy(w.kv_seg == -1).to(device)
    assert (g1[0][qpad] == 0).all() and (g1[1][kpad] == 0).all() and (g1[2][kpad] == 0).all()


def test_backward_is_deterministic(device):
    w, (q, k, v, dout), ids, masks, fp, bp = _doc32k(device)
    out, lse = flash_attention_forward(q, k, v, *ids, masks[0], w.scale, fp, bp)
    a = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, w.scale, fp, bp)
    b = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, w.scale, fp, bp)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def _run(data, scale, blocks=(64, 64)):
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    q, k, v = (x.detach().clone().requires_grad_(True) for x in (q, k, v))
    p = FlashAttentionParamsConfig(*blocks)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=p, bwd_params=p,
                                      calc_bwd_mask=True)
        out = flash_attention(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks, scale=scale, fwd_params=p,
                              bwd_params=p)
    out.backward(torch.ones_like(out))
    return out.detach(), q.grad, k.grad, v.grad


def test_all_padding_row_gives_zeros(device):
    data, scale = make_random_attention_inputs(2, 320, 320, 4, 2, 128, 128, seed=4, device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    q_seg = q_seg.clone(); kv_seg = kv_seg.clone()
    q_seg[1] = -1; kv_seg[1] = -1  # the whole second batch row is padding
    out, dq, dk, dv = _run((q, k, v, q_pos, q_seg, kv_pos, kv_seg), scale)
    for t in (out, dq, dk, dv):
        assert torch.isfinite(t).all()
        assert (t[1] == 0).all()
    assert out[0].abs().max() > 0


def test_single_token_sequence(device):
    """One token: the softmax is 1, so O = V of the head's group, dQ = dK = 0 and dV sums dO over the
    group.  The public wrapper asks for block-divisible lengths in the backward like the reference
    (flash_attention_triton.py:1607-1609); the kernels underneath take ragged lengths."""
    data, scale = make_random_attention_inputs(1, 1, 1, 4, 2, 64, 64, seed=9, device=device)
    q, k, v, *ids = data
    p = FlashAttentionParamsConfig(64, 64)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    out, lse = flash_attention_forward(q, k, v, *ids, masks[0], scale, p, p)
    dout = torch.ones_like(out)
    dq, dk, dv = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out, lse, dout, scale, p, p)
    assert torch.equal(out.view(1, 1, 2, 2, 64), v.view(1, 1, 2, 1, 64).expand(1, 1, 2, 2, 64))
    assert dq.abs().max() == 0 and dk.abs().max() == 0
    assert torch.equal(dv.float(), torch.full_like(dv.float(), 2.0))


@pytest.mark.parametrize("q_len, kv_len", [(0, 64), (64, 0), (0, 0), (0, 4096), (4096, 0)])
def test_empty_sequences(device, q_len, kv_len):
    q = torch.ones(1, q_len, 4, 64, dtype=torch.bfloat16, device=device)
    k = torch.ones(1, kv_len, 2, 64, dtype=torch.bfloat16, device=device)
    ids = [torch.zeros(1, n, dtype=torch.int32, device=device) for n in (q_len, q_len, kv_len, kv_len)]
    out, dq, dk, dv = _run((q, k, k.clone(), *ids), 0.125)
    assert out.shape == q.shape and dq.shape == q.shape and dk.shape == k.shape
    for t in (out, dq, dk, dv):
        assert (t == 0).all()


def test_batch_zero(device):
    q = torch.zeros(0, 64, 4, 64, dtype=torch.bfloat16, device=device)
    k = torch.zeros(0, 64, 2, 64, dtype=torch.bfloat16, device=device)
    ids = [torch.zeros(0, 64, dtype=torch.int32, device=device) for _ in range(4)]
    out, dq, dk, dv = _run((q, k, k.clone(), *ids), 0.125)
    assert out.numel() == 0 and dq.numel() == 0 and dk.numel() == 0 and dv.numel() == 0


def test_query_sequence_longer_than_one_bookkeeping_chunk(device):
    """135168 query rows are 2112 tiles of 64: the dK/dV kernel's live-tile bookkeeping takes 2048 tiles
    per pass, so this runs its chunked path; dK/dV (fp32) against the dense oracle."""
    from oracle import attention_oracle as ao
    sq, sk, d = 135168, 256, 128
    g = torch.Generator().manual_seed(21)
    q = torch.randn(1, sq, 1, d, generator=g).to(torch.bfloat16).to(device)
    k = torch.randn(1, sk, 1, d, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(1, sk, 1, d, generator=g).to(torch.bfloat16).to(device)
    dout = (torch.randn(1, sq, 1, d, generator=g) * 0.05).to(torch.bfloat16).to(device)
    # two documents; queries of each see the keys of their own half; constant positions = bidirectional
    q_seg = (torch.arange(sq) >= sq // 3).to(torch.int32)[None].to(device)
    kv_seg = (torch.arange(sk) >= sk // 2).to(torch.int32)[None].to(device)
    q_pos, kv_pos = torch.zeros_like(q_seg), torch.zeros_like(kv_seg)
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    scale = d ** -0.5
    out, lse = flash_attention_forward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks[0], scale, p, p)
    dq, dk, dv = flash_attention_backward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks[1], masks[2], out, lse,
                                          dout, scale, p, p, dkdv_fp32=True)
    f = lambda t: t.float().cpu().numpy()
    args = (f(q), f(k), f(v), q_pos.cpu().numpy(), q_seg.cpu().numpy(), kv_pos.cpu().numpy(), kv_seg.cpu().numpy(), scale)
    ref_dq, ref_dk, ref_dv = ao.attention_backward(*args, f(dout), dtype=np.float32, row_block=8192)
    for name, got, ref in (("dk", dk, ref_dk), ("dv", dv, ref_dv)):
        err = np.abs(f(got) - ref).max()
        assert err <= 2e-2 * max(1.0, np.abs(ref).max()), f"{name}: {err} (|ref| max {np.abs(ref).max()})"
    assert np.abs(f(dq) - ref_dq).max() <= 2e-2


def test_key_sequence_too_long_for_two_work_groups_per_cu(device):
    """With 262144 keys the tile bitmaps no longer fit beside the LDS ring of the configuration that
    runs two work-groups per compute unit, so forward and dQ take the one-work-group configuration:
    a chunk of 256 late queries over the whole key sequence against the dense oracle."""
    from oracle import attention_oracle as ao
    sq, sk, d = 256, 262144, 128
    g = torch.Generator().manual_seed(23)
    q = torch.randn(1, sq, 2, d, generator=g).to(torch.bfloat16).to(device)
    k = torch.randn(1, sk, 1, d, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(1, sk, 1, d, generator=g).to(torch.bfloat16).to(device)
    dout = torch.randn(1, sq, 2, d, generator=g).to(torch.bfloat16).to(device)
    kv_pos = torch.arange(sk, dtype=torch.int32)[None].to(device)
    q_pos = (torch.arange(sq, dtype=torch.int32) + (sk - sq - 1000))[None].to(device)
    # keys: padding at the front, then two documents; the queries belong to the second one
    kv_seg = torch.ones(1, sk, dtype=torch.int32)
    kv_seg[:, :5000] = -1
    kv_seg[:, 5000:70000] = 0
    kv_seg = kv_seg.to(device)
    q_seg = torch.ones(1, sq, dtype=torch.int32, device=device)
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    scale = d ** -0.5
    out, lse = flash_attention_forward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks[0], scale, p, p)
    dq, dk, dv = flash_attention_backward(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks[1], masks[2], out, lse,
                                          dout, scale, p, p, dkdv_fp32=True)
    f = lambda t: t.float().cpu().numpy()
    args = (f(q), f(k), f(v), q_pos.cpu().numpy(), q_seg.cpu().numpy(), kv_pos.cpu().numpy(), kv_seg.cpu().numpy(), scale)
    ref_out = ao.attention_forward(*args, dtype=np.float32)[0]
    ref_dq, ref_dk, ref_dv = ao.attention_backward(*args, f(dout), dtype=np.float32)
    assert np.abs(f(out) - ref_out).max() <= 2e-2
    for name, got, ref in (("dq", dq, ref_dq), ("dk", dk, ref_dk), ("dv", dv, ref_dv)):
        assert np.abs(f(got) - ref).max() <= 2e-2, name
    assert (f(dk)[0, :70000] == 0).all() and (f(dv)[0, :70000] == 0).all()


def test_hip_graph_replays_match_eager(device):
    """Forward + backward recorded once into a HIP graph and replayed on new inputs: the entry
    points enqueue kernels only (no allocation, no synchronisation, no memset), so every replay
    must equal the eager result on the same inputs - with eager work and synchronisations between
    the replays."""
    data, scale = make_random_attention_inputs(2, 2304, 2304, 8, 2, 128, 128, seed=9, num_pad_tokens=200,
                                               list_of_segment_lengths=[700, 900, -1], device=device)
    q, k, v, *ids = data
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    dout = torch.randn_like(q)

    def eager(q_, k_, v_, do_):
        out, lse = flash_attention_forward(q_, k_, v_, *ids, masks[0], scale, p, p)
        return (out, *flash_attention_backward(q_, k_, v_, *ids, masks[1], masks[2], out, lse, do_, scale, p, p))

    eager(q, k, v, dout)  # first call configures the kernels' LDS limits, which cannot be captured
    sq, sk, sv, sdo = (t.clone() for t in (q, k, v, dout))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        results = eager(sq, sk, sv, sdo)
    for seed in (1, 2, 3):
        g = torch.Generator().manual_seed(seed)
        new = [torch.randn(t.shape, generator=g).to(t.dtype).to(device) for t in (q, k, v, dout)]
        for static, fresh in zip((sq, sk, sv, sdo), new):
            static.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        want = eager(*new)
        torch.cuda.synchronize()
        for name, got, ref in zip(("out", "dq", "dk", "dv"), results, want):
            assert torch.equal(got, ref), f"{name}, replay {seed}"


def test_hip_graph_replays_of_the_split_forward(device):
    """Same for a decoding step (split mode: partial results in the workspace, combine kernel)."""
    data, scale = make_random_attention_inputs(4, 1, 4096, 16, 4, 128, 128, seed=5,
                                               start_query_position=(4000, 100, 2047, 3000), device=device)
    q, k, v, *ids = data
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=p)
    eager = lambda q_, k_, v_: flash_attention_forward(q_, k_, v_, *ids, masks[0], scale, p, p)[0]
    eager(q, k, v)
    sq, sk, sv = (t.clone() for t in (q, k, v))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        result = eager(sq, sk, sv)
    for seed in (1, 2, 3):
        g = torch.Generator().manual_seed(seed)
        new = [torch.randn(t.shape, generator=g).to(t.dtype).to(device) for t in (q, k, v)]
        for static, fresh in zip((sq, sk, sv), new):
            static.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(result, eager(*new)), f"replay {seed}"


def test_strided_views_give_the_same_bits_as_contiguous_tensors(device):
    """Q, K, V taken as views of one fused projection output ([B, S, (Hq + 2 Hkv) * D]) and dO as a
    transposed [B, H, S, D] tensor: the kernels read through strides, so outputs and gradients equal
    those for contiguous copies bit for bit (and no hidden copy is needed)."""
    b, s, hq, hkv, d = 2, 1024, 8, 2, 128
    g = torch.Generator().manual_seed(31)
    fused = torch.randn(b, s, (hq + 2 * hkv) * d, generator=g).to(torch.bfloat16).to(device)
    q = fused[..., :hq * d].view(b, s, hq, d)
    k = fused[..., hq * d:(hq + hkv) * d].view(b, s, hkv, d)
    v = fused[..., (hq + hkv) * d:].view(b, s, hkv, d)
    dout = torch.randn(b, hq, s, d, generator=g).to(torch.bfloat16).to(device).transpose(1, 2)
    assert not q.is_contiguous() and not k.is_contiguous() and not dout.is_contiguous()
    _, _, _, q_pos, q_seg, kv_pos, kv_seg = make_random_attention_inputs(
        b, s, s, hq, hkv, d, d, seed=1, num_pad_tokens=90, list_of_segment_lengths=[300, 500, -1],
        device=device)[0]
    ids = (q_pos, q_seg, kv_pos, kv_seg)
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    scale = d ** -0.5

    def run(q_, k_, v_, do_):
        out, lse = flash_attention_forward(q_, k_, v_, *ids, masks[0], scale, p, p)
        return (out, *flash_attention_backward(q_, k_, v_, *ids, masks[1], masks[2], out, lse, do_, scale, p, p))

    strided = run(q, k, v, dout)
    dense = run(q.contiguous(), k.contiguous(), v.contiguous(), dout.contiguous())
    for name, a, c in zip(("out", "dq", "dk", "dv"), strided, dense):
        assert torch.equal(a, c), name


def test_c_abi_rejects_bad_arguments_before_launching(device):
    """Error paths of kvax_fa_fwd / kvax_fa_bwd with real device pointers: each is reported with its
    code and a message, and nothing is enqueued (the outputs keep their contents)."""
    import ctypes as C

    from kvax_amd import _native
    from kvax_amd.ops.flash_attention import _base_args, _mask_ptrs, _strides3

    lib = _native.lib()
    data, scale = make_random_attention_inputs(1, 256, 256, 4, 2, 128, 128, seed=2, device=device)
    q, k, v, *ids = data
    p = FlashAttentionParamsConfig(128, 128)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=p, bwd_params=p, calc_bwd_mask=True)
    out = torch.full_like(q, 7.0)
    lse = torch.zeros(1, 4, 256, dtype=torch.float32, device=device)

    def args():
        a = _base_args(q, k, v, *ids, scale, p, p)
        a.out, a.lse, a.o_strides = out.data_ptr(), lse.data_ptr(), _strides3(out)
        a.fwd_mask = _mask_ptrs(masks[0])
        return a

    ws = torch.empty(1 << 16, dtype=torch.uint8, device=device)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    fwd = lambda a, w=ws, n=None: lib.kvax_fa_fwd(C.byref(a), w.data_ptr(), w.numel() if n is None else n, stream)

    assert fwd(args()) == 0
    torch.cuda.synchronize()
    good = out.clone()
    out.fill_(7.0)

    a = args()
    assert fwd(a, n=8) == -3 and b"workspace" in lib.kvax_last_error()                  # too small
    assert lib.kvax_fa_fwd(C.byref(a), ws.data_ptr() + 4, ws.numel() - 4, stream) == -1  # misaligned
    a = args(); a.q = q.data_ptr() + 2
    assert fwd(a) == -1 and b"aligned" in lib.kvax_last_error()
    a = args(); a.q_strides = (C.c_int64 * 3)(q.stride(0), q.stride(1) + 4, q.stride(2))
    assert fwd(a) == -1 and b"stride" in lib.kvax_last_error()
    a = args(); a.k_strides = (C.c_int64 * 3)(k.stride(0), 1 << 24, k.stride(2))
    assert fwd(a) == -2 and b"stride" in lib.kvax_last_error()
    a = args(); a.dtype = 5
    assert fwd(a) == -2
    a = args(); a.head_dim = 96
    assert fwd(a) == -2 and b"head_dim" in lib.kvax_last_error()
    a = args(); a.fwd_query_block = 0
    assert fwd(a) == -1
    a = args(); a.flags = 1 << 20
    assert fwd(a) == -1 and b"flags" in lib.kvax_last_error()
    a = args(); a.fwd_mask[2] = None
    assert fwd(a) == -1 and b"mask" in lib.kvax_last_error()
    # backward: gradient pointers and masks
    a = args()
    assert lib.kvax_fa_bwd(C.byref(a), ws.data_ptr(), ws.numel(), stream) == -1
    assert b"gradient" in lib.kvax_last_error()
    assert good.abs().max() > 0


def test_concurrent_host_threads(device):
    """Two host threads call the forward at the same time, each on its own stream with its own
    workspace and outputs (the library keeps no shared mutable state on this path; the kernels' LDS
    limits are set under a once-flag).  Both must reproduce the single-threaded result bit for bit."""
    import threading

    from kvax_amd.ops.flash_attention import flash_attention_forward
    from kvax_amd.utils.benchmarking import make_random_attention_inputs

    params = FlashAttentionParamsConfig(128, 128)
    cases = []
    for i, (sq, hq, hkv, d) in enumerate([(2048, 8, 2, 128), (1536, 4, 4, 64)]):
        data, scale = make_random_attention_inputs(2, sq, sq, hq, hkv, d, d, seed=40 + i, num_pad_tokens=100,
                                                   device=device)
        with attention_specs(*TP_SPECS):
            masks = create_attention_mask(*data[3:], fwd_params=params)
        want = flash_attention_forward(*data, masks[0], scale, params, params)
        cases.append((data, scale, masks, want))
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def worker(i):
        try:
            data, scale, masks, _ = cases[i]
            stream = torch.cuda.Stream(device=device)
            with torch.cuda.stream(stream):
                for _ in range(20):
                    results[i] = flash_attention_forward(*data, masks[0], scale, params, params)
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for (_, _, _, want), got in zip(cases, results):
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
