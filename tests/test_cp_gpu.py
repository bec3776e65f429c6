"""Context parallelism on one GPU and the index-based causal mode.

The reference checks its context-parallel path against its tensor-parallel one
(tests/test_attention.py:520-828): queries (and K/V) permuted for load balance, sharded along the
sequence, must give the same result as the unsharded run once un-permuted.  Here the shards run
one after another on the single GPU; the expectations are the same, plus the dense oracle.
"""
import numpy as np
import pytest
import torch

from kvax_amd import (
    FlashAttentionParamsConfig,
    Mesh,
    attention_specs,
    create_attention_mask,
    flash_attention,
    permute_tokens_context_parallelism,
    unpermute_tokens_context_parallelism,
)
from kvax_amd.ops.flash_attention import flash_attention_backward, flash_attention_forward
from kvax_amd.utils.benchmarking import (
    generate_random_segments_lengths,
    make_random_attention_inputs,
    workload,
)
from oracle import attention_oracle as ao
from tests.tolerances import check_close

pytestmark = pytest.mark.gpu
TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))
CP_SPECS = (("data", "context", None, None), ("data", None, None, None))
FWD = FlashAttentionParamsConfig(128, 128)
BWD = FlashAttentionParamsConfig(64, 128)


def _run(specs, mesh, data, scale, dout, sequential, permuted):
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    q, k, v = (x.detach().clone().requires_grad_(True) for x in (q, k, v))
    with attention_specs(*specs), mesh:
        masks = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=FWD, bwd_params=BWD,
                                      calc_bwd_mask=True)
        out = flash_attention(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks, scale=scale,
                              fwd_params=FWD, bwd_params=BWD, assume_sequential_positions=sequential,
                              permute_tokens_for_load_balance=permuted)
    out.backward(dout)
    return out.detach(), q.grad, k.grad, v.grad


@pytest.mark.parametrize("pad, nseg, sequential, permuted", [
    (0, 1, True, False), (1000, 1, False, False), (0, 1, True, True), (1000, 1, True, True),
    (0, 3, False, True), (1000, 12, False, True), (1000, 12, True, True), (0, 3, True, False),
])
def test_context_parallel_equals_unsharded(device, pad, nseg, sequential, permuted):
    cp, S = 4, 4096
    data, scale = make_random_attention_inputs(
        2, S, S, 8, 4, 128, 128, seed=nseg, num_pad_tokens=pad,
        list_of_segment_lengths=generate_random_segments_lengths(S, nseg), device=device)
    dout = torch.randn(data[0].shape, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).to(device)
    ref = _run(TP_SPECS, Mesh({"data": 1, "model": 1}), data, scale, dout, sequential, True)

    mesh = Mesh({"data": 1, "context": cp, "model": 1})
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    if permuted:
        with attention_specs(*CP_SPECS):
            q, k, v, q_pos, q_seg, dout_cp = permute_tokens_context_parallelism(
                (q, k, v, q_pos, q_seg, dout), mesh=mesh)
    else:
        dout_cp = dout
    got = _run(CP_SPECS, mesh, (q, k, v, q_pos, q_seg, kv_pos, kv_seg), scale, dout_cp, sequential, permuted)
    if permuted:
        with attention_specs(*CP_SPECS):
            got = unpermute_tokens_context_parallelism(got, mesh=mesh)
    live_q = (data[4] != -1)[:, :, None, None]
    live_k = (data[6] != -1)[:, :, None, None]
    names = ("out", "dq", "dk", "dv")
    for name, a, b, live in zip(names, got, ref, (live_q, live_q, live_k, live_k)):
        err = ((a.float() - b.float()).abs() * live).max().item()
        # sharding changes the order of the dK/dV sums (fp32 across shards, then one rounding)
        assert err <= (1.6e-2 if name in ("out", "dq") else 3.2e-2), f"{name}: {err}"


def test_sequential_positions_equal_explicit_arange(device):
    data, scale = make_random_attention_inputs(1, 1024, 1024, 4, 2, 64, 64, seed=2, num_pad_tokens=100,
                                               device=device)
    q, k, v, q_pos, q_seg, kv_pos, kv_seg = data
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(q_pos, q_seg, kv_pos, kv_seg, fwd_params=FWD)
        a = flash_attention(q, k, v, q_pos, q_seg, kv_pos, kv_seg, masks, scale=scale, fwd_params=FWD)
        # garbage positions must be ignored in the index-based mode
        b = flash_attention(q, k, v, q_pos * 0 + 5, q_seg, kv_pos * 0 + 9, kv_seg, masks, scale=scale,
                            fwd_params=FWD, assume_sequential_positions=True)
    assert torch.equal(a, b)


@pytest.mark.parametrize("rank, group", [(0, 1), (3, 1), (7, 1), (3, 6)])
def test_cp_shard_workload_against_oracle(device, rank, group):
    """One CP=8 shard of a 131072-token sequence at real shape; oracle on one GQA group (kv head
    `group`: query heads 4 * group ... 4 * group + 3)."""
    w = workload("cp_shard", cp_rank=rank)
    q, k, v, dout = w.draw_tensors(0, device, with_dout=True)
    ids = w.ids(device)
    fp, bp = FlashAttentionParamsConfig(*w.fwd_blocks), FlashAttentionParamsConfig(*w.bwd_blocks)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=fp, bwd_params=bp, calc_bwd_mask=True)
        assert tuple(masks[0].lower_bounds.shape) == (1, 1, 128)
        assert tuple(masks[2].lower_bounds.shape) == (1, 1, 1024)
        out = flash_attention(q, k, v, *ids, masks, scale=w.scale, fwd_params=fp, bwd_params=bp)
    out.backward(dout)
    heads = [4 * group + i for i in range(4)]
    f = lambda t: t.detach().float().cpu().numpy()
    args = (f(q), f(k), f(v), w.q_pos, w.q_seg, w.kv_pos, w.kv_seg, w.scale)
    ref_out, _ = ao.attention_forward(*args, dtype=np.float32, heads=heads, row_block=1024)
    ref_dq, ref_dk, ref_dv = ao.attention_backward(*args, f(dout), dtype=np.float32, heads=heads, row_block=1024)
    # 2e-2 plus the rounding of the 16-bit result (tests/tolerances.py)
    worst = {"out": check_close("out", out[:, :, heads], ref_out[:, :, heads]),
             "dq": check_close("dq", q.grad[:, :, heads], ref_dq[:, :, heads]),
             "dk": check_close("dk", k.grad[:, :, group], ref_dk[:, :, group]),
             "dv": check_close("dv", v.grad[:, :, group], ref_dv[:, :, group])}
    # dK/dV of the sampled kv head straight from the fp32 accumulators: plain 2e-2
    with torch.no_grad():
        out2, lse = flash_attention_forward(q, k, v, *ids, masks[0], w.scale, fp, bp)
        _, dk32, dv32 = flash_attention_backward(q, k, v, *ids, masks[1], masks[2], out2, lse, dout,
                                                 w.scale, fp, bp, dkdv_fp32=True)
    worst["dk fp32"] = check_close("dk fp32", dk32[:, :, group], ref_dk[:, :, group])
    worst["dv fp32"] = check_close("dv fp32", dv32[:, :, group], ref_dv[:, :, group])
    print(f"  cp_shard rank {rank} group {group}: " + ", ".join(f"{n} {e:.3e}" for n, e in worst.items()))


@pytest.mark.parametrize("heads, kv_heads, batch", [(6, 3, 1), (4, 2, 1), (2, 1, 1), (8, 8, 3)])
def test_work_distribution_modes(device, heads, kv_heads, batch):
    """Group counts that exercise every work-item mapping (>= 8 groups, a divisor of 8, neither)."""
    data, scale = make_random_attention_inputs(batch, 1536, 1536, heads, kv_heads, 128, 128, seed=heads,
                                               num_pad_tokens=70, device=device)
    dout = torch.randn(data[0].shape, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(device)
    out, dq, dk, dv = _run(TP_SPECS, Mesh({"data": 1}), data, scale, dout, False, True)
    f = lambda t: t.float().cpu().numpy()
    args = tuple(f(x) if x.dtype == torch.bfloat16 else x.cpu().numpy() for x in data) + (scale,)
    ref_out, _ = ao.attention_forward(*args)
    ref = ao.attention_backward(*args, f(dout))
    check_close("out", out, ref_out)
    for name, got, want in zip(("dq", "dk", "dv"), (dq, dk, dv), ref):
        check_close(name, got, want)
