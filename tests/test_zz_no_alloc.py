"""``kvax_fa_fwd_static``: the forward entry point that takes no workspace and allocates nothing.

It runs the kernels of ``kvax_fa_fwd`` on the library's own fixed scratch buffer, so its results must
be bit-identical to ``kvax_fa_fwd``'s.  Checked on two calls in a row, the second on a smaller input
(the buffer then still holds what the first call left), for the regular path (scratch = tile
summaries) and the split path used for decoding (scratch = tile summaries + partial results), and
the size limit is checked to fail cleanly.
"""
import ctypes as C

import pytest
import torch

from kvax_amd import _native, create_attention_mask
from kvax_amd.ops.flash_attention import _base_args, _mask_ptrs, _strides3, flash_attention_forward
from kvax_amd.utils import FlashAttentionParamsConfig, attention_specs
from kvax_amd.utils.benchmarking import make_random_attention_inputs

pytestmark = pytest.mark.gpu
TP_SPECS = (("data", None, "model", None), ("data", None, "model", None))
PARAMS = FlashAttentionParamsConfig(128, 128)


def _both_ways(data, scale):
    q, k, v, *ids = data
    with attention_specs(*TP_SPECS):
        masks = create_attention_mask(*ids, fwd_params=PARAMS)
    want_out, want_lse = flash_attention_forward(q, k, v, *ids, masks[0], scale, PARAMS, PARAMS)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((q.shape[0], q.shape[2], q.shape[1]), float("nan"), dtype=torch.float32, device=q.device)
    # The first call of a kernel variant on a device makes the runtime load its code object and look
    # up the scratch symbol; that warm-up call is what a caller does before capturing a graph.
    flash_attention_forward(q, k, v, *ids, masks[0], scale, PARAMS, PARAMS, buffers=(out, lse),
                            static_scratch=True)
    out.fill_(float("nan")), lse.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # device-wide: sees allocations torch's allocator does not
    flash_attention_forward(q, k, v, *ids, masks[0], scale, PARAMS, PARAMS, buffers=(out, lse),
                            static_scratch=True)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before, "the static-scratch call must not allocate"
    assert torch.cuda.mem_get_info()[0] == free_before, "the static-scratch call changed the free device memory"
    assert torch.equal(out, want_out), (out.float() - want_out.float()).abs().max().item()
    assert torch.equal(lse, want_lse)


# (batch, q_len, kv_len, heads, kv_heads, head_dim, padding): a larger call, then a smaller one
REGULAR = [(2, 2048, 2048, 8, 2, 128, 300), (1, 640, 640, 4, 4, 64, 50)]
SPLIT = [(4, 1, 16384, 32, 8, 128, 0), (2, 1, 3000, 8, 2, 128, 0)]


@pytest.mark.parametrize("cases", [REGULAR, SPLIT, REGULAR + SPLIT], ids=["regular", "split", "mixed"])
def test_static_scratch_equals_workspace_entry_point(device, cases):
    for i, (b, sq, sk, hq, hkv, d, pad) in enumerate(cases):
        start = sk - sq if sq == 1 else 0
        data, scale = make_random_attention_inputs(b, sq, sk, hq, hkv, d, d, seed=10 + i, num_pad_tokens=pad,
                                                   start_query_position=start, device=device)
        _both_ways(data, scale)


def test_static_scratch_rejects_oversized_requests(device):
    """A call whose scratch need exceeds the static buffer fails with KVAX_EWORKSPACE before
    anything is enqueued; the tensors are never touched, so the pointers may be fake."""
    lib = _native.lib()
    q = torch.empty((1, 1, 8, 128), dtype=torch.bfloat16, device=device)
    a = _native.FaArgs()
    # 64 rows decoding against 512k keys: the tile summaries alone exceed 8 MiB
    a.batch, a.q_len, a.kv_len, a.num_heads, a.num_kv_heads, a.head_dim = 64, 1, 1 << 19, 64, 8, 128
    need = lib.kvax_fa_fwd_workspace_bytes(C.byref(a))
    assert need > _native.KVAX_FA_FWD_STATIC_MAX_WORKSPACE
    for name in ("q", "k", "v", "out", "lse", "q_pos", "q_seg", "kv_pos", "kv_seg"):
        setattr(a, name, q.data_ptr())
    for s in ("q_strides", "k_strides", "v_strides", "o_strides"):
        setattr(a, s, (C.c_int64 * 3)(1024, 1024, 128))
    a.fwd_query_block = a.fwd_kv_block = 128
    a.dtype, a.scale = _native.KVAX_BF16, 1.0
    rc = lib.kvax_fa_fwd_static(C.byref(a), None)
    assert rc == -3, rc  # KVAX_EWORKSPACE
    assert b"static" in lib.kvax_last_error()
