"""Host-side logic and the C-ABI surface (no GPU): utils mirror the reference's behaviour, the
shared library loads and exports every symbol the header declares, and the ops refuse to run
without a GPU instead of falling back."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest
import torch

import kvax_amd
from kvax_amd import _native
from kvax_amd.utils import (
    PADDING_SEGMENT_ID,
    FlashAttentionParamsConfig,
    Mesh,
    attention_specs,
    permute_tokens_context_parallelism,
    unpermute_tokens_context_parallelism,
)
from kvax_amd.utils.common import get_default_flash_attention_params, pad_to_block_size
from kvax_amd.utils.math import get_multi_head_attention_tflops
from kvax_amd.utils.permutation import generate_shard_indices
from kvax_amd.utils.specs import get_attention_specs

ROOT = Path(__file__).resolve().parent.parent
CP = (("data", "context", None, None), ("data", None, None, None))


def test_header_symbols_are_exported():
    header = (ROOT / "include" / "kvax_amd.h").read_text()
    declared = set(re.findall(r"\b(kvax_[a-z_0-9]+)\s*\(", header))
    declared -= {"kvax_mask_desc", "kvax_fa_args"}
    assert {"kvax_mask_build", "kvax_fa_fwd", "kvax_fa_bwd", "kvax_last_error"} <= declared
    lib = _native.lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert lib.kvax_abi_version() == _native.ABI_VERSION


def test_ctypes_structs_match_the_header_layout():
    # 13 pointers + 12 mask pointers + 24 int64 strides + 14 int32/float fields
    assert ctypes.sizeof(_native.FaArgs) == 13 * 8 + 12 * 8 + 24 * 8 + 14 * 4
    assert ctypes.sizeof(_native.MaskDesc) == 4 * 4 + 4 * 8


def test_argument_validation_without_a_gpu():
    lib = _native.lib()
    assert lib.kvax_fa_fwd(None, None, 0, None) == -1
    assert b"null" in lib.kvax_last_error()
    a = _native.FaArgs()
    a.num_heads, a.num_kv_heads, a.head_dim = 8, 3, 128
    assert lib.kvax_fa_fwd(ctypes.byref(a), None, 0, None) == -1
    a.num_kv_heads, a.head_dim = 4, 48
    assert lib.kvax_fa_fwd(ctypes.byref(a), None, 0, None) == -2
    assert b"head_dim" in lib.kvax_last_error()
    d = (_native.MaskDesc * 1)()
    assert lib.kvax_mask_build(None, None, None, None, 1, 8, 8, 1, 1, d, 1, None, 0, None) == -1


def test_ops_refuse_cpu_tensors():
    ids = [torch.zeros((1, 64), dtype=torch.int32)] * 4
    with attention_specs(("data", None, "model", None), ("data", None, "model", None)):
        with pytest.raises(_native.KvaxNativeError):
            kvax_amd.create_attention_mask(*ids)
        q = torch.zeros((1, 64, 2, 64), dtype=torch.bfloat16)
        with pytest.raises(_native.KvaxNativeError):
            kvax_amd.flash_attention(q, q, q, *ids, mask=(None,))


def test_public_surface():
    for name in ("flash_attention", "create_attention_mask", "attention_specs", "PADDING_SEGMENT_ID",
                 "FlashAttentionParamsConfig", "permute_tokens_context_parallelism",
                 "unpermute_tokens_context_parallelism"):
        assert name in kvax_amd.__all__ and hasattr(kvax_amd, name)
    assert PADDING_SEGMENT_ID == -1
    assert FlashAttentionParamsConfig() == FlashAttentionParamsConfig(64, 64, 4, 3)
    assert get_default_flash_attention_params(backward=True).kv_block_size == 128


def test_specs_validation_and_restore():
    with pytest.raises(ValueError):
        get_attention_specs()
    with pytest.raises(ValueError, match="exactly 4"):
        with attention_specs(("a", None, None), ("a", None, None, None)):
            pass
    with pytest.raises(ValueError, match="Batch"):
        with attention_specs(("a", None, None, None), ("b", None, None, None)):
            pass
    with pytest.raises(ValueError, match="sharded key/value"):
        with attention_specs(("a", "c", None, None), ("a", "c", None, None)):
            pass
    with pytest.raises(ValueError, match="head_dim"):
        with attention_specs(("a", None, None, "x"), ("a", None, None, "x")):
            pass
    with attention_specs(*CP):
        assert get_attention_specs().query_specs[1] == "context"
        with attention_specs(("d", None, "m", None), ("d", None, "m", None)):
            assert get_attention_specs().query_specs[1] is None
        assert get_attention_specs().query_specs[1] == "context"
    with pytest.raises(ValueError):
        get_attention_specs()


def test_permutation_closed_form_and_round_trip():
    assert generate_shard_indices(8) == [0, 7, 1, 6, 2, 5, 3, 4]
    x = torch.arange(2 * 64 * 3).reshape(2, 64, 3)
    ids = torch.arange(64).expand(2, 64)
    with attention_specs(*CP), Mesh({"data": 1, "context": 4, "model": 1}) as mesh:
        px, pids = permute_tokens_context_parallelism((x, ids))
        chunks = pids[0].reshape(8, 8)[:, 0] // 8
        assert chunks.tolist() == [0, 7, 1, 6, 2, 5, 3, 4]
        # shard r of 4 owns original chunks r and 7 - r
        for r in range(4):
            own = pids[0].reshape(4, 16)[r]
            assert set((own // 8).tolist()) == {r, 7 - r}
        back = unpermute_tokens_context_parallelism(px, mesh=mesh)
        assert torch.equal(back, x)
        assert torch.equal(unpermute_tokens_context_parallelism((pids,))[0], ids)
    with attention_specs(*CP):
        with pytest.raises(ValueError):
            permute_tokens_context_parallelism(x)  # no mesh anywhere


def test_pad_to_block_size_and_flops_model():
    pos = torch.arange(10).reshape(1, 10)
    seg = torch.zeros((1, 10), dtype=torch.int64)
    emb = torch.ones((1, 10, 2, 4))
    (e,), p, s = pad_to_block_size((emb,), pos, seg, 8, pos_fill_value=-7)
    assert e.shape == (1, 16, 2, 4) and e[:, 10:].abs().sum() == 0
    assert p[0, 10:].tolist() == [-7] * 6 and s[0, 10:].tolist() == [-1] * 6
    t = get_multi_head_attention_tflops(2, 1024, 1024, 8, 128, 128, causal=True,
                                        forward_pass=True, backward_pass=True)
    assert t == pytest.approx(2 * 8 * 4 * 128 * 1024 * 1024 * 0.5 * 3.5 / 1e12)


def _toy_mask():
    from kvax_amd.utils.typing import AttentionMask

    # 4 query blocks x 4 kv blocks, causal with two documents of two blocks each.
    lower = torch.tensor([[[0, 0, 2, 2]]], dtype=torch.int32)
    upper = torch.tensor([[[1, 2, 3, 4]]], dtype=torch.int32)
    lower_full = torch.tensor([[[0, 0, 2, 2]]], dtype=torch.int32)
    upper_full = torch.tensor([[[0, 1, 2, 3]]], dtype=torch.int32)
    return AttentionMask(lower, upper, lower_full, upper_full)


def test_mask_pictures_and_sparsity():
    from kvax_amd.ops.mask_creator import (
        calculate_mask_sparsity, mask_block_levels, print_mask, render_mask,
    )

    mask = _toy_mask()
    levels = mask_block_levels(mask, 4)
    assert levels.tolist() == [[1, 0, 0, 0], [2, 1, 0, 0], [0, 0, 1, 0], [0, 0, 2, 1]]
    text = render_mask(mask, 4)
    rows = [line[2:-2] for line in text.splitlines() if line.startswith("||")]
    assert rows == ["░░      ", "██░░    ", "    ░░  ", "    ██░░"]
    # Pooled 2x2: no cell is uniformly full, the off-diagonal cells are uniformly skipped.
    pooled = render_mask(mask, 4, max_rows=2, max_columns=2)
    assert [l[2:-2] for l in pooled.splitlines() if l.startswith("||")] == ["░░  ", "  ░░"]
    # Blocks in [lower, upper) over all blocks: 6 of 16.
    assert calculate_mask_sparsity(mask, 64, 64, 256, 256) == pytest.approx(6 / 16)
    print_mask(mask, 4)  # logs; must not raise


def test_mask_picture_of_a_sharded_mask():
    from kvax_amd.ops.mask_creator import mask_block_levels
    from kvax_amd.utils.typing import AttentionMask

    # dK/dV-style mask with 2 query shards: bounds are local to each shard's 2 inner blocks.
    lower = torch.tensor([[[0, 1], [0, 0]]], dtype=torch.int32)
    upper = torch.tensor([[[2, 2], [1, 2]]], dtype=torch.int32)
    zeros = torch.zeros_like(lower)
    levels = mask_block_levels(AttentionMask(lower, upper, zeros, zeros), 4)
    assert levels.tolist() == [[1, 1, 1, 0], [0, 1, 1, 1]]
    with pytest.raises(ValueError):
        mask_block_levels(AttentionMask(lower, upper, zeros, zeros), 3)


def _fa_args(batch, q_len, kv_len, heads, kv_heads, head_dim):
    a = _native.FaArgs()
    a.batch, a.q_len, a.kv_len = batch, q_len, kv_len
    a.num_heads, a.num_kv_heads, a.head_dim = heads, kv_heads, head_dim
    return a


def test_workspace_sizes_follow_the_shapes():
    """The workspace functions are pure functions of the shapes (no GPU needed): 32 bytes per
    64-row tile and batch row for the summaries; the forward adds room for partial results only
    where it runs in its split mode (short query sequences); the backward holds delta, both
    summaries, the order of the dK/dV work items and the counters of their queues."""
    lib = _native.lib()
    fwd = lambda *s: lib.kvax_fa_fwd_workspace_bytes(ctypes.byref(_fa_args(*s)))
    bwd = lambda *s: lib.kvax_fa_bwd_workspace_bytes(ctypes.byref(_fa_args(*s)))
    assert fwd(1, 32768, 32768, 32, 8, 128) == 32 * 512                 # training shape: summaries only
    assert fwd(4, 8192, 8192, 16, 16, 128) == 4 * 32 * 128
    # one query per row: split mode with at most 32 rows per kv head, which walks every tile of its
    # windows and needs no summaries - partial results only
    partial_bytes = fwd(8, 1, 32768, 32, 8, 128)
    assert partial_bytes > 0
    # 40 queries per row (160 rows per kv head): split mode with live-tile lists - summaries as well
    assert fwd(8, 40, 32768, 32, 8, 128) > 8 * 32 * 512
    # 64 work items (8 rows x 8 kv heads) x windows x 4 rows x (128 + 2) floats, 16-byte aligned pieces
    assert partial_bytes % (64 * 4 * 4) == 0
    windows = partial_bytes // (64 * 4 * (128 + 2) * 4)
    assert 2 <= windows <= 64 and windows * 64 * 4 * 130 * 4 == partial_bytes
    assert fwd(8, 1, 64, 32, 8, 128) == 8 * 32                          # too short to divide
    # the wide forward variant adds one list of live tiles (4 header words + one per kv tile) per 256
    # query rows; the request is ignored where the variant does not apply
    wide = _fa_args(1, 32768, 32768, 32, 8, 128)
    wide.flags = _native.KVAX_FA_FWD_WIDE
    assert lib.kvax_fa_fwd_workspace_bytes(ctypes.byref(wide)) == 32 * 512 + 128 * (4 + 512) * 4
    wide = _fa_args(1, 32768, 32768, 32, 8, 64)
    wide.flags = _native.KVAX_FA_FWD_WIDE
    assert lib.kvax_fa_fwd_workspace_bytes(ctypes.byref(wide)) == 32 * 512
    assert fwd(0, 1, 32768, 32, 8, 128) == 0
    delta = 1 * 32 * 32768 * 4
    order = (2 * 256 + 1 + 8) * 4 + 12      # 256 kv work items, an arrival counter, 8 queue counters; padded to 16
    assert bwd(1, 32768, 32768, 32, 8, 128) == delta + 2 * 32 * 512 + order


def test_too_long_key_sequences_are_refused_without_a_gpu():
    """The forward and dQ kernels keep per-tile bitmaps of the key sequence in LDS; a sequence they
    cannot hold is refused before anything is enqueued (so this runs without a GPU: non-null dummy
    pointers are never dereferenced)."""
    lib = _native.lib()
    a = _fa_args(1, 128, 2_000_000, 8, 2, 128)
    dummy = 0x1000
    for field in ("q", "k", "v", "out", "lse", "q_pos", "q_seg", "kv_pos", "kv_seg", "dout", "dq", "dk", "dv"):
        setattr(a, field, dummy)
    for name in ("q_strides", "k_strides", "v_strides", "o_strides", "do_strides", "dq_strides",
                 "dk_strides", "dv_strides"):
        setattr(a, name, (ctypes.c_int64 * 3)(0, 1024, 128))
    a.fwd_query_block = a.fwd_kv_block = a.bwd_query_block = a.bwd_kv_block = 128
    a.dtype, a.scale = _native.KVAX_BF16, 0.1
    for m in (a.fwd_mask, a.dq_mask, a.dkdv_mask):
        for i in range(4):
            m[i] = dummy
    need = lib.kvax_fa_fwd_workspace_bytes(ctypes.byref(a))
    assert lib.kvax_fa_fwd(ctypes.byref(a), dummy, need, None) == -2
    assert b"LDS" in lib.kvax_last_error()
    need = lib.kvax_fa_bwd_workspace_bytes(ctypes.byref(a))
    assert lib.kvax_fa_bwd(ctypes.byref(a), dummy, need, None) == -2
    assert b"LDS" in lib.kvax_last_error()


def test_error_strings_are_per_thread():
    """Two host threads fail in different ways at the same time, many times: each must read back its
    own message (the last-error text is thread-local; no GPU is needed, nothing is launched)."""
    import threading

    lib = _native.lib()
    problems = []

    def worker(head_dim, expect):
        a = _fa_args(1, 128, 128, 8, 2, head_dim)
        for _ in range(2000):
            rc = lib.kvax_fa_fwd(ctypes.byref(a), None, 0, None)
            msg = lib.kvax_last_error()
            if rc >= 0 or expect not in msg:
                problems.append((head_dim, rc, msg))
                return

    # head_dim 100 is refused as unsupported; head_dim 128 with null tensors as a null pointer
    threads = [threading.Thread(target=worker, args=(100, b"head_dim 100")),
               threading.Thread(target=worker, args=(128, b"null tensor pointer"))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not problems, problems[:3]
