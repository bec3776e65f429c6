"""``flash_attention``: block-sparse document-mask attention on MI355X.

Host-side mirror of the reference's public op (kvax/ops/flash_attention_triton.py:2027-2178):
same name, arguments, defaults and layouts -- query ``[batch, q_len, heads, head_dim]``, key /
value ``[batch, kv_len, kv_heads, head_dim]``, int32 positions and segment ids, the mask tuple of
``create_attention_mask`` -- and the same errors for unsupported use (bias, missing masks).  It is
differentiable with respect to query, key and value (``torch.autograd.Function`` plays the role
of the reference's ``jax.custom_vjp``, :1882-1944).  The device work is two calls into the C ABI:
``kvax_fa_fwd`` and ``kvax_fa_bwd``.

Context parallelism: when the attention specs name a mesh axis for the query sequence, the query
axis is treated as ``cp`` contiguous shards, exactly what ``shard_map`` hands to each device in
the reference.  This build has one GPU, so the shards are evaluated one after another on it and
dK/dV are summed over shards (the reference's psum of the replicated operands' cotangents).
"""
from __future__ import annotations

import ctypes as C

import torch

from kvax_amd import _native
from kvax_amd.utils.common import (
    FlashAttentionParamsConfig,
    get_default_flash_attention_params,
)
from kvax_amd.utils.permutation import unpermute_tokens_context_parallelism
from kvax_amd.utils.sharding import context_parallel_degree
from kvax_amd.utils.specs import get_attention_specs
from kvax_amd.utils.typing import AttentionMask, DeviceArray

SUPPORTED_HEAD_DIMS = (64, 128, 256)  # what the kernels are built for
# What ``flash_attention`` takes for query/key: the reference's list (flash_attention_triton.py:1397).
# Sizes between the built ones (16, 32, 192) and a different value head_dim are zero-padded.
ACCEPTED_HEAD_DIMS = (16, 32, 64, 128, 192, 256)
_DTYPES = {torch.bfloat16: _native.KVAX_BF16, torch.float16: _native.KVAX_F16}


def _strides3(t: torch.Tensor):
    if t.stride(3) != 1:
        raise ValueError("the head_dim axis must be contiguous")
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def _mask_ptrs(mask) -> "C.c_void_p * 4":
    arrays = mask.flatten() if isinstance(mask, AttentionMask) else tuple(mask)
    out = (C.c_void_p * 4)()
    for i, a in enumerate(arrays):
        if a.dtype != torch.int32 or not a.is_contiguous():
            raise ValueError("mask arrays must be contiguous int32")
        out[i] = a.data_ptr()
    return out


def _ids(x: torch.Tensor, name: str, shape) -> torch.Tensor:
    if tuple(x.shape) != tuple(shape):
        raise ValueError(f"{name} has shape {tuple(x.shape)}, expected {tuple(shape)}")
    return x.to(torch.int32).contiguous()


def _check_inputs(query, key, value):
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise ValueError("query, key and value must be rank-4 [batch, seq, heads, head_dim]")
    if not query.is_cuda:
        raise _native.KvaxNativeError(
            f"query lives on {query.device}: flash_attention only runs on the GPU")
    if query.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {query.dtype}; bf16 and fp16 are supported")
    if key.dtype != query.dtype or value.dtype != query.dtype:
        raise TypeError("query, key and value must share one dtype")
    b, sq, hq, d = query.shape
    bk, sk, hkv, dk_ = key.shape
    if value.shape[:3] != key.shape[:3]:
        raise ValueError(f"key {tuple(key.shape)} and value {tuple(value.shape)} must match "
                         "in batch, length and heads")
    if bk != b or dk_ != d:
        raise ValueError("query and key/value disagree on batch size or head_dim")
    if d not in ACCEPTED_HEAD_DIMS:
        raise ValueError(f"Attention hid_dim can take values {list(ACCEPTED_HEAD_DIMS)}")
    if not 1 <= value.shape[3] <= SUPPORTED_HEAD_DIMS[-1]:
        raise ValueError(f"value head_dim {value.shape[3]} is outside 1..{SUPPORTED_HEAD_DIMS[-1]}")
    if hq % hkv != 0:
        raise ValueError(f"num_heads {hq} must be divisible by num_kv_heads {hkv}")


def _base_args(query, key, value, q_pos, q_seg, kv_pos, kv_seg, scale, fwd_params, bwd_params):
    b, sq, hq, d = query.shape
    sk, hkv = key.shape[1], key.shape[2]
    a = _native.FaArgs()
    a.q, a.k, a.v = query.data_ptr(), key.data_ptr(), value.data_ptr()
    a.q_pos, a.q_seg = q_pos.data_ptr(), q_seg.data_ptr()
    a.kv_pos, a.kv_seg = kv_pos.data_ptr(), kv_seg.data_ptr()
    a.q_strides, a.k_strides, a.v_strides = _strides3(query), _strides3(key), _strides3(value)
    a.batch, a.q_len, a.kv_len = b, sq, sk
    a.num_heads, a.num_kv_heads, a.head_dim = hq, hkv, d
    a.fwd_query_block, a.fwd_kv_block = fwd_params.query_block_size, fwd_params.kv_block_size
    a.bwd_query_block, a.bwd_kv_block = bwd_params.query_block_size, bwd_params.kv_block_size
    a.dtype = _DTYPES[query.dtype]
    a.flags = 0
    a.scale = float(scale)
    return a


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def flash_attention_forward(query, key, value, q_pos, q_seg, kv_pos, kv_seg, fwd_mask, scale,
                            fwd_params, bwd_params, buffers=None, static_scratch=False, flags=0):
    """One device's forward: returns (out like query, lse fp32 [batch, heads, q_len]).
    ``buffers`` = (out, lse) lets a caller reuse its output tensors.  With ``static_scratch`` (and
    ``buffers``) the call goes through ``kvax_fa_fwd_static`` and allocates no device memory: the
    scratch memory is the library's own fixed buffer, shared by all calls on the GPU.  ``flags``:
    ``_native.KVAX_FA_FWD_WIDE`` selects the kernel variant with 64 query rows per wavefront."""
    b, sq, hq, d = query.shape
    if buffers is not None:
        out, lse = buffers
    else:
        out = torch.empty_like(query)
        lse = torch.empty((b, hq, sq), dtype=torch.float32, device=query.device)
    a = _base_args(query, key, value, q_pos, q_seg, kv_pos, kv_seg, scale, fwd_params, bwd_params)
    a.out, a.lse, a.o_strides = out.data_ptr(), lse.data_ptr(), _strides3(out)
    a.fwd_mask = _mask_ptrs(fwd_mask)
    a.flags = flags
    lib = _native.lib()
    if static_scratch:
        with torch.cuda.device(query.device):
            stream = torch.cuda.current_stream().cuda_stream
            rc = lib.kvax_fa_fwd_static(C.byref(a), C.c_void_p(stream))
        _native.check(rc, "kvax_fa_fwd_static")
        return out, lse
    ws = _workspace(lib.kvax_fa_fwd_workspace_bytes(C.byref(a)), query.device)
    with torch.cuda.device(query.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.kvax_fa_fwd(C.byref(a), ws.data_ptr(), ws.numel(), C.c_void_p(stream))
    _native.check(rc, "kvax_fa_fwd")
    return out, lse


def backward_workspace_bytes(query, key) -> int:
    """Size of the scratch buffer ``kvax_fa_bwd`` needs for these shapes (delta + tile summaries)."""
    a = _native.FaArgs()
    a.batch, a.q_len, a.num_heads = query.shape[0], query.shape[1], query.shape[2]
    a.kv_len, a.num_kv_heads, a.head_dim = key.shape[1], key.shape[2], key.shape[3]
    return int(_native.lib().kvax_fa_bwd_workspace_bytes(C.byref(a)))


def flash_attention_backward(query, key, value, q_pos, q_seg, kv_pos, kv_seg, dq_mask, dkdv_mask,
                             out, lse, dout, scale, fwd_params, bwd_params, dkdv_fp32=False,
                             flags=0, buffers=None):
    """One device's backward: returns (dq, dk, dv); dq in the dtype of query, dk / dv too unless
    ``dkdv_fp32`` asks for the kernels' fp32 accumulators (used to sum context shards)."""
    kv_dtype = torch.float32 if dkdv_fp32 else key.dtype
    if buffers is not None:  # (dq, dk, dv, workspace) reused across calls, e.g. by the benchmark
        dq, dk, dv, ws = buffers
    else:
        dq = torch.empty_like(query)
        dk = torch.empty(key.shape, dtype=kv_dtype, device=key.device)
        dv = torch.empty(value.shape, dtype=kv_dtype, device=value.device)
        ws = None
    dout = dout if dout.stride(3) == 1 else dout.contiguous()
    a = _base_args(query, key, value, q_pos, q_seg, kv_pos, kv_seg, scale, fwd_params, bwd_params)
    a.out, a.lse, a.o_strides = out.data_ptr(), lse.data_ptr(), _strides3(out)
    a.dout, a.do_strides = dout.data_ptr(), _strides3(dout)
    a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    a.dq_strides, a.dk_strides, a.dv_strides = _strides3(dq), _strides3(dk), _strides3(dv)
    a.dq_mask, a.dkdv_mask = _mask_ptrs(dq_mask), _mask_ptrs(dkdv_mask)
    a.flags = (_native.KVAX_FA_DKDV_F32 if dkdv_fp32 else 0) | flags
    lib = _native.lib()
    if not hasattr(lib, "kvax_fa_bwd"):
        raise _native.KvaxNativeError("libkvax_amd.so was built without kvax_fa_bwd")
    if ws is None:
        ws = _workspace(lib.kvax_fa_bwd_workspace_bytes(C.byref(a)), query.device)
    with torch.cuda.device(query.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.kvax_fa_bwd(C.byref(a), ws.data_ptr(), ws.numel(), C.c_void_p(stream))
    _native.check(rc, "kvax_fa_bwd")
    return dq, dk, dv


def _slice_mask(mask, shard: int, cp: int, kv_outer: bool):
    """The part of a global mask that ``shard_map`` would hand to one context shard."""
    arrays = mask.flatten() if isinstance(mask, AttentionMask) else tuple(mask)
    if cp == 1:
        return tuple(a.contiguous() for a in arrays)
    if kv_outer:  # [batch, cp, n_kv_blocks] -> [batch, 1, n_kv_blocks]
        return tuple(a[:, shard:shard + 1].contiguous() for a in arrays)
    n = arrays[0].shape[-1] // cp  # [batch, 1, n_q_blocks] split along the last axis
    return tuple(a[..., shard * n:(shard + 1) * n].contiguous() for a in arrays)


class _FlashAttentionFn(torch.autograd.Function):
    """Counterpart of flash_attention_triton_single_device + defvjp (:1882-1944), applied to
    every context shard in turn."""

    @staticmethod
    def forward(ctx, query, key, value, q_pos, q_seg, kv_pos, kv_seg, masks, scale, fwd_params,
                bwd_params, cp):
        b, sq = query.shape[:2]
        sk = key.shape[1]
        q_pos, q_seg = _ids(q_pos, "query_positions", (b, sq)), _ids(q_seg, "query_segment_ids", (b, sq))
        kv_pos, kv_seg = _ids(kv_pos, "kv_positions", (b, sk)), _ids(kv_seg, "kv_segment_ids", (b, sk))
        if sq % cp:
            raise ValueError(f"query length {sq} does not split into {cp} context shards")
        n = sq // cp
        if cp > 1 and n % fwd_params.query_block_size:
            raise ValueError("context shards must hold whole query blocks")
        outs, lses = [], []
        for r in range(cp):
            sl = slice(r * n, (r + 1) * n)
            o, l = flash_attention_forward(
                query[:, sl], key, value, q_pos[:, sl].contiguous(), q_seg[:, sl].contiguous(),
                kv_pos, kv_seg, _slice_mask(masks[0], r, cp, False), scale, fwd_params, bwd_params)
            outs.append(o)
            lses.append(l)
        out = outs[0] if cp == 1 else torch.cat(outs, dim=1)
        lse = lses[0] if cp == 1 else torch.cat(lses, dim=2)
        ctx.save_for_backward(query, key, value, q_pos, q_seg, kv_pos, kv_seg, out, lse)
        ctx.masks, ctx.scale, ctx.cp = masks, scale, cp
        ctx.fwd_params, ctx.bwd_params = fwd_params, bwd_params
        return out

    @staticmethod
    def backward(ctx, dout):
        query, key, value, q_pos, q_seg, kv_pos, kv_seg, out, lse = ctx.saved_tensors
        masks, cp = ctx.masks, ctx.cp
        if len(masks) != 3:
            raise ValueError("Length of mask_tensors should be equal to two")
        bwd = ctx.bwd_params
        if query.shape[1] // cp % bwd.query_block_size or query.shape[1] // cp % bwd.kv_block_size \
                or key.shape[1] % bwd.kv_block_size:
            raise ValueError(
                "backward needs sequence lengths divisible by the backward block sizes")
        n = query.shape[1] // cp
        dqs, dk, dv = [], None, None
        for r in range(cp):
            sl = slice(r * n, (r + 1) * n)
            dq_r, dk_r, dv_r = flash_attention_backward(
                query[:, sl], key, value, q_pos[:, sl].contiguous(), q_seg[:, sl].contiguous(),
                kv_pos, kv_seg, _slice_mask(masks[1], r, cp, False),
                _slice_mask(masks[2], r, cp, True), out[:, sl], lse[:, :, sl].contiguous(),
                dout[:, sl], ctx.scale, ctx.fwd_params, bwd, dkdv_fp32=cp > 1)
            dqs.append(dq_r)
            if dk is None:
                dk, dv = dk_r, dv_r
            else:
                dk += dk_r
                dv += dv_r
        dq = dqs[0] if cp == 1 else torch.cat(dqs, dim=1)
        return (dq, dk.to(key.dtype), dv.to(value.dtype)) + (None,) * 9


def flash_attention(
    query: DeviceArray,
    key: DeviceArray,
    value: DeviceArray,
    query_positions: DeviceArray,
    query_segment_ids: DeviceArray,
    kv_positions: DeviceArray,
    kv_segment_ids: DeviceArray,
    mask: tuple[AttentionMask, ...],
    scale: float = 1.0,
    bias: DeviceArray | None = None,
    fwd_params: FlashAttentionParamsConfig | None = None,
    bwd_params: FlashAttentionParamsConfig | None = None,
    assume_sequential_positions: bool = False,
    memory_optimized_gqa_backward: bool = False,
    permute_tokens_for_load_balance: bool = True,
    debug: bool = False,
    mesh=None,
) -> DeviceArray:
    """Attention over packed documents with a block-sparse mask.

    Arguments and defaults as in the reference (flash_attention_triton.py:2027-2095).

    Precondition on the ids (the reference's too): along every sequence the documents lie one after
    another, i.e. a segment id never comes back once another id has followed it (``0 0 1 1 2`` is
    fine, ``0 1 0`` is not; padding, id -1, may sit anywhere).  The block mask's mask-free range
    ``[lower_full, upper_full)`` is computed from per-block id extremes and is only right for such
    layouts; the kernels trust it, so ids that return to an earlier value give wrong results
    without an error.  Ids need not be sorted or dense (``5 5 2 2 7`` is fine).
    Query/key head dims 16, 32, 64, 128, 192, 256 and any value head dim up to 256 are taken (the
    kernels run at 64, 128 or 256; other sizes are zero-padded here).
    ``memory_optimized_gqa_backward`` is accepted and has no effect: dK/dV are always reduced
    over the query heads of a group inside the kernel, which is what the flag asks for.
    ``debug`` (passed to the Triton launcher in the reference) checks the precondition below on the
    ids and raises ``ValueError`` when it does not hold.  With ``assume_sequential_positions`` the causal test uses
    token indices (plus the shard offset under context parallelism, :1421-1451) instead of the
    position arrays; the indices are materialised here and passed as positions.
    """
    del memory_optimized_gqa_backward
    if bias is not None:
        raise NotImplementedError("Bias is not supported in Flash multi head attention")
    if mask is None or len(mask) == 0:
        raise ValueError("Length of mask_tensors should be at least equal to one")
    if len(mask) not in (1, 3):
        raise ValueError(f"The case with num_mask_tensors={len(mask)} is not supported.")
    get_attention_specs()
    _check_inputs(query, key, value)
    if debug:
        _check_documents_are_contiguous(query_segment_ids, "query_segment_ids")
        _check_documents_are_contiguous(kv_segment_ids, "kv_segment_ids")
    cp = context_parallel_degree(mesh)
    if fwd_params is None:
        fwd_params = get_default_flash_attention_params(backward=False)
    if bwd_params is None:
        bwd_params = get_default_flash_attention_params(backward=True)
    if cp > 1 and permute_tokens_for_load_balance:
        # callers pass K/V permuted like the queries; attention needs them in original order
        key, value = unpermute_tokens_context_parallelism((key, value), mesh=mesh)
    if assume_sequential_positions:
        query_positions, kv_positions = _sequential_positions(
            query, key, cp, permute_tokens_for_load_balance)
    # Head dims the kernels are not built for: zero columns change neither Q K^T nor the real
    # columns of P V, so the tensors are padded to the next built size and the output is cut back
    # (autograd does the same to the gradients).
    d_qk, d_v = query.shape[3], value.shape[3]
    d_run = next(d for d in SUPPORTED_HEAD_DIMS if d >= max(d_qk, d_v))
    if d_qk != d_run:
        query = torch.nn.functional.pad(query, (0, d_run - d_qk))
        key = torch.nn.functional.pad(key, (0, d_run - d_qk))
    if d_v != d_run:
        value = torch.nn.functional.pad(value, (0, d_run - d_v))
    out = _FlashAttentionFn.apply(
        query, key, value, query_positions, query_segment_ids, kv_positions, kv_segment_ids,
        tuple(mask), float(scale), fwd_params, bwd_params, cp)
    return out if d_v == d_run else out[..., :d_v]


def _check_documents_are_contiguous(segment_ids: torch.Tensor, name: str) -> None:
    """Raises ValueError when, along some row, a segment id comes back after another id has followed
    it (padding, id -1, is ignored): the number of runs of equal ids must equal the number of ids."""
    for b in range(segment_ids.shape[0]):
        row = segment_ids[b]
        row = row[row != -1]
        if row.numel() == 0:
            continue
        runs = 1 + int((row[1:] != row[:-1]).sum().item())
        if runs != torch.unique(row).numel():
            raise ValueError(
                f"{name}[{b}]: a segment id comes back after another one has followed it; the block "
                "mask and the attention kernels need every document to be one contiguous run")


def _sequential_positions(query, key, cp: int, permuted: bool):
    """Index-based positions: kv token j has position j; query token i of shard r has the global
    index the reference derives from ``query_global_offset`` (:1421-1451)."""
    b, sq = query.shape[:2]
    sk = key.shape[1]
    dev = query.device
    kv_pos = torch.arange(sk, dtype=torch.int32, device=dev).expand(b, sk).contiguous()
    if cp == 1:
        q_pos = torch.arange(sq, dtype=torch.int32, device=dev)
    else:
        n = sq // cp
        local = torch.arange(n, dtype=torch.int32, device=dev)
        parts = []
        for r in range(cp):
            if permuted:
                half = n // 2
                first = r * half + local[:half]
                second = (2 * cp - r - 1) * half + (local[half:] - half)
                parts.append(torch.cat([first, second]))
            else:
                parts.append(r * n + local)
        q_pos = torch.cat(parts)
    return q_pos.expand(b, sq).contiguous(), kv_pos
