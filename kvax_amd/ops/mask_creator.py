"""``create_attention_mask``: block-sparse attention masks from positions and segment ids.

Host-side mirror of the reference's kvax/ops/mask_creator.py: same function names, arguments,
defaults and return types (``tuple[AttentionMask, ...]`` of length 1 or 3 whose fields are
int32 ``[batch, shards, n_outer_blocks]``).  The device work is one call into the C ABI
(``kvax_mask_build``), which builds all requested masks with two kernel launches.
"""
from __future__ import annotations

import ctypes as C
import logging

import torch

from kvax_amd import _native
from kvax_amd.utils.common import (
    FlashAttentionParamsConfig,
    get_default_flash_attention_params,
)
from kvax_amd.utils.sharding import context_parallel_degree
from kvax_amd.utils.specs import get_attention_specs
from kvax_amd.utils.typing import AttentionMask, DeviceArray

logger = logging.getLogger(__name__)


def _as_ids(x: DeviceArray, name: str) -> torch.Tensor:
    if x.dim() != 2:
        raise ValueError(f"{name} must be [batch, seq_len], got shape {tuple(x.shape)}")
    if not x.is_cuda:
        raise _native.KvaxNativeError(
            f"{name} lives on {x.device}: the mask builder only runs on the GPU"
        )
    if x.dtype is torch.int32 and x.is_contiguous():
        return x
    return x.to(torch.int32).contiguous()


_LAYOUTS: dict = {}

try:  # the stream handle without building a torch.cuda.Stream object around it (4 us of a 27 us call)
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover - older or newer torch without the private helper
    def _raw_stream(index: int) -> int:
        return torch.cuda.current_stream(index).cuda_stream


def _layout(lib, batch, q_len, kv_len, requests, num_q_shards):
    """Where the masks of a call lie in its one allocation (in int32 words after the workspace), and
    the workspace size; a function of the shapes and block sizes, remembered per distinct call."""
    key = (batch, q_len, kv_len, requests, num_q_shards)
    hit = _LAYOUTS.get(key)
    if hit is not None:
        return hit
    descs = (_native.MaskDesc * len(requests))()
    shapes = []
    words = 0
    for d, (qbs, kbs, kv_outer) in zip(descs, requests):
        n_outer = -(-kv_len // kbs) if kv_outer else -(-q_len // qbs)
        shards = num_q_shards if kv_outer else 1
        d.query_block_size, d.kv_block_size, d.kv_outer = qbs, kbs, int(kv_outer)
        shapes.append((words, batch, shards, n_outer))
        words += (4 * batch * shards * n_outer + 3) // 4 * 4  # masks start on 16-byte boundaries
    ws_bytes = lib.kvax_mask_workspace_bytes(batch, q_len, kv_len, descs, len(requests))
    ws_words = (max(ws_bytes, 16) + 15) // 16 * 4
    if len(_LAYOUTS) > 256:
        _LAYOUTS.clear()
    _LAYOUTS[key] = (shapes, words, ws_bytes, ws_words)
    return _LAYOUTS[key]


def build_masks(
    query_positions: DeviceArray,
    query_segment_ids: DeviceArray,
    kv_positions: DeviceArray,
    kv_segment_ids: DeviceArray,
    requests: list[tuple[int, int, bool]],
    skip_pad_tokens: bool = True,
    num_q_shards: int = 1,
) -> list[AttentionMask]:
    """Build one mask per ``(query_block_size, kv_block_size, kv_outer)`` request in one call.

    The host side of a call is kept short (it is most of the call's latency: the two kernels take
    under 10 us): one device allocation holds the workspace and every mask, whose tensors are views
    of it."""
    if not 1 <= len(requests) <= _native.KVAX_MAX_MASKS:
        raise ValueError(f"between 1 and {_native.KVAX_MAX_MASKS} masks per call")
    q_pos = _as_ids(query_positions, "query_positions")
    q_seg = _as_ids(query_segment_ids, "query_segment_ids")
    kv_pos = _as_ids(kv_positions, "kv_positions")
    kv_seg = _as_ids(kv_segment_ids, "kv_segment_ids")
    if q_pos.shape != q_seg.shape or kv_pos.shape != kv_seg.shape:
        raise ValueError("positions and segment ids must have equal shapes")
    if q_pos.shape[0] != kv_pos.shape[0]:
        raise ValueError("query and kv batch sizes differ")
    batch, q_len = q_pos.shape
    kv_len = kv_pos.shape[1]
    device = q_pos.device
    lib = _native.lib()
    descs = (_native.MaskDesc * len(requests))()
    layout = _layout(lib, batch, q_len, kv_len, tuple(requests), num_q_shards)
    shapes, words, ws_bytes, ws_words = layout
    for d, (qbs, kbs, kv_outer) in zip(descs, requests):
        d.query_block_size, d.kv_block_size, d.kv_outer = qbs, kbs, int(kv_outer)
    buf = torch.empty(ws_words + words, dtype=torch.int32, device=device)
    base = buf.data_ptr()
    masks = []
    for d, (off, b, shards, n_outer) in zip(descs, shapes):
        n = b * shards * n_outer
        first = base + 4 * (ws_words + off)
        d.lower, d.upper, d.lower_full, d.upper_full = first, first + 4 * n, first + 8 * n, first + 12 * n
    _, b, shards, n_outer = shapes[0]
    n4 = 4 * b * shards * n_outer
    if n4 % 4 == 0 and all(sh[1:] == shapes[0][1:] for sh in shapes):
        # equal shapes lie back to back: one view of all of them and one unbind
        flat = buf[ws_words:ws_words + len(shapes) * n4].view(len(shapes) * 4, b, shards, n_outer).unbind(0)
        masks = [AttentionMask(*flat[4 * i:4 * i + 4]) for i in range(len(shapes))]
    else:
        for off, b, shards, n_outer in shapes:
            n = b * shards * n_outer
            views = buf[ws_words + off:ws_words + off + 4 * n].view(4, b, shards, n_outer).unbind(0)
            masks.append(AttentionMask(*views))
    index = device.index
    current = torch.cuda.current_device()
    stream = _raw_stream(current if index is None else index)
    if index is None or index == current:
        rc = lib.kvax_mask_build(
            q_pos.data_ptr(), q_seg.data_ptr(), kv_pos.data_ptr(), kv_seg.data_ptr(),
            batch, q_len, kv_len, num_q_shards, int(skip_pad_tokens),
            descs, len(requests), base, ws_bytes, C.c_void_p(stream),
        )
    else:
        with torch.cuda.device(device):
            rc = lib.kvax_mask_build(
                q_pos.data_ptr(), q_seg.data_ptr(), kv_pos.data_ptr(), kv_seg.data_ptr(),
                batch, q_len, kv_len, num_q_shards, int(skip_pad_tokens),
                descs, len(requests), base, ws_bytes, C.c_void_p(stream),
            )
    _native.check(rc, "kvax_mask_build")
    return masks


def compute_attention_mask(
    query_positions: DeviceArray,
    query_segment_ids: DeviceArray,
    kv_positions: DeviceArray,
    kv_segment_ids: DeviceArray,
    kv_block_size: int,
    query_block_size: int,
    skip_pad_tokens: bool = True,
    calculate_dkdv_mask: bool = False,
    mesh=None,
) -> AttentionMask:
    """One mask (kvax/ops/mask_creator.py:338-374)."""
    get_attention_specs()  # same precondition as the reference: specs must be set
    return build_masks(
        query_positions, query_segment_ids, kv_positions, kv_segment_ids,
        [(query_block_size, kv_block_size, calculate_dkdv_mask)],
        skip_pad_tokens=skip_pad_tokens, num_q_shards=context_parallel_degree(mesh),
    )[0]


def create_attention_mask(
    query_positions: DeviceArray,
    query_segment_ids: DeviceArray,
    kv_positions: DeviceArray,
    kv_segment_ids: DeviceArray,
    fwd_params: FlashAttentionParamsConfig | None = None,
    bwd_params: FlashAttentionParamsConfig | None = None,
    calc_bwd_mask: bool = False,
    skip_pad_tokens: bool = True,
    mesh=None,
) -> tuple[AttentionMask, ...]:
    """Forward mask and, with ``calc_bwd_mask``, the dQ and dK/dV masks.

    Same contract as kvax/ops/mask_creator.py:377-490.  The dQ mask uses the backward block
    sizes swapped (query blocks of ``bwd_params.kv_block_size``, :459-460); the dK/dV mask has
    one entry per kv block.  Unlike the reference, ``bwd_params=None`` works (it falls back to
    the default backward parameters instead of dereferencing None, cf. :454-457).
    """
    get_attention_specs()
    if fwd_params is None:
        fwd_params = get_default_flash_attention_params(backward=False)
    requests = [(fwd_params.query_block_size, fwd_params.kv_block_size, False)]
    if calc_bwd_mask:
        if bwd_params is None:
            bwd_params = get_default_flash_attention_params(backward=True)
        requests.append((bwd_params.kv_block_size, bwd_params.query_block_size, False))
        requests.append((bwd_params.query_block_size, bwd_params.kv_block_size, True))
    return tuple(
        build_masks(
            query_positions, query_segment_ids, kv_positions, kv_segment_ids, requests,
            skip_pad_tokens=skip_pad_tokens, num_q_shards=context_parallel_degree(mesh),
        )
    )


def calculate_mask_sparsity(
    mask: AttentionMask, query_block_size: int, kv_block_size: int, query_seq_len: int,
    kv_seq_len: int,
) -> float:
    """Fraction of (query block, kv block) pairs inside [lower, upper)
    (kvax/ops/mask_creator.py:601-625)."""
    visited = (mask.upper_bounds.long() - mask.lower_bounds.long()).sum().item()
    batch = mask.lower_bounds.shape[0]
    return visited / (query_seq_len // query_block_size) / (kv_seq_len // kv_block_size) / batch


def mask_block_levels(mask: AttentionMask, num_inner_blocks: int, batch_index: int = 0) -> torch.Tensor:
    """``[n_outer_blocks, num_inner_blocks]`` int8 grid of one batch entry: 0 = block skipped,
    1 = visited with the element mask, 2 = visited without it.  Shard ``s`` of a context-parallel
    mask covers the inner blocks ``[s * num_inner_blocks / shards, (s + 1) * num_inner_blocks / shards)``
    (kvax/ops/mask_creator.py:507-533)."""
    lower = mask.lower_bounds[batch_index].cpu().long()
    shards, _ = lower.shape
    if num_inner_blocks % shards:
        raise ValueError(f"{num_inner_blocks} inner blocks do not split over {shards} shards")
    col = torch.arange(num_inner_blocks // shards).view(1, 1, -1)

    def inside(lo, hi):
        lo = lo[batch_index].cpu().long().unsqueeze(-1)
        hi = hi[batch_index].cpu().long().unsqueeze(-1)
        return (col >= lo) & (col < hi)

    visited = inside(mask.lower_bounds, mask.upper_bounds)
    full = inside(mask.lower_full_bounds, mask.upper_full_bounds) & visited
    levels = visited.to(torch.int8) + full.to(torch.int8)  # [shards, n_outer, inner/shards]
    return levels.permute(1, 0, 2).reshape(lower.shape[1], num_inner_blocks)


def render_mask(
    mask: AttentionMask, num_inner_blocks: int, print_only_first_in_batch: bool = True,
    fit_in_screen: bool = True, max_rows: int = 32, max_columns: int = 64,
) -> str:
    """Text picture of a block mask: two characters per cell, solid where every block of the
    cell is visited without the element mask, blank where every block is skipped, shaded
    otherwise.  With ``fit_in_screen`` the grid is pooled down to ``max_rows`` x ``max_columns``
    cells (same picture as kvax/ops/mask_creator.py:493-598 draws)."""
    batch = mask.lower_bounds.shape[0]
    text = "Attention masks:\n"
    for b in range(1 if print_only_first_in_batch else batch):
        levels = mask_block_levels(mask, num_inner_blocks, b)
        rows, cols = levels.shape
        row_step = max(-(-rows // max_rows), 1) if fit_in_screen else 1
        col_step = max(-(-cols // max_columns), 1) if fit_in_screen else 1
        # Pool with padding that counts as "skipped", so ragged edge cells read as partial.
        padded = torch.zeros((-(-rows // row_step) * row_step, -(-cols // col_step) * col_step),
                             dtype=torch.int8)
        padded[:rows, :cols] = levels
        cells = padded.view(padded.shape[0] // row_step, row_step, padded.shape[1] // col_step, col_step)
        all_full = (cells == 2).all(dim=3).all(dim=1)
        all_skipped = (cells == 0).all(dim=3).all(dim=1)
        width = all_full.shape[1]
        text += "\n  " + "==" * width + "  \n"
        for full_row, skipped_row in zip(all_full.tolist(), all_skipped.tolist()):
            line = "".join("██" if f else "  " if s else "░░" for f, s in zip(full_row, skipped_row))
            text += "||" + line + "||\n"
        text += "  " + "==" * width + "  \n\n"
    return text


def print_mask(
    mask: AttentionMask, num_inner_blocks: int, print_only_first_in_batch: bool = True,
    fit_in_screen: bool = True,
) -> None:
    """Log the picture of ``render_mask`` at INFO level (kvax/ops/mask_creator.py:493-598)."""
    logger.info(render_mask(mask, num_inner_blocks, print_only_first_in_batch, fit_in_screen))
