"""Constants and launch-parameter config for the attention hot path.

Mirrors the public names of the reference's ``kvax/utils/common.py`` (PADDING_SEGMENT_ID at
common.py:9, FlashAttentionParamsConfig at common.py:13-18, get_default_flash_attention_params at
common.py:21-41, pad_to_block_size at common.py:44-74).  The defaults are keyed for MI355X rather
than H100: the block sizes are the *mask granularity* the caller sees; the HIP kernels pick their
own register/LDS tiling underneath.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import torch

PADDING_SEGMENT_ID = -1
MI355X_NAME = "MI355X"
INT32_MAX = 2**31 - 1


@dataclass(frozen=True)
class FlashAttentionParamsConfig:
    """Block sizes of the block-sparse mask (and of the kernels' outer tiles).

    ``num_warps`` / ``num_stages`` are accepted for source compatibility with callers written
    against the reference; the HIP kernels have a fixed wavefront count and pipeline depth, so
    the two fields are carried but not interpreted.
    """

    query_block_size: int = 64
    kv_block_size: int = 64
    num_warps: int = 4
    num_stages: int = 3


def get_default_flash_attention_params(backward: bool) -> FlashAttentionParamsConfig:
    """Default block sizes.

    The reference (common.py:21-41) requires a GPU and returns 128x128 forward / 64x128 backward
    on H100 and 64x64 elsewhere.  Here 128x128 is the default for both directions on gfx950: the
    backward kernels are kv-stationary with 128-row kv tiles and iterate query tiles of 128.
    No GPU query is made, so the defaults are also available on a CPU-only host.
    """
    del backward
    return FlashAttentionParamsConfig(
        query_block_size=128, kv_block_size=128, num_warps=4, num_stages=2
    )


def padded_length(seq_len: int, block_size: int) -> int:
    return (seq_len + block_size - 1) // block_size * block_size


def pad_to_block_size(
    embeddings: Sequence[torch.Tensor] | None,
    positions: torch.Tensor | None,
    segment_ids: torch.Tensor | None,
    block_size: int,
    pos_fill_value: int,
    transposed_inputs: bool = False,
):
    """Right-pad the sequence axis to a multiple of ``block_size``.

    Same contract as common.py:44-74: embeddings are zero padded (sequence axis 1 for BSHD,
    axis 2 when ``transposed_inputs``), positions are padded with ``pos_fill_value`` and segment
    ids with PADDING_SEGMENT_ID.  The HIP entry points do this padding virtually (bounds checks
    in the kernels), so this helper is only used by the CPU oracle and by callers that want
    materialised padded arrays.
    """
    seq_len = positions.shape[1]
    pad_len = padded_length(seq_len, block_size) - seq_len
    if pad_len > 0:
        if embeddings is not None:
            axis = 2 if transposed_inputs else 1
            padded = []
            for e in embeddings:
                shape = list(e.shape)
                shape[axis] = pad_len
                padded.append(torch.cat([e, e.new_zeros(shape)], dim=axis))
            embeddings = padded
        if positions is not None:
            positions = torch.nn.functional.pad(positions, (0, pad_len), value=pos_fill_value)
        if segment_ids is not None:
            segment_ids = torch.nn.functional.pad(
                segment_ids, (0, pad_len), value=PADDING_SEGMENT_ID
            )
    return embeddings, positions, segment_ids
