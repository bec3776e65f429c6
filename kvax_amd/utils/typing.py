"""Array and mask types (layout contract of kvax/utils/typing.py:15-36)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

DeviceArray = torch.Tensor
# One entry per tensor axis: a mesh-axis name (str) or None, as in jax PartitionSpec tuples.
Specs = Tuple[Optional[str], ...]

FlattenedAttentionMask = Tuple[DeviceArray, DeviceArray, DeviceArray, DeviceArray]


@dataclass
class AttentionMask:
    """Block-sparse bounds of one mask, each int32 of shape [batch, shards, n_outer_blocks].

    For a query-outer mask (forward, dQ) entry ``[b, 0, i]`` describes query block ``i``:
    kv blocks in ``[lower, upper)`` may hold attendable pairs and those in
    ``[lower_full, upper_full)`` are attendable everywhere.  For the kv-outer mask (dK/dV) the
    entry describes kv block ``i`` and the bounds index query blocks (shard-local under context
    parallelism).  Field and flatten order follow typing.py:22-36.
    """

    lower_bounds: DeviceArray
    upper_bounds: DeviceArray
    lower_full_bounds: DeviceArray
    upper_full_bounds: DeviceArray

    def flatten(self) -> FlattenedAttentionMask:
        return (
            self.lower_bounds,
            self.upper_bounds,
            self.lower_full_bounds,
            self.upper_full_bounds,
        )

    @classmethod
    def unflatten(cls, flatten_mask: FlattenedAttentionMask) -> "AttentionMask":
        lower, upper, lower_full, upper_full = flatten_mask
        return cls(
            lower_bounds=lower,
            upper_bounds=upper,
            lower_full_bounds=lower_full,
            upper_full_bounds=upper_full,
        )
