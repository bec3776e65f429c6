"""Load-balancing token permutation for causal context parallelism.

The sequence axis (axis 1) is cut into ``2*cp`` equal chunks which are reordered as
``[0, 2cp-1, 1, 2cp-2, ...]`` so that shard ``r`` of ``cp`` owns original chunks ``r`` and
``2cp-1-r``: one cheap and one expensive chunk under a causal mask.  Behaviour follows
kvax/utils/permutation.py:9-116.
"""
from __future__ import annotations

from typing import Sequence

import torch

from kvax_amd.utils.sharding import get_query_context_mesh_axis_size
from kvax_amd.utils.typing import DeviceArray


def generate_shard_indices(num_shards: int, reverse: bool = False) -> list[int]:
    """Chunk order ``[(i, num_shards-1-i) for i < num_shards/2]`` flattened, or its inverse."""
    order = []
    for i in range(num_shards // 2):
        order += [i, num_shards - 1 - i]
    if not reverse:
        return order
    inverse = [0] * len(order)
    for dst, src in enumerate(order):
        inverse[src] = dst
    return inverse


def apply_permutation(
    inputs: Sequence[DeviceArray], num_shards: int, reverse_permutation: bool
) -> list[DeviceArray]:
    order = generate_shard_indices(num_shards, reverse=reverse_permutation)
    outputs = []
    for x in inputs:
        seq = x.shape[1]
        if seq % num_shards != 0:
            raise ValueError(
                f"sequence length {seq} is not divisible by the number of chunks {num_shards}"
            )
        idx = torch.as_tensor(order, device=x.device, dtype=torch.long)
        chunks = x.reshape(x.shape[0], num_shards, seq // num_shards, *x.shape[2:])
        outputs.append(chunks.index_select(1, idx).reshape(x.shape))
    return outputs


def _run(inputs, mesh, reverse: bool):
    num_shards = 2 * get_query_context_mesh_axis_size(mesh)
    single = isinstance(inputs, torch.Tensor)
    if single:
        inputs = (inputs,)
    lead = tuple(inputs[0].shape[:2])
    for x in inputs:
        if tuple(x.shape[:2]) != lead:
            raise AssertionError(
                f"inputs must share their (batch, sequence) prefix, got {lead} and "
                f"{tuple(x.shape[:2])}"
            )
    outputs = apply_permutation(inputs, num_shards, reverse)
    return outputs[0] if single else outputs


def permute_tokens_context_parallelism(inputs, mesh=None):
    """Reorder tokens along axis 1 for balanced causal work across context shards."""
    return _run(inputs, mesh, reverse=False)


def unpermute_tokens_context_parallelism(inputs, mesh=None):
    """Inverse of :func:`permute_tokens_context_parallelism`."""
    return _run(inputs, mesh, reverse=True)
