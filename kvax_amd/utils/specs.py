"""Global sharding specs for the attention operands.

Behavioural mirror of kvax/utils/specs.py: an ``attention_specs(query_specs, kv_specs)`` context
manager sets two 4-tuples of mesh-axis names (batch, sequence, heads, head_dim); validation
rules follow specs.py:28-50.  On one GPU the specs only select *which* axis would be the
context-parallel one; nothing is distributed.
"""
from __future__ import annotations

from contextlib import contextmanager
from dataclasses import dataclass
from enum import IntEnum
from typing import Generator

from kvax_amd.utils.typing import Specs


@dataclass
class AttentionSpecs:
    query_specs: Specs | None = None
    kv_specs: Specs | None = None


class Axes(IntEnum):
    batch = 0
    query_sequence = 1
    kv_sequence = 1
    heads = 2
    kv_heads = 2
    head_dim = 3


_attention_specs = AttentionSpecs()


def _validate_attention_specs(query_specs: Specs, kv_specs: Specs) -> None:
    for name, specs in (("query_specs", query_specs), ("kv_specs", kv_specs)):
        if len(specs) != 4:
            raise ValueError(f"{name} must have exactly 4 dimensions, got {len(specs)}.")
    if query_specs[Axes.batch] != kv_specs[Axes.batch]:
        raise ValueError(
            "Batch dimension sharding must match between query_specs and kv_specs."
        )
    if query_specs[Axes.head_dim] != kv_specs[Axes.head_dim]:
        raise ValueError(
            "head_dim dimension sharding must match between query_specs and kv_specs."
        )
    if kv_specs[Axes.kv_sequence] is not None:
        raise ValueError(
            "Context parallelism with sharded key/value tensors is not supported."
        )
    if kv_specs[Axes.head_dim] is not None:
        raise ValueError("Sharding of attention_head_dim is not supported.")


def set_attention_specs(query_specs: Specs, kv_specs: Specs) -> None:
    _validate_attention_specs(query_specs, kv_specs)
    _attention_specs.query_specs = tuple(query_specs)
    _attention_specs.kv_specs = tuple(kv_specs)


def get_attention_specs() -> AttentionSpecs:
    if _attention_specs.query_specs is None or _attention_specs.kv_specs is None:
        raise ValueError(
            "Attention specifications must be initialised "
            "before calling get_attention_specs."
        )
    return _attention_specs


@contextmanager
def attention_specs(query_specs: Specs, kv_specs: Specs) -> Generator[None, None, None]:
    """Set the specs for the duration of a ``with`` block and restore the previous ones after."""
    saved = (_attention_specs.query_specs, _attention_specs.kv_specs)
    set_attention_specs(query_specs, kv_specs)
    try:
        yield
    finally:
        _attention_specs.query_specs, _attention_specs.kv_specs = saved
