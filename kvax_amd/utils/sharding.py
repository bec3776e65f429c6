"""Mesh bookkeeping for the single-GPU build.

The reference wraps every op in ``jax.experimental.shard_map`` over a jax ``Mesh``
(kvax/utils/sharding.py:37-67) and reads the context-parallel axis name and size from the global
attention specs (sharding.py:70-86).  This build runs on one GPU, so a mesh is only a mapping
``axis name -> size`` that tells the host code how many query shards a context-parallel call is
split into; the shards are then evaluated one after another on the same device.

Any object with a ``shape`` mapping (a jax ``Mesh`` included) is accepted wherever a mesh is.
"""
from __future__ import annotations

import threading
from typing import Mapping

from kvax_amd.utils.specs import Axes, get_attention_specs


class Mesh:
    """Minimal named-axis mesh: ``Mesh({"data": 1, "context": 8, "model": 1})``.

    Usable as a context manager to install itself as the thread's global mesh, like
    ``with jax_mesh:`` does for the reference (sharding.py:16-34).
    """

    def __init__(self, shape: Mapping[str, int]):
        self.shape = dict(shape)
        for name, size in self.shape.items():
            if not isinstance(size, int) or size < 1:
                raise ValueError(f"mesh axis {name!r} must have a positive integer size")

    @property
    def axis_names(self) -> tuple[str, ...]:
        return tuple(self.shape)

    def __enter__(self) -> "Mesh":
        stack = _mesh_stack()
        stack.append(self)
        return self

    def __exit__(self, *exc) -> None:
        _mesh_stack().pop()

    def __repr__(self) -> str:
        return f"Mesh({self.shape})"


_tls = threading.local()


def _mesh_stack() -> list:
    if not hasattr(_tls, "stack"):
        _tls.stack = []
    return _tls.stack


def _get_global_mesh():
    stack = _mesh_stack()
    return stack[-1] if stack else None


def _check_mesh_or_get_global(mesh):
    """Explicit mesh, else the innermost ``with Mesh(...)``; error if neither exists."""
    if mesh is None:
        mesh = _get_global_mesh()
    if mesh is None:
        raise ValueError(
            "Mesh weren't provided."
            " Either mesh should not be None or global Mesh needs to be set as"
            " a context."
        )
    return mesh


def get_query_context_mesh_axis_name(mesh=None, require_mesh: bool = True) -> str | None:
    """Name of the mesh axis the query sequence is sharded over (None: no context parallelism)."""
    if require_mesh:
        _check_mesh_or_get_global(mesh)
    return get_attention_specs().query_specs[Axes.query_sequence]


def get_query_context_mesh_axis_size(mesh=None) -> int:
    mesh = _check_mesh_or_get_global(mesh)
    axis = get_query_context_mesh_axis_name(mesh)
    if axis not in mesh.shape:
        raise ValueError(f"Mesh axis {axis} is not present in the device mesh shape.")
    return int(mesh.shape[axis])


def context_parallel_degree(mesh=None) -> int:
    """Number of query shards: 1 unless the specs name a context axis present in the mesh."""
    axis = get_attention_specs().query_specs[Axes.query_sequence]
    if axis is None:
        return 1
    mesh = _check_mesh_or_get_global(mesh)
    if axis not in mesh.shape:
        raise ValueError(f"Mesh axis {axis} is not present in the device mesh shape.")
    return int(mesh.shape[axis])
