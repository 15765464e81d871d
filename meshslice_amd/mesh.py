"""Host emulation of the 2-D device mesh the reference builds with jax.sharding.Mesh.

The reference reads two attributes of its mesh object: ``mesh.axis_names`` and
``mesh.devices.shape`` (reference TensorParallel.py:349-350,359; ShardedLayers.py:28).  This class
offers exactly those.  No second GPU exists in this build: a mesh device is a coordinate ``(i, j)``
whose shards and received slices are extracted into the one GPU's HBM when its body runs.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import numpy as np


def create_device_mesh(shape: Tuple[int, int]) -> np.ndarray:
    """Logical device ids laid out as an ``R x C`` array (stand-in for mesh_utils.create_device_mesh)."""
    r, c = int(shape[0]), int(shape[1])
    if r < 1 or c < 1:
        raise ValueError(f"mesh shape must be positive, got {shape}")
    return np.arange(r * c).reshape(r, c)


class Mesh:
    """``Mesh(devices, axis_names=('row', 'col'))`` with ``devices`` an ``R x C`` array."""

    def __init__(self, devices, axis_names: Sequence[str] = ("row", "col")):
        devices = np.asarray(devices)
        if devices.ndim != 2:
            raise ValueError("the device mesh must be 2-D")
        if len(axis_names) != 2:
            raise ValueError("a 2-D mesh needs two axis names")
        self.devices = devices
        self.axis_names = tuple(axis_names)

    @property
    def shape(self) -> Tuple[int, int]:
        return tuple(int(s) for s in self.devices.shape)

    def __repr__(self) -> str:
        return f"Mesh({self.shape[0]}x{self.shape[1]}, axis_names={self.axis_names})"


class PartitionSpec(tuple):
    """``P(row, col)``: names the mesh axes that shard dim 0 and dim 1 of a matrix."""

    def __new__(cls, *names):
        return super().__new__(cls, names)


P = PartitionSpec


class NamedSharding:
    """Pairs a mesh with a partition spec (kept for call-site compatibility; data stays global)."""

    def __init__(self, mesh: Mesh, spec: PartitionSpec):
        self.mesh = mesh
        self.spec = spec


def device_put(x, sharding: NamedSharding = None):
    """Arrays stay whole on the one GPU; the sharding is applied logically when a body runs."""
    return x
