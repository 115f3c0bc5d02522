"""``MpmdMesh``: a device mesh with one axis designated as the pipeline
(MPMD) axis (reference: src/jaxpp/mesh.py:27-167).

JAX is the host in the reference and a ``jax.sharding.Mesh`` is what it wraps;
here the wrapped mesh is a :class:`DeviceMesh` - device ids in an ndarray plus
axis names - which is all the pipeline runtime reads from it.  One GPU executes
every MPMD group of the mesh, the way the reference's compiler tests map every
``mpmd_idx`` to the same device (tests/test_transformations.py:122-129).
"""
from __future__ import annotations

import dataclasses
from functools import cached_property
from typing import ClassVar

import numpy as np


@dataclasses.dataclass(frozen=True)
class DeviceMesh:
    """Stand-in for ``jax.sharding.Mesh``: ``devices`` ndarray + ``axis_names``."""

    devices: np.ndarray
    axis_names: tuple

    def __post_init__(self):
        object.__setattr__(self, "devices", np.asarray(self.devices))
        object.__setattr__(self, "axis_names", tuple(self.axis_names))
        if self.devices.ndim != len(self.axis_names):
            raise ValueError(f"{self.devices.ndim}-d device array with axes {self.axis_names}")

    @property
    def shape(self) -> dict:
        return dict(zip(self.axis_names, self.devices.shape))

    is_multi_process = False

    def __hash__(self):
        return hash((self.devices.tobytes(), self.devices.shape, self.axis_names))

    def __eq__(self, other):
        return (isinstance(other, DeviceMesh) and self.axis_names == other.axis_names
                and np.array_equal(self.devices, other.devices))


@dataclasses.dataclass(frozen=True)
class MpmdMesh:
    jax_mesh: DeviceMesh
    mpmd_axis_name: str
    mesh_stack: ClassVar[list] = []

    def __post_init__(self):
        if self.mpmd_axis_name not in self.jax_mesh.axis_names:
            raise ValueError(f"{self.mpmd_axis_name!r} is not an axis of {self.jax_mesh.axis_names}")

    def __enter__(self):
        MpmdMesh.mesh_stack.append(self)
        return self

    def __exit__(self, exc_type, exc_value, traceback):
        self.mesh_stack.pop()

    @cached_property
    def mpmd_axis(self) -> int:
        return self.jax_mesh.axis_names.index(self.mpmd_axis_name)

    @cached_property
    def mpmd_dim(self) -> int:
        return self.jax_mesh.shape[self.mpmd_axis_name]

    @cached_property
    def device_coords(self) -> dict:
        return {int(dev): coord for coord, dev in np.ndenumerate(self.jax_mesh.devices)}

    @cached_property
    def device_mpmd_idx(self) -> dict:
        return {dev: coord[self.mpmd_axis] for dev, coord in self.device_coords.items()}

    @cached_property
    def unstack(self) -> list:
        """One mesh per MPMD group, the MPMD axis kept with size 1."""
        return [DeviceMesh(part, self.jax_mesh.axis_names)
                for part in np.split(self.jax_mesh.devices, self.mpmd_dim, self.mpmd_axis)]

    @property
    def mpmd_idx_for_mesh(self) -> dict:
        return {mesh: i for i, mesh in enumerate(self.unstack)}

    def lowering_mesh(self) -> DeviceMesh:
        return self.mpmd_submesh([0]).jax_mesh

    def mpmd_submesh(self, mpmd_indices: list) -> "MpmdMesh":
        assert isinstance(mpmd_indices, list)
        return MpmdMesh(DeviceMesh(np.take(self.jax_mesh.devices, mpmd_indices, self.mpmd_axis),
                                   self.jax_mesh.axis_names), self.mpmd_axis_name)
