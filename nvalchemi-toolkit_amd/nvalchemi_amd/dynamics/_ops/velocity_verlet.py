"""Torch custom ops for the two velocity-Verlet halves.

Same schemas and mutation sets as ``nvalchemi::vv_position_update`` (mutates positions,
velocities) and ``nvalchemi::vv_velocity_finalize`` (mutates velocities),
nvalchemi/dynamics/_ops/velocity_verlet.py:50-138:

    r(t+dt) = r + v dt + 1/2 (F/m) dt^2 ,  v(t+dt/2) = v + 1/2 (F/m) dt
    v(t+dt) = v(t+dt/2) + 1/2 (F_new/m) dt

``dt`` is per system ``[M]`` and is looked up through ``batch_idx``.  The ``*_masked``
functions take an extra ``active [M]`` mask: systems with ``False`` are left untouched.
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = ["vv_position_update", "vv_velocity_finalize", "vv_position_update_masked",
           "vv_velocity_finalize_masked"]


@torch.library.custom_op("nvalchemi_amd::vv_position_update", mutates_args={"positions", "velocities"})
def vv_position_update(positions: torch.Tensor, velocities: torch.Tensor, forces: torch.Tensor,
                       masses: torch.Tensor, dt: torch.Tensor, batch_idx: torch.Tensor) -> None:
    _lib.vv_position_update(positions, velocities, forces, masses, dt, batch_idx)


@vv_position_update.register_fake
def _(positions, velocities, forces, masses, dt, batch_idx) -> None:
    pass


@torch.library.custom_op("nvalchemi_amd::vv_velocity_finalize", mutates_args={"velocities"})
def vv_velocity_finalize(velocities: torch.Tensor, forces_new: torch.Tensor, masses: torch.Tensor,
                         dt: torch.Tensor, batch_idx: torch.Tensor) -> None:
    _lib.vv_velocity_finalize(velocities, forces_new, masses, dt, batch_idx)


@vv_velocity_finalize.register_fake
def _(velocities, forces_new, masses, dt, batch_idx) -> None:
    pass


def vv_position_update_masked(positions, velocities, forces, masses, dt, batch_idx, active=None) -> None:
    _lib.vv_position_update(positions, velocities, forces, masses, dt, batch_idx, active)


def vv_velocity_finalize_masked(velocities, forces_new, masses, dt, batch_idx, active=None) -> None:
    _lib.vv_velocity_finalize(velocities, forces_new, masses, dt, batch_idx, active)
