"""Torch custom ops for the BAOAB Langevin integrator.

Same schemas and mutation sets as ``nvalchemi::langevin_half_step`` (mutates positions,
velocities) and ``nvalchemi::langevin_finalize`` (mutates velocities),
nvalchemi/dynamics/_ops/langevin.py:48-174:

    B  v += (F/m) dt/2      A  r += v dt/2      O  v = c1 v + c2 xi      A  r += v dt/2
    (after the forces at the new positions)     B  v += (F_new/m) dt/2

with ``c1 = exp(-friction dt)``, ``c2 = sqrt(kT/m (1 - c1^2))``, ``xi`` standard normal.
``temperature`` is kT in energy units, per system ``[M]``, like ``dt`` and ``friction``.  The
deviates of atom ``i`` depend on ``(random_seed, i)`` only; the stream is this library's own
(Philox4x32-10), not the reference's.  The ``*_masked`` functions take an ``active [M]`` mask.
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = ["langevin_half_step", "langevin_finalize", "langevin_half_step_masked", "langevin_finalize_masked"]


@torch.library.custom_op("nvalchemi_amd::langevin_half_step", mutates_args={"positions", "velocities"})
def langevin_half_step(positions: torch.Tensor, velocities: torch.Tensor, forces: torch.Tensor,
                       masses: torch.Tensor, dt: torch.Tensor, temperature: torch.Tensor, friction: torch.Tensor,
                       random_seed: int, batch_idx: torch.Tensor) -> None:
    _lib.langevin_half_step(positions, velocities, forces, masses, dt, temperature, friction, random_seed, batch_idx)


@langevin_half_step.register_fake
def _(positions, velocities, forces, masses, dt, temperature, friction, random_seed, batch_idx) -> None:
    pass


@torch.library.custom_op("nvalchemi_amd::langevin_finalize", mutates_args={"velocities"})
def langevin_finalize(velocities: torch.Tensor, forces_new: torch.Tensor, masses: torch.Tensor,
                      dt: torch.Tensor, batch_idx: torch.Tensor) -> None:
    _lib.vv_velocity_finalize(velocities, forces_new, masses, dt, batch_idx)


@langevin_finalize.register_fake
def _(velocities, forces_new, masses, dt, batch_idx) -> None:
    pass


def langevin_half_step_masked(positions, velocities, forces, masses, dt, temperature, friction, random_seed,
                              batch_idx, active=None) -> None:
    _lib.langevin_half_step(positions, velocities, forces, masses, dt, temperature, friction, random_seed,
                            batch_idx, active)


def langevin_finalize_masked(velocities, forces_new, masses, dt, batch_idx, active=None) -> None:
    _lib.vv_velocity_finalize(velocities, forces_new, masses, dt, batch_idx, active)
