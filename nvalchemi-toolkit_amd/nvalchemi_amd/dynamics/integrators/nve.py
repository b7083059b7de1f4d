"""``NVE``: microcanonical dynamics by velocity Verlet (mirror of
nvalchemi/dynamics/integrators/nve.py:56-178).  ``dt`` is given in femtoseconds and held
per system in internal time units; ``pre_update`` moves positions and half-kicks velocities
with the forces of the previous evaluation, ``post_update`` finishes the kick with the new
forces."""

from __future__ import annotations

from typing import Any

import torch

from .._ops._bridge import _make_state_batch, _to_per_system
from .._ops.velocity_verlet import vv_position_update_masked, vv_velocity_finalize_masked
from .._units import fs_to_internal_time
from ..base import BaseDynamics

__all__ = ["NVE"]


class NVE(BaseDynamics):
    __needs_keys__: set[str] = {"forces"}
    __provides_keys__: set[str] = {"positions", "velocities"}
    _honors_active_mask = True

    def __init__(self, model, dt: float | torch.Tensor, n_steps: int | None = None, hooks: list | None = None,
                 convergence_hook: Any = None, **kwargs: Any) -> None:
        super().__init__(model=model, n_steps=n_steps, hooks=hooks, convergence_hook=convergence_hook, **kwargs)
        self._dt_init = fs_to_internal_time(dt)

    def _init_state(self, batch) -> None:
        M = batch.num_graphs
        self._state = _make_state_batch(
            {"dt": _to_per_system(self._dt_init, M, batch.device, batch.positions.dtype)}, batch.device)

    def _make_new_state(self, n: int, template_batch):
        return _make_state_batch(
            {"dt": _to_per_system(self._dt_init, n, template_batch.device, template_batch.positions.dtype)},
            template_batch.device)

    def pre_update(self, batch) -> None:
        vv_position_update_masked(batch.positions, batch.velocities, batch.forces, batch.atomic_masses,
                                  self._state.dt, batch.batch_idx, self._active_mask)

    def post_update(self, batch) -> None:
        vv_velocity_finalize_masked(batch.velocities, batch.forces, batch.atomic_masses, self._state.dt,
                                    batch.batch_idx, self._active_mask)

    def post_then_pre_update(self, batch) -> bool:
        """``post_update`` of one step and ``pre_update`` of the next in one launch; False where that form does
        not exist (float64 arrays), and the caller makes the two calls."""
        if batch.positions.dtype != torch.float32:
            return False
        from ... import _lib

        _lib.vv_finalize_then_update(batch.positions, batch.velocities, batch.forces, batch.atomic_masses,
                                     self._state.dt, batch.batch_idx, self._active_mask)
        return True
