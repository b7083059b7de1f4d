"""``NVTLangevin``: canonical sampling by BAOAB Langevin dynamics (mirror of
nvalchemi/dynamics/integrators/nvt_langevin.py:49-196).  ``dt`` in femtoseconds, ``temperature``
in Kelvin, ``friction`` in 1/fs, each a scalar or per system; held per system in internal units
(kT in eV).  ``pre_update`` runs B-A-O-A with ``random_seed + step_count`` as the seed of the
step, ``post_update`` the final half kick with the new forces."""

from __future__ import annotations

from typing import Any

import torch

from .._ops._bridge import _make_state_batch, _to_per_system
from .._ops.langevin import langevin_finalize_masked, langevin_half_step_masked
from .._units import fs_to_internal_time, per_fs_to_internal_rate
from ..base import BaseDynamics
from ..hooks._utils import KB_EV

__all__ = ["NVTLangevin"]


class NVTLangevin(BaseDynamics):
    __needs_keys__: set[str] = {"forces"}
    __provides_keys__: set[str] = {"positions", "velocities"}
    _honors_active_mask = True

    def __init__(self, model, dt: float | torch.Tensor, temperature: float | torch.Tensor,
                 friction: float | torch.Tensor, random_seed: int = 42, n_steps: int | None = None,
                 hooks: list | None = None, convergence_hook: Any = None, **kwargs: Any) -> None:
        super().__init__(model=model, n_steps=n_steps, hooks=hooks, convergence_hook=convergence_hook, **kwargs)
        self._dt_init = fs_to_internal_time(dt)
        self._temperature_init = temperature
        self._friction_init = per_fs_to_internal_rate(friction)
        self._random_seed = random_seed

    def _state_dict(self, n: int, dev, dtype) -> dict[str, torch.Tensor]:
        return {"dt": _to_per_system(self._dt_init, n, dev, dtype),
                "temperature": _to_per_system(self._temperature_init * KB_EV, n, dev, dtype),
                "friction": _to_per_system(self._friction_init, n, dev, dtype)}

    def _init_state(self, batch) -> None:
        self._state = _make_state_batch(self._state_dict(batch.num_graphs, batch.device, batch.positions.dtype),
                                        batch.device)

    def _make_new_state(self, n: int, template_batch):
        return _make_state_batch(self._state_dict(n, template_batch.device, template_batch.positions.dtype),
                                 template_batch.device)

    def pre_update(self, batch) -> None:
        s = self._state
        langevin_half_step_masked(batch.positions, batch.velocities, batch.forces, batch.atomic_masses, s.dt,
                                  s.temperature, s.friction, self._random_seed + self.step_count, batch.batch_idx,
                                  self._active_mask)

    def post_update(self, batch) -> None:
        langevin_finalize_masked(batch.velocities, batch.forces, batch.atomic_masses, self._state.dt,
                                 batch.batch_idx, self._active_mask)
