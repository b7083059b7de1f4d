"""``NVTNoseHoover``: canonical sampling with a Nose-Hoover chain thermostat (mirror of
nvalchemi/dynamics/integrators/nvt_nose_hoover.py:62-281).  ``dt`` and ``thermostat_time`` in
femtoseconds, ``temperature`` in Kelvin, each a scalar or per system; held per system in internal
units (kT in eV).  A step is chain(dt/2) - kick - drift | forces | kick - chain(dt/2); the chain
state (``nhc_eta``, ``nhc_eta_dot``, ``nhc_Q``, ``nhc_ndof``) lives with the other per-system
state and follows its systems through a refill."""

from __future__ import annotations

from typing import Any

import torch

from .._ops._bridge import _make_state_batch, _to_per_system
from .._ops.nose_hoover import (nhc_chain_update_masked, nhc_compute_masses, nhc_position_update_masked,
                                nhc_velocity_half_step_masked)
from .._units import fs_to_internal_time
from ..base import BaseDynamics
from ..hooks._utils import KB_EV

__all__ = ["NVTNoseHoover"]


class NVTNoseHoover(BaseDynamics):
    __needs_keys__: set[str] = {"forces"}
    __provides_keys__: set[str] = {"positions", "velocities"}
    _honors_active_mask = True

    def __init__(self, model, dt: float | torch.Tensor, temperature: float | torch.Tensor,
                 thermostat_time: float | torch.Tensor, chain_length: int = 3, yoshida_order: int = 3,
                 n_steps: int | None = None, hooks: list | None = None, convergence_hook: Any = None,
                 **kwargs: Any) -> None:
        super().__init__(model=model, n_steps=n_steps, hooks=hooks, convergence_hook=convergence_hook, **kwargs)
        if yoshida_order not in (3, 5):
            raise ValueError(f"yoshida_order must be 3 or 5, got {yoshida_order}")
        if chain_length < 1:
            raise ValueError(f"chain_length must be >= 1, got {chain_length}")
        self._dt_init = fs_to_internal_time(dt)
        self._temperature_init = temperature
        self._thermostat_time_init = fs_to_internal_time(thermostat_time)
        self.chain_length = chain_length
        self.yoshida_order = yoshida_order

    def _state_dict(self, n: int, dev, dtype, Q: torch.Tensor, ndof: torch.Tensor) -> dict[str, torch.Tensor]:
        C = self.chain_length
        return {"dt": _to_per_system(self._dt_init, n, dev, dtype),
                "temperature": _to_per_system(self._temperature_init * KB_EV, n, dev, dtype),
                "thermostat_time": _to_per_system(self._thermostat_time_init, n, dev, dtype),
                "nhc_ndof": ndof,
                "nhc_eta": torch.zeros(n, C, dtype=dtype, device=dev),
                "nhc_eta_dot": torch.zeros(n, C, dtype=dtype, device=dev),
                "nhc_Q": Q,
                "nhc_ke2": torch.zeros(n, dtype=dtype, device=dev),
                "nhc_total_scale": torch.zeros(n, dtype=dtype, device=dev)}

    def _init_state(self, batch) -> None:
        M, dev, dtype = batch.num_graphs, batch.device, batch.positions.dtype
        kT = _to_per_system(self._temperature_init * KB_EV, M, dev, dtype)
        tau = _to_per_system(self._thermostat_time_init, M, dev, dtype)
        Q = nhc_compute_masses(kT, tau, batch.atomic_masses, batch.batch_idx, self.chain_length)
        ndof = (batch.num_nodes_per_graph.to(device=dev) * 3).to(dtype)
        self._state = _make_state_batch(self._state_dict(M, dev, dtype, Q, ndof), dev)

    def _make_new_state(self, n: int, template_batch):
        """State for ``n`` systems that join a running batch.  Their atom counts are not known here:
        like the reference (:169-213) the chain masses and the degrees of freedom are taken from the
        mean system size of the batch."""
        dev, dtype = template_batch.device, template_batch.positions.dtype
        kT = _to_per_system(self._temperature_init * KB_EV, n, dev, dtype)
        tau = _to_per_system(self._thermostat_time_init, n, dev, dtype)
        per_system = template_batch.num_nodes // max(template_batch.num_graphs, 1)
        ndof = torch.full((n,), per_system * 3, dtype=dtype, device=dev)
        Q = (kT * tau * tau).unsqueeze(1).repeat(1, self.chain_length)
        Q[:, 0] = Q[:, 0] * ndof
        return _make_state_batch(self._state_dict(n, dev, dtype, Q.contiguous(), ndof), dev)

    def _chain(self, batch) -> None:
        s = self._state
        nhc_chain_update_masked(batch.velocities, batch.atomic_masses, s.nhc_eta, s.nhc_eta_dot, s.nhc_Q,
                                s.temperature, s.dt, s.nhc_ndof, s.nhc_ke2, s.nhc_total_scale, batch.batch_idx,
                                True, self.yoshida_order, self._active_mask)

    def pre_update(self, batch) -> None:
        self._chain(batch)
        nhc_velocity_half_step_masked(batch.velocities, batch.forces, batch.atomic_masses, self._state.dt,
                                      batch.batch_idx, self._active_mask)
        nhc_position_update_masked(batch.positions, batch.velocities, self._state.dt, batch.batch_idx,
                                   self._active_mask)

    def post_update(self, batch) -> None:
        nhc_velocity_half_step_masked(batch.velocities, batch.forces, batch.atomic_masses, self._state.dt,
                                      batch.batch_idx, self._active_mask)
        self._chain(batch)
