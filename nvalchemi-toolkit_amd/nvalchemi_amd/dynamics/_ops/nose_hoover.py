"""Torch custom ops for the Nose-Hoover chain (NHC) thermostat.

Same names, argument orders and mutation sets as nvalchemi/dynamics/_ops/nose_hoover.py:

``nhc_compute_masses`` (:54-127)
    ``Q_1 = N_f kT tau^2``, ``Q_k = kT tau^2`` for ``k > 1``, per system, ``N_f`` three times the
    system's atom count.  (The reference notes that its kernel may apply the first system's
    values to all; here every system gets its own.)
``nhc_chain_update`` (:143-246)
    advances the chain by half a step and scales the velocities: mutates ``velocities``, ``eta``,
    ``eta_dot``, ``ke2``, ``total_scale`` (``step_scale`` and ``dt_chain`` are scratch of the
    reference's kernel: accepted, left as they are).  The reference's op has no argument for the
    order of the Suzuki-Yoshida factorisation; here it is a trailing ``yoshida_order`` (1, 3, 5).
``nhc_velocity_half_step`` (:248-289)
    ``v += (F/m) dt/2``.
``nhc_position_update`` (:291-325)
    ``r += v dt``.

``temperature`` is kT in energy units per system ``[M]``, like ``dt``.  The ``*_masked`` functions
take an ``active [M]`` mask.  The reference's kernel is inside its kernel library: the chain
propagator here is the published one (Martyna, Tuckerman, Tobias, Klein 1996).
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = ["nhc_compute_masses", "nhc_chain_update", "nhc_velocity_half_step", "nhc_position_update",
           "nhc_chain_update_masked", "nhc_velocity_half_step_masked", "nhc_position_update_masked"]


def nhc_compute_masses(temperature: torch.Tensor, thermostat_time: torch.Tensor, masses: torch.Tensor,
                       batch_idx: torch.Tensor, chain_length: int) -> torch.Tensor:
    """Chain masses ``[M, chain_length]`` in the dtype of ``temperature`` (kT)."""
    M = temperature.shape[0]
    ndof = (torch.bincount(batch_idx.to(torch.long), minlength=M) * 3).to(temperature.dtype)
    q = (temperature * thermostat_time * thermostat_time).unsqueeze(1).repeat(1, chain_length)
    q[:, 0] = q[:, 0] * ndof
    return q.contiguous()


@torch.library.custom_op("nvalchemi_amd::nhc_chain_update",
                         mutates_args={"velocities", "eta", "eta_dot", "ke2", "total_scale", "step_scale",
                                       "dt_chain"})
def nhc_chain_update(velocities: torch.Tensor, masses: torch.Tensor, eta: torch.Tensor, eta_dot: torch.Tensor,
                     Q: torch.Tensor, temperature: torch.Tensor, dt: torch.Tensor, ndof: torch.Tensor,
                     ke2: torch.Tensor, total_scale: torch.Tensor, step_scale: torch.Tensor,
                     dt_chain: torch.Tensor, batch_idx: torch.Tensor, compute_ke: bool = True,
                     yoshida_order: int = 3) -> None:
    _lib.nhc_chain_update(velocities, masses, eta, eta_dot, Q, temperature, dt, ndof, ke2, total_scale, batch_idx,
                          compute_ke, yoshida_order)


@nhc_chain_update.register_fake
def _(velocities, masses, eta, eta_dot, Q, temperature, dt, ndof, ke2, total_scale, step_scale, dt_chain,
      batch_idx, compute_ke=True, yoshida_order=3) -> None:
    pass


@torch.library.custom_op("nvalchemi_amd::nhc_velocity_half_step", mutates_args={"velocities"})
def nhc_velocity_half_step(velocities: torch.Tensor, forces: torch.Tensor, masses: torch.Tensor, dt: torch.Tensor,
                           batch_idx: torch.Tensor) -> None:
    _lib.vv_velocity_finalize(velocities, forces, masses, dt, batch_idx)


@nhc_velocity_half_step.register_fake
def _(velocities, forces, masses, dt, batch_idx) -> None:
    pass


@torch.library.custom_op("nvalchemi_amd::nhc_position_update", mutates_args={"positions"})
def nhc_position_update(positions: torch.Tensor, velocities: torch.Tensor, dt: torch.Tensor,
                        batch_idx: torch.Tensor) -> None:
    _lib.nhc_position_update(positions, velocities, dt, batch_idx)


@nhc_position_update.register_fake
def _(positions, velocities, dt, batch_idx) -> None:
    pass


def nhc_chain_update_masked(velocities, masses, eta, eta_dot, Q, temperature, dt, ndof, ke2, total_scale,
                            batch_idx, compute_ke=True, yoshida_order=3, active=None) -> None:
    _lib.nhc_chain_update(velocities, masses, eta, eta_dot, Q, temperature, dt, ndof, ke2, total_scale, batch_idx,
                          compute_ke, yoshida_order, active)


def nhc_velocity_half_step_masked(velocities, forces, masses, dt, batch_idx, active=None) -> None:
    _lib.vv_velocity_finalize(velocities, forces, masses, dt, batch_idx, active)


def nhc_position_update_masked(positions, velocities, dt, batch_idx, active=None) -> None:
    _lib.nhc_position_update(positions, velocities, dt, batch_idx, active)
