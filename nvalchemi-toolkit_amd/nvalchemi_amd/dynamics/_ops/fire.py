"""Torch custom op and public wrapper for the FIRE step.

Same schema and mutation set as ``nvalchemi::_fire_step_op`` and the same public
``fire_step`` signature (nvalchemi/dynamics/_ops/fire.py:79-140,245-362).  Per system, with
the reductions ``vf = sum F.v``, ``vv = sum v.v``, ``ff = sum F.F`` taken over the arrays as
passed in, "an MD integration step followed by FIRE velocity mixing and adaptive parameter
updates" (nvalchemi/dynamics/_ops/fire.py:270-272):

    MD      : v1 = v + dt F/m ; dr = dt v1 ; |dr| > maxstep -> dr *= maxstep/|dr| ; r += dr
              (dt as stored)
    vf >= 0 : v <- (1-alpha) v1 + alpha sqrt(vv/ff) F        (alpha as stored)
              n+ += 1 ; if n+ > n_min : dt = min(dt f_inc, dt_max) ; alpha *= f_alpha
    vf < 0  : v <- 0 ; n+ = 0 ; dt = max(dt f_dec, dt_min) ; alpha = alpha_start

All atoms of a system see the same pre-update scalars.  The reference's own step is in a kernel
library outside its tree, so what its sentences leave open (the side of ``vf == 0``, ``>`` against
``>=`` for ``n_min``, the Euler form) is this library's choice, and the whole step is unpinned
against the reference's output.  With the sums taken at entry and the mixing applied to the kicked
velocity, the step is less damped than a mix-then-integrate FIRE.  Only the vanilla branch exists:
``fire_step`` raises ``NotImplementedError`` for a non-zero ``uphill_flag``.
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = ["fire_step", "fire2_step_coord"]


@torch.library.custom_op(
    "nvalchemi_amd::_fire_step_op",
    mutates_args={"positions", "velocities", "alpha", "dt", "n_steps_positive", "vf", "vv", "ff"},
)
def _fire_step_op(positions: torch.Tensor, velocities: torch.Tensor, forces: torch.Tensor,
                  masses: torch.Tensor, alpha: torch.Tensor, dt: torch.Tensor, alpha_start: torch.Tensor,
                  f_alpha: torch.Tensor, dt_min: torch.Tensor, dt_max: torch.Tensor, maxstep: torch.Tensor,
                  n_steps_positive: torch.Tensor, n_min: torch.Tensor, f_dec: torch.Tensor,
                  f_inc: torch.Tensor, uphill_flag: torch.Tensor, vf: torch.Tensor, vv: torch.Tensor,
                  ff: torch.Tensor, batch_idx: torch.Tensor, compute_reductions: bool = True) -> None:
    _lib.fire_step(positions, velocities, forces, masses, alpha, dt, alpha_start, f_alpha, dt_min, dt_max,
                   maxstep, n_steps_positive, n_min, f_dec, f_inc, uphill_flag, vf, vv, ff, batch_idx,
                   compute_reductions)


@_fire_step_op.register_fake
def _(positions, velocities, forces, masses, alpha, dt, alpha_start, f_alpha, dt_min, dt_max, maxstep,
      n_steps_positive, n_min, f_dec, f_inc, uphill_flag, vf, vv, ff, batch_idx,
      compute_reductions=True) -> None:
    pass


def fire_step(positions: torch.Tensor, velocities: torch.Tensor, forces: torch.Tensor,
              masses: torch.Tensor, alpha: torch.Tensor, dt: torch.Tensor, n_steps_positive: torch.Tensor,
              alpha_start: torch.Tensor, f_alpha: torch.Tensor, dt_min: torch.Tensor, dt_max: torch.Tensor,
              maxstep: torch.Tensor, n_min: torch.Tensor, f_dec: torch.Tensor, f_inc: torch.Tensor,
              uphill_flag: torch.Tensor, *, vf: torch.Tensor | None = None, vv: torch.Tensor | None = None,
              ff: torch.Tensor | None = None, batch_idx: torch.Tensor | None = None,
              compute_reductions: bool = True, active: torch.Tensor | None = None,
              uphill_checked: bool = False) -> None:
    """Full FIRE step; mutates positions, velocities, alpha, dt, n_steps_positive (and the
    scratch ``vf``/``vv``/``ff``, allocated when ``None``).  ``active [M] bool`` (extension):
    systems with ``False`` are left untouched.

    Only vanilla FIRE is built: a non-zero ``uphill_flag`` raises ``NotImplementedError`` (its
    semantics are not stated anywhere in the reference's tree).  Looking at the flag costs a
    read-back from the device; a caller that has made the flag itself and knows it to be zero
    (the ``FIRE`` class) says so with ``uphill_checked=True`` (extension) and pays nothing."""
    if not uphill_checked and uphill_flag is not None and bool((uphill_flag != 0).any()):
        raise NotImplementedError("fire_step: uphill_flag = 1 (FIRE with uphill step checks) is not implemented")
    M = alpha.shape[0]
    dtype, device = positions.dtype, positions.device
    if vf is None:
        vf = torch.zeros(M, dtype=dtype, device=device)
    if vv is None:
        vv = torch.zeros(M, dtype=dtype, device=device)
    if ff is None:
        ff = torch.zeros(M, dtype=dtype, device=device)
    if batch_idx is None:
        batch_idx = torch.zeros(positions.shape[0], dtype=torch.int32, device=device)
    _lib.fire_step(positions, velocities, forces, masses, alpha, dt, alpha_start, f_alpha, dt_min, dt_max,
                   maxstep, n_steps_positive, n_min, f_dec, f_inc, uphill_flag, vf, vv, ff, batch_idx,
                   compute_reductions, active)


def fire2_step_coord(positions: torch.Tensor, velocities: torch.Tensor, forces: torch.Tensor,
                     batch_idx: torch.Tensor, alpha: torch.Tensor, dt: torch.Tensor, nsteps_inc: torch.Tensor, *,
                     vf: torch.Tensor | None = None, v_sumsq: torch.Tensor | None = None,
                     f_sumsq: torch.Tensor | None = None, max_norm: torch.Tensor | None = None,
                     delaystep: int = 60, dtgrow: float = 1.05, dtshrink: float = 0.75, alphashrink: float = 0.985,
                     alpha0: float = 0.09, tmax: float = 0.08, tmin: float = 0.005, maxstep: float = 0.1,
                     active: torch.Tensor | None = None) -> None:
    """One FIRE 2.0 step with fixed cells; same arguments and defaults as ``fire2_step_coord`` of
    nvalchemi/dynamics/_ops/fire.py:467-557.  Mutates ``positions``, ``velocities``, ``alpha``, ``dt``,
    ``nsteps_inc`` and, when given, the outputs ``vf``, ``v_sumsq``, ``f_sumsq`` (sum F.v, v.v, F.F per
    system at entry) and ``max_norm`` (largest atomic displacement before the ``maxstep`` limit).
    ``active [M] bool`` (extension): systems with ``False`` are left untouched.

    The reference delegates the step to its kernel library; what runs here is FIRE 2.0 as published
    with its LAMMPS implementation (Guenole et al. 2020), semi-implicit Euler with unit masses:
    downhill (``sum F.v > 0``) the velocity is kicked, then mixed with the force direction; past
    ``delaystep`` downhill steps in a row ``dt`` grows (up to ``tmax``) and ``alpha`` decays; otherwise
    the positions go half a step back, the velocities restart from zero, ``alpha`` from ``alpha0`` and
    ``dt`` shrinks (not below ``tmin``).  A system's step is scaled down so that no atom moves further
    than ``maxstep``."""
    _lib.fire2_step(positions, velocities, forces, batch_idx, alpha, dt, nsteps_inc, vf, v_sumsq, f_sumsq, max_norm,
                    delaystep=delaystep, dtgrow=dtgrow, dtshrink=dtshrink, alphashrink=alphashrink, alpha0=alpha0,
                    tmax=tmax, tmin=tmin, maxstep=maxstep, active=active)
