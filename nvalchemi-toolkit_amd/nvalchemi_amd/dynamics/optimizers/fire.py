"""``FIRE``: fixed-cell FIRE optimizer (mirror of the ``FIRE`` class of
nvalchemi/dynamics/optimizers/fire.py:79-290).  Defaults: ``maxstep=0.2, n_min=5, f_dec=0.5,
f_inc=1.1, alpha_start=0.1, f_alpha=0.99``, ``dt_max = 10 dt``, ``dt_min = 0.02 dt``; ``dt`` is
used as given (it is not converted from femtoseconds).  ``pre_update`` performs the whole
FIRE step with the forces of the previous evaluation; ``post_update`` does nothing.

The order of the step (MD integration, then velocity mixing, then the parameter update, with the
sums taken at entry) is the one the reference's sentences give; its kernel is in a library outside
its tree, so the step is not pinned against the reference's output.  This order damps the first
kicks less than mixing before integrating would: from a start with pairs far up the repulsive
wall (a random gas) give ``maxstep`` a value well below the nearest-neighbor distance."""

from __future__ import annotations

from typing import Any

import torch

from .._ops._bridge import _make_state_batch, _to_per_system
from .._ops.fire import fire_step
from ..base import BaseDynamics

__all__ = ["FIRE"]

_FIRE_DEFAULTS = dict(maxstep=0.2, n_min=5, f_dec=0.5, f_inc=1.1, alpha_start=0.1, f_alpha=0.99)


class FIRE(BaseDynamics):
    __needs_keys__: set[str] = {"forces"}
    __provides_keys__: set[str] = {"positions", "velocities"}
    _honors_active_mask = True

    def __init__(self, model, dt: float | torch.Tensor, dt_max: float | torch.Tensor | None = None,
                 dt_min: float | torch.Tensor | None = None, maxstep: float = _FIRE_DEFAULTS["maxstep"],
                 n_min: int = _FIRE_DEFAULTS["n_min"], f_dec: float = _FIRE_DEFAULTS["f_dec"],
                 f_inc: float = _FIRE_DEFAULTS["f_inc"], alpha_start: float = _FIRE_DEFAULTS["alpha_start"],
                 f_alpha: float = _FIRE_DEFAULTS["f_alpha"], uphill: bool | torch.Tensor = False,
                 n_steps: int | None = None, hooks: list | None = None, convergence_hook: Any = None,
                 **kwargs: Any) -> None:
        super().__init__(model=model, n_steps=n_steps, hooks=hooks, convergence_hook=convergence_hook, **kwargs)
        if (isinstance(uphill, torch.Tensor) and bool(uphill.any())) or (not isinstance(uphill, torch.Tensor) and uphill):
            raise NotImplementedError("FIRE with uphill step checks is not implemented (vanilla FIRE only)")
        self._dt_init = dt
        self._dt_max_init = dt_max
        self._dt_min_init = dt_min
        self.maxstep = maxstep
        self.n_min = n_min
        self.f_dec = f_dec
        self.f_inc = f_inc
        self.alpha_start = alpha_start
        self.f_alpha = f_alpha

    def _state_dict(self, M: int, dev, dtype) -> dict[str, torch.Tensor]:
        dt = _to_per_system(self._dt_init, M, dev, dtype)
        dt_max = _to_per_system(self._dt_max_init, M, dev, dtype) if self._dt_max_init is not None else dt * 10.0
        dt_min = _to_per_system(self._dt_min_init, M, dev, dtype) if self._dt_min_init is not None else dt * 0.02
        full = lambda v, t=dtype: torch.full((M,), v, dtype=t, device=dev)  # noqa: E731
        return {
            "dt": dt, "dt_max": dt_max, "dt_min": dt_min, "alpha": full(self.alpha_start),
            "alpha_start": full(self.alpha_start), "f_alpha": full(self.f_alpha), "maxstep": full(self.maxstep),
            "n_min": full(self.n_min, torch.int32), "f_dec": full(self.f_dec), "f_inc": full(self.f_inc),
            "uphill_flag": torch.zeros(M, dtype=torch.int32, device=dev),
            "n_steps_positive": torch.zeros(M, dtype=torch.int32, device=dev),
            "vf": torch.zeros(M, dtype=dtype, device=dev), "vv": torch.zeros(M, dtype=dtype, device=dev),
            "ff": torch.zeros(M, dtype=dtype, device=dev),
        }

    def _init_state(self, batch) -> None:
        self._state = _make_state_batch(self._state_dict(batch.num_graphs, batch.device, batch.positions.dtype),
                                        batch.device)

    def _make_new_state(self, n: int, template_batch):
        return _make_state_batch(self._state_dict(n, template_batch.device, template_batch.positions.dtype),
                                 template_batch.device)

    def pre_update(self, batch) -> None:
        s = self._state
        fire_step(batch.positions, batch.velocities, batch.forces, batch.atomic_masses, s.alpha, s.dt,
                  s.n_steps_positive, s.alpha_start, s.f_alpha, s.dt_min, s.dt_max, s.maxstep, s.n_min,
                  s.f_dec, s.f_inc, s.uphill_flag, vf=s.vf, vv=s.vv, ff=s.ff, batch_idx=batch.batch_idx,
                  active=self._active_mask, uphill_checked=True)  # the flag is this class's own zeros

    def post_update(self, batch) -> None:
        """No-op; the new forces are consumed by the next ``pre_update``."""
