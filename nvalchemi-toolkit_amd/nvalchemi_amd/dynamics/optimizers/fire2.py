"""``FIRE2``: fixed-cell FIRE 2.0 optimizer (mirror of the ``FIRE2`` class of
nvalchemi/dynamics/optimizers/fire2.py:94-254).  Defaults: ``delaystep=60, dtgrow=1.05, dtshrink=0.75,
alphashrink=0.985, alpha0=0.09, tmax=0.08, tmin=0.005, maxstep=0.1``; ``dt`` is used as given.
``pre_update`` performs the whole step with the forces of the previous evaluation; ``post_update`` does
nothing.  The variable-cell class of the reference (``FIRE2VariableCell``) is not provided."""

from __future__ import annotations

from typing import Any

import torch

from .._ops._bridge import _make_state_batch, _to_per_system
from .._ops.fire import fire2_step_coord
from ..base import BaseDynamics

__all__ = ["FIRE2"]

_FIRE2_DEFAULTS = dict(delaystep=60, dtgrow=1.05, dtshrink=0.75, alphashrink=0.985, alpha0=0.09, tmax=0.08,
                       tmin=0.005, maxstep=0.1)


class FIRE2(BaseDynamics):
    __needs_keys__: set[str] = {"forces"}
    __provides_keys__: set[str] = {"positions", "velocities"}
    _honors_active_mask = True

    def __init__(self, model, dt: float | torch.Tensor, delaystep: int = _FIRE2_DEFAULTS["delaystep"],
                 dtgrow: float = _FIRE2_DEFAULTS["dtgrow"], dtshrink: float = _FIRE2_DEFAULTS["dtshrink"],
                 alphashrink: float = _FIRE2_DEFAULTS["alphashrink"], alpha0: float = _FIRE2_DEFAULTS["alpha0"],
                 tmax: float = _FIRE2_DEFAULTS["tmax"], tmin: float = _FIRE2_DEFAULTS["tmin"],
                 maxstep: float = _FIRE2_DEFAULTS["maxstep"], n_steps: int | None = None,
                 hooks: list | None = None, convergence_hook: Any = None, **kwargs: Any) -> None:
        super().__init__(model=model, n_steps=n_steps, hooks=hooks, convergence_hook=convergence_hook, **kwargs)
        self._dt_init = dt
        self.delaystep = delaystep
        self.dtgrow = dtgrow
        self.dtshrink = dtshrink
        self.alphashrink = alphashrink
        self.alpha0 = alpha0
        self.tmax = tmax
        self.tmin = tmin
        self.maxstep = maxstep

    def _state_dict(self, n: int, dev, dtype) -> dict[str, torch.Tensor]:
        zeros = lambda: torch.zeros(n, dtype=dtype, device=dev)  # noqa: E731
        return {"dt": _to_per_system(self._dt_init, n, dev, dtype),
                "alpha": torch.full((n,), self.alpha0, dtype=dtype, device=dev),
                "nsteps_inc": torch.zeros(n, dtype=torch.int32, device=dev),
                "vf": zeros(), "v_sumsq": zeros(), "f_sumsq": zeros()}

    def _init_state(self, batch) -> None:
        self._state = _make_state_batch(self._state_dict(batch.num_graphs, batch.device, batch.positions.dtype),
                                        batch.device)

    def _make_new_state(self, n: int, template_batch):
        return _make_state_batch(self._state_dict(n, template_batch.device, template_batch.positions.dtype),
                                 template_batch.device)

    def pre_update(self, batch) -> None:
        s = self._state
        fire2_step_coord(batch.positions, batch.velocities, batch.forces, batch.batch_idx, s.alpha, s.dt,
                         s.nsteps_inc, vf=s.vf, v_sumsq=s.v_sumsq, f_sumsq=s.f_sumsq, delaystep=self.delaystep,
                         dtgrow=self.dtgrow, dtshrink=self.dtshrink, alphashrink=self.alphashrink,
                         alpha0=self.alpha0, tmax=self.tmax, tmin=self.tmin, maxstep=self.maxstep,
                         active=self._active_mask)

    def post_update(self, batch) -> None:
        """No-op; the new forces are consumed by the next ``pre_update``."""
