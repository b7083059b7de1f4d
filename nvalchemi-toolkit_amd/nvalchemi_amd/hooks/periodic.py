"""``WrapPeriodicHook``: wrap positions back into the cell under periodic boundary conditions.

Mirror of nvalchemi/hooks/periodic.py:42-218.  ``wrap_positions_into_cell`` reduces all three
fractional coordinates to ``[0, 1)`` (``frac = positions @ inv(cell)``, rows of ``cell`` are the
lattice vectors), maps back to Cartesian, and keeps of the result only the Cartesian components
whose own ``pbc`` flag is set -- the masking the reference applies after its wrap kernel
(:111-113).  One kernel, in place, instead of a clone, the wrap, a gather of ``pbc`` and a
``where``.
"""

from __future__ import annotations

from enum import Enum

import torch

from .. import _lib
from ._context import HookContext

__all__ = ["WrapPeriodicHook", "wrap_positions_into_cell"]


@torch.library.custom_op("nvalchemi_amd::wrap_positions_", mutates_args=("positions",))
def _wrap_positions_(positions: torch.Tensor, cell: torch.Tensor, pbc: torch.Tensor,
                     batch_idx: torch.Tensor) -> None:
    _lib.wrap_positions(positions, cell, pbc, batch_idx)


@_wrap_positions_.register_fake
def _(positions, cell, pbc, batch_idx) -> None:
    pass


def wrap_positions_into_cell(positions: torch.Tensor, cell: torch.Tensor, pbc: torch.Tensor,
                             batch_idx: torch.Tensor) -> torch.Tensor:
    """Wrap ``positions`` (V, 3) in place and return the same tensor."""
    if positions.dtype not in (torch.float32, torch.float64):
        raise TypeError("wrap_positions_into_cell: float32 or float64 positions")
    _wrap_positions_(positions, cell.to(positions.dtype).contiguous(), pbc.to(torch.bool).contiguous(),
                     batch_idx.to(torch.int32))
    return positions


class WrapPeriodicHook:
    """Wrap ``batch.positions`` into the cell every ``frequency`` steps
    (``DynamicsStage.AFTER_POST_UPDATE`` in the reference's examples)."""

    #: a call is one kernel on the batch's own tensors: a dynamics may capture it in a HIP graph
    graph_safe = True

    def __init__(self, frequency: int = 1, stage: Enum | None = None) -> None:
        self.frequency = frequency
        self.stage = stage

    def _wrap_positions(self, batch) -> None:
        cell = batch.cell
        pbc = batch.pbc
        if cell.dim() == 4:
            cell = cell.squeeze(1)
        if pbc.dim() == 3:
            pbc = pbc.squeeze(1)
        wrap_positions_into_cell(batch.positions, cell, pbc, batch.batch_idx)

    def __call__(self, ctx: HookContext, stage: Enum) -> None:
        self._wrap_positions(ctx.batch)
