"""Verlet-skin displacement test as a torch custom op.

Same schema and mutation set as ``nvalchemi::_batch_neighbor_list_rebuild_inplace``
(nvalchemi/dynamics/_ops/neighbor_list_rebuild.py:37-139): ``rebuild_flags`` (pre-allocated,
``(M,)`` bool) is cleared and then set for every system holding an atom that moved more than
``skin_distance_threshold`` from ``reference_positions``; with ``update_reference_positions`` the
reference of the flagged systems is overwritten with the current positions.  Nothing is
allocated and the host is not synchronised.  ``cell_inv`` is accepted and ignored: the kernel
inverts the cell itself.  A shape mismatch between the two position tensors flags every system,
as the reference does (:95-98).
"""

from __future__ import annotations

import torch

from ... import _lib

__all__ = ["batch_neighbor_list_rebuild_inplace"]


@torch.library.custom_op("nvalchemi_amd::_batch_neighbor_list_rebuild_inplace",
                         mutates_args=("reference_positions", "rebuild_flags"))
def _batch_neighbor_list_rebuild_inplace(
    reference_positions: torch.Tensor, current_positions: torch.Tensor, batch_idx: torch.Tensor,
    rebuild_flags: torch.Tensor, skin_distance_threshold: float, update_reference_positions: bool = False,
    cell: torch.Tensor | None = None, cell_inv: torch.Tensor | None = None, pbc: torch.Tensor | None = None,
) -> None:
    if reference_positions.shape != current_positions.shape:
        rebuild_flags.fill_(True)
        return
    _lib.nl_rebuild_check(reference_positions, current_positions, batch_idx, rebuild_flags,
                          skin_distance_threshold, update_reference_positions,
                          cell if pbc is not None else None, pbc if cell is not None else None)


@_batch_neighbor_list_rebuild_inplace.register_fake
def _(reference_positions, current_positions, batch_idx, rebuild_flags, skin_distance_threshold,
      update_reference_positions=False, cell=None, cell_inv=None, pbc=None) -> None:
    pass


def batch_neighbor_list_rebuild_inplace(
    reference_positions: torch.Tensor, current_positions: torch.Tensor, batch_idx: torch.Tensor,
    rebuild_flags: torch.Tensor, skin_distance_threshold: float, update_reference_positions: bool = False,
    cell: torch.Tensor | None = None, cell_inv: torch.Tensor | None = None, pbc: torch.Tensor | None = None,
) -> None:
    """Write per-system rebuild flags into ``rebuild_flags`` in place (see the module note)."""
    _batch_neighbor_list_rebuild_inplace(reference_positions, current_positions, batch_idx, rebuild_flags,
                                         skin_distance_threshold, update_reference_positions, cell, cell_inv, pbc)
