"""``compute_neighbors``: one-shot neighbor data for a ``Batch``.

Mirror of nvalchemi/neighbors.py:56-277: resolves cutoff/format/half_list from a
``NeighborConfig``, drops cell and pbc when no system is periodic (:223-225), estimates K
(capped at ceil16(max atoms per system) without PBC, :227-236), builds, grows K by
``int(1.5*max)+1`` while ``max(count) >= K`` (:269-273), and publishes either the three
matrix keys on the atoms group or the COO edges group; stamps ``_neighbor_list_cutoff``.
"""

from __future__ import annotations

import torch

from ._neighbor_ops import estimate_max_neighbors, get_neighbor_list_from_neighbor_matrix, neighbor_list
from .data.batch import Batch, SegmentedGroup
from .models.base import NeighborConfig, NeighborListFormat

__all__ = ["compute_neighbors"]


def _raise_on_truncated_search(n_atoms: int, n_systems: int, device, cutoff: float) -> None:
    """The search looks at 32 periodic images per axis and direction at most: a cell that is singular
    or thinner than cutoff / 32 gives a truncated list, which the build reports in its status bits.
    Called where the host waits for the device anyway."""
    if n_atoms == 0:
        return
    from . import _lib

    now = int(_lib.nl_status(n_atoms, n_systems, device)[0])
    if now & _lib.NL_STATUS_CELL_TOO_THIN:
        raise ValueError(f"a periodic cell is singular or thinner than cutoff / 32 (cutoff {cutoff}): "
                         "its neighbor list would be truncated")


def _write_neighbor_data_to_batch(batch: Batch, neighbor_matrix: torch.Tensor, num_neighbors: torch.Tensor,
                                  neighbor_matrix_shifts: torch.Tensor | None,
                                  format: NeighborListFormat, cutoff: float,
                                  search_cutoff: float | None = None) -> None:
    """Publish neighbor data on *batch* (MATRIX: three atom keys; COO: a new edges group
    with per-graph edge counts) and stamp the cutoff.  ``search_cutoff`` is the radius the
    matrix was actually searched with (cutoff plus skin, a full list); it is kept on the batch
    together with the identity of the matrix so that a pair kernel may derive shifts from
    positions where the cell is wide enough."""
    object.__setattr__(batch, "_neighbor_search_cutoff", None)
    if format == NeighborListFormat.COO:
        coo = get_neighbor_list_from_neighbor_matrix(neighbor_matrix, num_neighbors,
                                                     neighbor_matrix_shifts, fill_value=batch.num_nodes)
        edges = coo[0].T  # (E, 2) int32, already laid out row by row
        if not edges.is_contiguous():
            edges = edges.contiguous()
        edge_ptr = coo[1]
        data = {"neighbor_list": edges}
        if len(coo) > 2:
            data["neighbor_list_shifts"] = coo[2]
        # edges of one graph are contiguous: per-graph counts from the atom-level CSR pointer
        bptr = batch.batch_ptr.to(torch.long)
        ep = edge_ptr[bptr]
        seg = (ep[1:] - ep[:-1]).to(torch.int32)
        group = SegmentedGroup(data, seg, batch.device)
        group._edge_ptr = edge_ptr
        batch._storage.groups["edges"] = group
    else:
        atoms = batch._atoms_group
        if atoms is None:
            raise RuntimeError("Cannot store neighbor data: batch has no atoms group.")
        atoms["neighbor_matrix"] = neighbor_matrix
        atoms["num_neighbors"] = num_neighbors
        if neighbor_matrix_shifts is not None:
            atoms["neighbor_matrix_shifts"] = neighbor_matrix_shifts
        if search_cutoff is not None:
            object.__setattr__(batch, "_neighbor_search_cutoff",
                               (float(search_cutoff), neighbor_matrix.data_ptr(), tuple(neighbor_matrix.shape)))
    batch._neighbor_list_cutoff = cutoff


def compute_neighbors(batch: Batch, cutoff: float | None = None, *, config: NeighborConfig | None = None,
                      format: NeighborListFormat = NeighborListFormat.MATRIX,
                      max_neighbors: int | None = None, half_list: bool = False) -> None:
    """Compute a neighbor list and write it into *batch* in place.

    Pass either *config* (then the scalar arguments are ignored) or *cutoff*.

    Raises
    ------
    ValueError
        If neither *cutoff* nor *config* is given.
    """
    if config is not None:
        cutoff = config.cutoff
        format = config.format
        half_list = config.half_list
    elif cutoff is None:
        raise ValueError("Either 'cutoff' or 'config' must be provided.")

    N = batch.num_nodes
    device = batch.device
    pbc = getattr(batch, "pbc", None)
    cell = getattr(batch, "cell", None)
    if pbc is not None and not bool(pbc.any()):
        pbc = None
        cell = None
    if cell is None:
        pbc = None

    if max_neighbors is None:
        max_neighbors = estimate_max_neighbors(cutoff=cutoff)
        if pbc is None and batch.max_num_nodes > 0:
            cap = ((batch.max_num_nodes + 15) // 16) * 16
            max_neighbors = min(max_neighbors, cap)

    batch_ptr = batch.batch_ptr.to(torch.int32)
    batch_idx = batch.batch_idx.to(torch.int32)

    while True:
        nb_matrix = torch.full((N, max_neighbors), N, dtype=torch.int32, device=device)
        nb_counts = torch.zeros(N, dtype=torch.int32, device=device)
        nb_shifts = None
        if pbc is not None:
            nb_shifts = torch.zeros(N, max_neighbors, 3, dtype=torch.int32, device=device)
        neighbor_list(positions=batch.positions, cutoff=cutoff, cell=cell, pbc=pbc,
                      max_neighbors=max_neighbors, half_fill=half_list, batch_ptr=batch_ptr,
                      batch_idx=batch_idx, neighbor_matrix=nb_matrix, num_neighbors=nb_counts,
                      neighbor_matrix_shifts=nb_shifts, rebuild_flags=None, tail_mode=0)
        actual_max = int(nb_counts.max()) if N > 0 else 0
        if actual_max < max_neighbors:
            break
        max_neighbors = int(actual_max * 1.5) + 1
    _raise_on_truncated_search(N, batch.num_graphs, device, cutoff)

    _write_neighbor_data_to_batch(batch, nb_matrix, nb_counts, nb_shifts, format, cutoff,
                                  search_cutoff=None if half_list else cutoff)
