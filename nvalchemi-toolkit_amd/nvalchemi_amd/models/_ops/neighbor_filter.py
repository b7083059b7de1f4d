"""Filtering and converting neighbor data for a model whose cutoff is tighter than the one the
list was built with.  Mirror of nvalchemi/models/_ops/neighbor_filter.py: ``filter_neighbor_matrix``
(:43-144), ``filter_neighbor_list`` (:147-224), ``neighbor_matrix_to_list`` (:227-283) and
``prepare_neighbors_for_model`` (:286-430) with the same arguments, results and errors.  The
reference does this in Torch; here the distance tests and the row compaction are HIP kernels
(``csrc/filter.hip``, ``csrc/coo.hip``).

Geometry: ``r_ij = r_j - r_i + shift . cell`` with the rows of ``cell`` as lattice vectors, kept iff
``|r_ij|^2 < cutoff^2`` (strict).  Evaluated in double on the float32 inputs, where the reference
rounds to float32 along the way: results can differ only for pairs within float32 rounding of the
cutoff.  float32 positions only.
"""

from __future__ import annotations

import torch
from torch import Tensor

from nvalchemi_amd import _lib
from nvalchemi_amd.models.base import NeighborListFormat

__all__ = ["filter_neighbor_list", "filter_neighbor_matrix", "neighbor_matrix_to_list", "prepare_neighbors_for_model"]


def _f32(positions: Tensor) -> None:
    if positions.dtype != torch.float32:
        raise NotImplementedError("the HIP neighbor filter takes float32 positions")


def _cell_args(cell: Tensor | None, batch_idx: Tensor | None, dtype) -> tuple[Tensor | None, Tensor | None]:
    if cell is None:
        return None, None
    if cell.dim() == 2:
        return cell.to(dtype).contiguous(), None
    if batch_idx is None:
        raise ValueError("batch_idx is required when cell has shape (B, 3, 3).")
    return cell.to(dtype).contiguous(), batch_idx.to(torch.int32).contiguous()


def filter_neighbor_matrix(positions: Tensor, cutoff: float, neighbor_matrix: Tensor, num_neighbors: Tensor,
                           fill_value: int, cell: Tensor | None = None,
                           neighbor_matrix_shifts: Tensor | None = None,
                           batch_idx: Tensor | None = None) -> tuple[Tensor, Tensor, Tensor | None]:
    """``(neighbor_matrix (N,K), num_neighbors (N), neighbor_matrix_shifts (N,K,3) | None)`` with the
    entries beyond ``cutoff`` removed: survivors packed to the front of each row in their order,
    ``fill_value`` (zero shifts) behind them.  Slots are valid by their index (``< fill_value``)."""
    _f32(positions)
    N, K = neighbor_matrix.shape
    use_cell = cell is not None and neighbor_matrix_shifts is not None
    c, bi = _cell_args(cell, batch_idx, positions.dtype) if use_cell else (None, None)
    nm = neighbor_matrix.to(torch.int32).contiguous()
    sh = None if neighbor_matrix_shifts is None else neighbor_matrix_shifts.to(torch.int32).contiguous()
    out_nm = torch.empty_like(nm)
    out_nn = torch.empty(N, dtype=torch.int32, device=nm.device)
    out_sh = None if sh is None else torch.empty_like(sh)
    _lib.nl_filter_matrix(positions.contiguous(), c, nm, sh, bi, fill_value, cutoff, out_nm, out_nn, out_sh)
    return out_nm, out_nn.to(num_neighbors.dtype), out_sh


def filter_neighbor_list(positions: Tensor, cutoff: float, neighbor_list: Tensor, neighbor_ptr: Tensor,
                         cell: Tensor | None = None, neighbor_list_shifts: Tensor | None = None,
                         batch_idx: Tensor | None = None) -> tuple[Tensor, Tensor, Tensor | None]:
    """``(neighbor_list (M',2), neighbor_ptr (N+1), neighbor_list_shifts (M',3) | None)`` with the
    edges beyond ``cutoff`` removed.  One host synchronisation (the number of survivors), as in the
    reference."""
    _f32(positions)
    N = positions.shape[0]
    use_cell = cell is not None and neighbor_list_shifts is not None
    c, bi = _cell_args(cell, batch_idx, positions.dtype) if use_cell else (None, None)
    nl = neighbor_list.to(torch.int32).contiguous()
    sh = None if neighbor_list_shifts is None else neighbor_list_shifts.to(torch.int32).contiguous()
    keep = torch.empty(nl.shape[0], dtype=torch.bool, device=nl.device)
    _lib.nl_filter_coo_flags(positions.contiguous(), c, nl, sh if use_cell else None, bi, cutoff, keep)
    keep_idx = keep.nonzero(as_tuple=False).squeeze(1)
    new_nl = neighbor_list[keep_idx]
    out_shifts = None if neighbor_list_shifts is None else neighbor_list_shifts[keep_idx]
    counts = torch.bincount(neighbor_list[:, 0][keep_idx].to(torch.long), minlength=N).to(neighbor_ptr.dtype)
    new_ptr = torch.zeros(N + 1, dtype=neighbor_ptr.dtype, device=positions.device)
    new_ptr[1:] = counts.cumsum(0)
    return new_nl, new_ptr, out_shifts


def neighbor_matrix_to_list(neighbor_matrix: Tensor, num_neighbors: Tensor, fill_value: int,
                            neighbor_matrix_shifts: Tensor | None = None) -> tuple[Tensor, Tensor, Tensor | None]:
    """Dense matrix to ``(neighbor_list (M,2) int32, neighbor_ptr (N+1) int32, shifts (M,3) | None)``
    in row-major order.  The rows must be packed (valid entries first, as every builder and
    :func:`filter_neighbor_matrix` leave them): the first ``num_neighbors[i]`` slots of row ``i``
    are its edges."""
    N, K = neighbor_matrix.shape
    dev = neighbor_matrix.device
    nm = neighbor_matrix.to(torch.int32).contiguous()
    nn = num_neighbors.to(torch.int32).contiguous()
    ptr = torch.empty(N + 1, dtype=torch.int32, device=dev)
    _lib.nl_edge_ptr(nn, K, ptr)
    M = int(ptr[-1]) if N > 0 else 0  # the one synchronisation: the output's size
    nl = torch.empty((M, 2), dtype=torch.int32, device=dev)
    sh = None if neighbor_matrix_shifts is None else neighbor_matrix_shifts.to(torch.int32).contiguous()
    out_sh = None if sh is None else torch.empty((M, 3), dtype=torch.int32, device=dev)
    if M > 0:
        _lib.nl_matrix_to_coo(nm, sh, ptr, nl, out_sh)
    return nl, ptr, out_sh


def prepare_neighbors_for_model(data, model_cutoff: float, target_format: NeighborListFormat,
                                fill_value: int) -> dict[str, Tensor]:
    """Neighbor tensors in the format a model expects, filtered to ``model_cutoff`` when the batch's
    list was built with a larger one (``data._neighbor_list_cutoff``).  MATRIX: ``neighbor_matrix``,
    ``num_neighbors`` (+ ``neighbor_matrix_shifts``); COO: ``neighbor_list``, ``edge_ptr``
    (+ ``neighbor_list_shifts``)."""
    built_cutoff = getattr(data, "_neighbor_list_cutoff", None)
    needs_filter = built_cutoff is not None and (built_cutoff - model_cutoff) > 1e-6
    positions = data.positions
    cell = getattr(data, "cell", None)
    batch_idx = getattr(data, "batch_idx", None)
    has_matrix = getattr(data, "neighbor_matrix", None) is not None
    has_list = getattr(data, "neighbor_list", None) is not None

    def matrix_inputs():
        nm, nn, ns = data.neighbor_matrix, data.num_neighbors, getattr(data, "neighbor_matrix_shifts", None)
        if needs_filter:
            nm, nn, ns = filter_neighbor_matrix(positions=positions, cutoff=model_cutoff, neighbor_matrix=nm,
                                                num_neighbors=nn, fill_value=fill_value, cell=cell,
                                                neighbor_matrix_shifts=ns, batch_idx=batch_idx)
        return nm, nn, ns

    if target_format == NeighborListFormat.MATRIX:
        if not has_matrix:
            raise RuntimeError("prepare_neighbors_for_model: target format is MATRIX but the batch has no "
                               "'neighbor_matrix'.  Ensure a NeighborListHook with format=MATRIX is registered.")
        nm, nn, ns = matrix_inputs()
        out = {"neighbor_matrix": nm, "num_neighbors": nn}
        if ns is not None:
            out["neighbor_matrix_shifts"] = ns
        return out
    if has_matrix:
        nm, nn, ns = matrix_inputs()
        nl, ptr, shifts = neighbor_matrix_to_list(neighbor_matrix=nm, num_neighbors=nn, fill_value=fill_value,
                                                  neighbor_matrix_shifts=ns)
        out = {"neighbor_list": nl, "edge_ptr": ptr}
        if shifts is not None:
            out["neighbor_list_shifts"] = shifts
        return out
    if has_list:
        nl, ptr, us = data.neighbor_list, data.edge_ptr, getattr(data, "neighbor_list_shifts", None)
        if needs_filter:
            nl, ptr, us = filter_neighbor_list(positions=positions, cutoff=model_cutoff, neighbor_list=nl,
                                               neighbor_ptr=ptr, cell=cell, neighbor_list_shifts=us,
                                               batch_idx=batch_idx)
        out = {"neighbor_list": nl, "edge_ptr": ptr}
        if us is not None:
            out["neighbor_list_shifts"] = us
        return out
    raise RuntimeError("prepare_neighbors_for_model: batch has neither 'neighbor_matrix' nor 'neighbor_list'.  "
                       "Ensure a NeighborListHook is registered before calling the model.")
