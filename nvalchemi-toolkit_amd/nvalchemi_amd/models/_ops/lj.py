"""Torch custom ops for the Lennard-Jones pair kernel.

Same schemas (argument order, mutation sets, returns) as
``nvalchemi::lj_energy_forces_batch`` and ``nvalchemi::lj_energy_forces_virial_batch``
(nvalchemi/models/_ops/lj.py:116-130,246-260), registered under the ``nvalchemi_amd``
namespace with fake implementations so ``torch.compile`` can treat them as opaque.  Neither
registers autograd: forces and virials are analytic.

``lj_energy_forces_system_batch`` is the fused form this package's model wrapper uses: one
launch also returns the per-system energies (fp64 accumulation of the float32 atomic
energies, nvalchemi/models/lj.py:467-477) and, on request, the per-system virial, so no
``(N,)`` upcast, scatter or per-atom virial detour runs afterwards.

Sign convention: ``W = -dE/d(strain) = -sum r_ij (x) F_ij``; the wrapper turns it into the
tensile-positive Cauchy stress ``sigma = -W / V``.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ... import _lib


def _check_dtype(positions: Tensor) -> None:
    """float32 (the tuned kernel; pair math is double internally) or float64 (a plain kernel: shifts
    always read, no staging, no walk order), as the reference's ops take both."""
    if positions.dtype not in (torch.float32, torch.float64):
        raise TypeError(f"Lennard-Jones positions must be float32 or float64, got {positions.dtype}")


def _shifts_or_none(neighbor_matrix_shifts: Tensor | None) -> Tensor | None:
    if neighbor_matrix_shifts is None or neighbor_matrix_shifts.numel() == 0:
        return None
    return neighbor_matrix_shifts.contiguous()


@torch.library.custom_op("nvalchemi_amd::lj_energy_forces_batch", mutates_args=())
def lj_energy_forces_batch(positions: Tensor, cells: Tensor, neighbor_matrix: Tensor,
                           neighbor_matrix_shifts: Tensor, num_neighbors: Tensor, batch_idx: Tensor,
                           fill_value: int, epsilon: float, sigma: float, cutoff: float,
                           switch_width: float, half_list: bool) -> tuple[Tensor, Tensor]:
    """Per-atom LJ energies ``(N)`` and forces ``(N,3)`` for a batch of systems."""
    _check_dtype(positions)
    N = positions.shape[0]
    e = torch.empty(N, dtype=positions.dtype, device=positions.device)
    f = torch.empty(N, 3, dtype=positions.dtype, device=positions.device)
    _lib.lj_energy_forces(positions.contiguous(), cells.to(positions.dtype).contiguous(), neighbor_matrix.contiguous(),
                          neighbor_matrix_shifts.contiguous(), num_neighbors.contiguous(),
                          batch_idx.contiguous(), fill_value, epsilon, sigma, cutoff, switch_width,
                          half_list, e, f)
    return e, f


@lj_energy_forces_batch.register_fake
def _(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx, fill_value,
      epsilon, sigma, cutoff, switch_width, half_list):
    N = positions.shape[0]
    return (torch.empty(N, dtype=positions.dtype, device=positions.device),
            torch.empty(N, 3, dtype=positions.dtype, device=positions.device))


@torch.library.custom_op("nvalchemi_amd::lj_energy_forces_virial_batch", mutates_args=())
def lj_energy_forces_virial_batch(positions: Tensor, cells: Tensor, neighbor_matrix: Tensor,
                                  neighbor_matrix_shifts: Tensor, num_neighbors: Tensor,
                                  batch_idx: Tensor, fill_value: int, epsilon: float, sigma: float,
                                  cutoff: float, switch_width: float,
                                  half_list: bool) -> tuple[Tensor, Tensor, Tensor]:
    """As above plus virials ``(B,9)`` row-major, ``B = cells.shape[0]``."""
    _check_dtype(positions)
    N = positions.shape[0]
    B = cells.shape[0]
    e = torch.empty(N, dtype=positions.dtype, device=positions.device)
    f = torch.empty(N, 3, dtype=positions.dtype, device=positions.device)
    w = torch.empty(B, 9, dtype=positions.dtype, device=positions.device)
    _lib.lj_energy_forces(positions.contiguous(), cells.to(positions.dtype).contiguous(), neighbor_matrix.contiguous(),
                          neighbor_matrix_shifts.contiguous(), num_neighbors.contiguous(),
                          batch_idx.contiguous(), fill_value, epsilon, sigma, cutoff, switch_width,
                          half_list, e, f, virials=w)
    return e, f, w


@lj_energy_forces_virial_batch.register_fake
def _(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors, batch_idx, fill_value,
      epsilon, sigma, cutoff, switch_width, half_list):
    N = positions.shape[0]
    B = cells.shape[0]
    return (torch.empty(N, dtype=positions.dtype, device=positions.device),
            torch.empty(N, 3, dtype=positions.dtype, device=positions.device),
            torch.empty(B, 9, dtype=positions.dtype, device=positions.device))


def lj_energy_forces_system_batch(positions: Tensor, cells: Tensor, neighbor_matrix: Tensor,
                                  neighbor_matrix_shifts: Tensor | None, num_neighbors: Tensor,
                                  batch_idx: Tensor, fill_value: int, epsilon: float, sigma: float,
                                  cutoff: float, switch_width: float, half_list: bool,
                                  compute_virial: bool = False, out: dict | None = None,
                                  row_order: Tensor | None = None, neighbor_list_cutoff: float = 0.0,
                                  pair_tiles: tuple | None = None):
    """Fused launch: ``(atomic_energies (N), forces (N,3), system_energies (B), virials (B,9) |
    None)``.  ``neighbor_matrix_shifts=None`` means all shifts are zero (no ``(N,K,3)`` zeros
    tensor is needed).  ``out`` may carry preallocated result tensors under those names.
    ``row_order`` (a permutation of the atoms that keeps every system together, e.g. the cell
    order of the neighbor build) only changes the order in which rows are worked on.
    ``neighbor_list_cutoff`` (the radius the matrix was searched with, 0.0 if unknown) lets the
    kernel derive shifts from positions, instead of reading them, in systems whose cell is wider
    than twice that radius in every direction; the results are the same.  ``pair_tiles`` (what the
    neighbor hook leaves for systems too large to stage: the positions in ``row_order``, the tiles of the search
    and each pair's place in its tile) changes where neighbor positions are read from, nothing else."""
    _check_dtype(positions)
    N = positions.shape[0]
    B = cells.shape[0]
    dev, dt = positions.device, positions.dtype
    out = out or {}
    e = out.get("atomic_energies")
    if e is None:
        e = torch.empty(N, dtype=dt, device=dev)
    f = out.get("forces")
    if f is None:
        f = torch.empty(N, 3, dtype=dt, device=dev)
    es = out.get("system_energies")
    if es is None:
        es = torch.empty(B, dtype=dt, device=dev)
    w = None
    if compute_virial:
        w = out.get("virials")
        if w is None:
            w = torch.empty(B, 9, dtype=dt, device=dev)
    _lib.lj_energy_forces(positions, cells.to(dt), neighbor_matrix, _shifts_or_none(neighbor_matrix_shifts),
                          num_neighbors, batch_idx, fill_value, epsilon, sigma, cutoff, switch_width,
                          half_list, e, f, virials=w, system_energies=es, row_order=row_order,
                          neighbor_list_cutoff=neighbor_list_cutoff, pair_tiles=None if half_list else pair_tiles)
    return e, f, es, w
