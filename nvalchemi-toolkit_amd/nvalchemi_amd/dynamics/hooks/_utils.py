"""Per-system observables computed on the device: segmented reductions of per-atom values,
kinetic energy and temperature per system.

Mirror of nvalchemi/dynamics/hooks/_utils.py:45-290 (``scatter_reduce_per_graph``,
``kinetic_energy_per_graph``, ``temperature_per_graph``, ``KB_EV``) with the same signatures and
return shapes; the Warp launches behind the reference's custom ops are replaced by
``nvamd_segment_reduce`` / ``nvamd_kinetic_energy``.  float32 only; ``batch_idx`` must be sorted
(as batching guarantees).  Sums are accumulated in float64 and rounded once.
"""

from __future__ import annotations

from typing import Literal

import torch

from ... import _lib

__all__ = ["KB_EV", "ScatterReduce", "scatter_reduce_per_graph", "kinetic_energy_per_graph",
           "temperature_per_graph"]

#: Boltzmann constant in eV/K (NIST 2018 CODATA value).
KB_EV: float = 8.617333262e-5

ScatterReduce = Literal["amax", "sum", "amin", "mean"]


def _f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.float32:
        raise TypeError(f"{what}: float32 only, got {t.dtype}")
    return t.contiguous()


@torch.library.custom_op("nvalchemi_amd::segmented_reduce", mutates_args=())
def _segmented_reduce(values: torch.Tensor, idx: torch.Tensor, num_segments: int, reduce: str) -> torch.Tensor:
    out = torch.empty(num_segments, device=values.device, dtype=values.dtype)
    _lib.segment_reduce(_f32(values, "values"), idx.to(torch.int32).contiguous(), out, reduce)
    return out


@_segmented_reduce.register_fake
def _(values, idx, num_segments, reduce):
    return torch.empty(num_segments, device=values.device, dtype=values.dtype)


@torch.library.custom_op("nvalchemi_amd::compute_kinetic_energy", mutates_args=())
def _compute_ke(velocities: torch.Tensor, masses: torch.Tensor, batch_idx: torch.Tensor,
                num_graphs: int) -> torch.Tensor:
    ke = torch.empty(num_graphs, device=velocities.device, dtype=velocities.dtype)
    _lib.kinetic_energy(_f32(velocities, "velocities"), _f32(masses, "masses"),
                        batch_idx.to(torch.int32).contiguous(), ke)
    return ke


@_compute_ke.register_fake
def _(velocities, masses, batch_idx, num_graphs):
    return torch.empty(num_graphs, device=velocities.device, dtype=velocities.dtype)


def scatter_reduce_per_graph(values: torch.Tensor, batch_idx: torch.Tensor, num_graphs: int,
                             reduce: ScatterReduce = "amax") -> torch.Tensor:
    """Reduce a 1-D per-atom tensor ``(V,)`` to ``(B,)`` per system with ``amax`` / ``sum`` /
    ``amin`` / ``mean`` (anything else means ``mean``, as in the reference's dispatch)."""
    if reduce not in ("sum", "amax", "amin"):
        reduce = "mean"
    return _segmented_reduce(values, batch_idx, num_graphs, reduce)


def kinetic_energy_per_graph(velocities: torch.Tensor, masses: torch.Tensor, batch_idx: torch.Tensor,
                             num_graphs: int) -> torch.Tensor:
    """``0.5 * sum(m_i |v_i|^2)`` per system, shape ``(B, 1)``; masses ``(V,)`` or ``(V, 1)``."""
    m = masses.squeeze(-1) if masses.dim() > 1 else masses
    return _compute_ke(velocities, m, batch_idx, num_graphs).unsqueeze(-1)


def temperature_per_graph(velocities: torch.Tensor, masses: torch.Tensor, batch_idx: torch.Tensor,
                          num_graphs: int, atoms_per_graph: torch.Tensor,
                          conversion_factor: float = KB_EV) -> torch.Tensor:
    """Instantaneous kinetic temperature per system, ``T = 2 KE / (3 N k_B)`` with 3N degrees of
    freedom (no constraint correction), shape ``(B,)``."""
    ke = kinetic_energy_per_graph(velocities, masses, batch_idx, num_graphs).squeeze(-1)
    return (2.0 * ke) / (3.0 * atoms_per_graph.float() * conversion_factor)
