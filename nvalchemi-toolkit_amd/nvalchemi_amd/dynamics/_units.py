"""Time units (mirror of nvalchemi/dynamics/_units.py:22-27): with positions in Angstrom,
energies in eV and masses in amu, one internal time unit is 10.180505710759414 fs."""

from __future__ import annotations

import torch

FS_PER_INTERNAL_TIME: float = 10.180505710759414


def fs_to_internal_time(value: float | torch.Tensor) -> float | torch.Tensor:
    return value / FS_PER_INTERNAL_TIME


def per_fs_to_internal_rate(value: float | torch.Tensor) -> float | torch.Tensor:
    return value * FS_PER_INTERNAL_TIME
