"""Time units of the integrators.

Positions are in Angstrom, energies in eV, masses in amu, so velocities are in sqrt(eV/amu) and the
kernels' unit of time is Angstrom * sqrt(amu/eV):

    sqrt(1.66053906660e-27 kg / 1.602176634e-19 J) * 1e-10 m = 1.0180505710759414e-14 s

i.e. 10.180505710759414 fs.  The public classes take femtoseconds (and rates in 1/fs) and convert
once, when their per-system state is made.  Names as in nvalchemi/dynamics/_units.py:22-36.
"""

from __future__ import annotations

from typing import TypeVar

import torch

Number = TypeVar("Number", float, torch.Tensor)

#: femtoseconds in one unit of kernel time
FS_PER_INTERNAL_TIME: float = 10.180505710759414


def fs_to_internal_time(value: Number) -> Number:
    """A time in femtoseconds, in kernel time."""
    return value / FS_PER_INTERNAL_TIME


def internal_time_to_fs(value: Number) -> Number:
    """A kernel time, in femtoseconds."""
    return value * FS_PER_INTERNAL_TIME


def per_fs_to_internal_rate(value: Number) -> Number:
    """A rate in 1/fs (a friction, a collision frequency), per unit of kernel time."""
    return value * FS_PER_INTERNAL_TIME
