"""Per-system integrator state helpers (mirror of nvalchemi/dynamics/_ops/_bridge.py:32-102)."""

from __future__ import annotations

import torch

from ...data.batch import Batch, UniformGroup


def _make_state_batch(system_data: dict[str, torch.Tensor], device: torch.device) -> Batch:
    """A system-only ``Batch`` holding ``[M, ...]`` tensors, readable as attributes."""
    m = next(iter(system_data.values())).shape[0] if system_data else 0
    return Batch._construct(device, {"system": UniformGroup(system_data, m, device)})


def _to_per_system(val: float | torch.Tensor, M: int, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    """Broadcast a scalar, ``[]``, ``[1, ...]`` or ``[M, ...]`` value to a contiguous ``[M, ...]``."""
    if isinstance(val, torch.Tensor):
        tensor = val.to(device=device, dtype=dtype)
        if tensor.ndim == 0:
            return tensor.expand(M).contiguous()
        leading = tensor.shape[0]
        if leading not in (1, M):
            raise ValueError(f"Expected leading dimension 1 or {M} for per-system broadcast, "
                             f"got shape {tuple(tensor.shape)}.")
        return tensor.expand((M, *tensor.shape[1:])).contiguous()
    return torch.full((M,), float(val), dtype=dtype, device=device)
