"""Context objects handed to hooks (mirror of nvalchemi/hooks/_context.py:32-80)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


@dataclass(kw_only=True)
class HookContext:
    batch: Any
    model: Any = None
    global_rank: int = 0
    workflow: Any = None


@dataclass(kw_only=True)
class DynamicsContext(HookContext):
    step_count: int = 0
    converged_mask: torch.Tensor | None = None
