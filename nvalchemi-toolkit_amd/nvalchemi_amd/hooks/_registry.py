"""Flat-list hook storage and stage/frequency-gated dispatch.

Mirror of nvalchemi/hooks/_registry.py:26-177: ``register_hook(hook, stage=)`` validates the
frequency and the stage type; ``_call_hooks(stage, batch)`` builds one context and calls
every hook whose stage matches (or whose ``_runs_on_stage`` says so) when
``step_count % hook.frequency == 0``.
"""

from __future__ import annotations

from enum import Enum
from typing import Any

from ._context import HookContext


class HookRegistryMixin:
    hooks: list
    step_count: int
    _stage_type: Any = None

    def _init_hooks(self, hooks: list | None = None) -> None:
        self.hooks = []
        if hooks:
            for hook in hooks:
                self.register_hook(hook)

    def register_hook(self, hook: Any, stage: Enum | None = None) -> None:
        if not isinstance(hook.frequency, int) or hook.frequency < 1:
            raise ValueError(f"Hook frequency must be a positive integer, got {hook.frequency}")
        if stage is not None:
            hook.stage = stage
        stage_type = self._stage_type
        has_custom_dispatch = getattr(hook, "_runs_on_stage", None) is not None
        if getattr(hook, "stage", None) is None and not has_custom_dispatch:
            raise TypeError(f"Hook {type(hook).__name__} has no stage assigned. "
                            "Pass stage= to the hook constructor or to register_hook().")
        if (stage_type is not None and not has_custom_dispatch and hook.stage is not None
                and not isinstance(hook.stage, stage_type)):
            expected = stage_type.__name__ if isinstance(stage_type, type) else " | ".join(t.__name__ for t in stage_type)
            raise TypeError(f"Hook {hook!r} has stage={hook.stage!r} (type {type(hook.stage).__name__}), "
                            f"but this engine only accepts {expected} stages.")
        on_register = getattr(hook, "on_register", None)
        if on_register is not None:
            if not callable(on_register):
                raise TypeError(f"Hook {type(hook).__name__}.on_register must be callable.")
            on_register(self)
        self.hooks.append(hook)

    def _build_context(self, batch: Any) -> HookContext:
        return HookContext(batch=batch, model=getattr(self, "model", None), workflow=self)

    def _call_hooks(self, stage: Enum, batch: Any) -> None:
        if not self.hooks:
            return
        ctx = None
        for hook in self.hooks:
            runs_on_stage = getattr(hook, "_runs_on_stage", None)
            if runs_on_stage is not None:
                if not runs_on_stage(stage):
                    continue
            elif stage != hook.stage:
                continue
            if self.step_count % hook.frequency == 0:
                if ctx is None:
                    ctx = self._build_context(batch)
                hook(ctx, stage)
