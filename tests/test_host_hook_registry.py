"""The hook registry shared by the engines (nvalchemi/hooks/_registry.py:26-177, _context.py:60-139):
the reference's own cases (test/hooks/test_registry.py:48-330, test_context.py:24-95) restated."""

from enum import Enum
from unittest.mock import MagicMock

import pytest

from nvalchemi_amd.hooks._context import DynamicsContext, HookContext
from nvalchemi_amd.hooks._registry import HookRegistryMixin


class StageA(Enum):
    A = 0
    B = 1


class StageX(Enum):
    X = 0


class Engine(HookRegistryMixin):
    def __init__(self):
        self.step_count = 0
        self._init_hooks()


class TypedEngine(HookRegistryMixin):
    _stage_type = StageA

    def __init__(self):
        self.step_count = 0
        self._init_hooks()


def hook(stage, frequency=1, log=None, runs_on=None):
    class H:
        def __call__(self, ctx, st):
            if log is not None:
                log.append((ctx, st))

    h = H()
    h.frequency, h.stage = frequency, stage
    if runs_on is not None:
        h._runs_on_stage = runs_on
    return h


def test_registration_and_dispatch():
    e = Engine()
    assert e.hooks == []
    h = hook(StageA.A)
    e.register_hook(h)
    assert e.hooks == [h]
    for bad in (0, -1):
        with pytest.raises(ValueError, match="positive integer"):
            e.register_hook(hook(StageA.A, frequency=bad))
    seeded = HookRegistryMixin()
    seeded.step_count = 0
    seeded._init_hooks(hooks=[hook(StageA.A)])
    assert len(seeded.hooks) == 1

    e = Engine()
    e.step_count = 1
    log_a, log_b = [], []
    e.register_hook(hook(StageA.A, log=log_a))
    e.register_hook(hook(StageA.B, log=log_b))
    batch = MagicMock()
    e._call_hooks(StageA.A, batch)
    assert [s for _, s in log_a] == [StageA.A] and log_b == []
    ctx = log_a[0][0]
    assert isinstance(ctx, HookContext) and ctx.batch is batch
    # a hook may say for itself on which stages it runs
    e = Engine()
    many, never = [], []
    e.register_hook(hook(StageA.A, log=many, runs_on=lambda st: st in {StageA.A, StageA.B}))
    e.register_hook(hook(StageA.A, log=never, runs_on=lambda st: False))
    e._call_hooks(StageA.A, MagicMock())
    e._call_hooks(StageA.B, MagicMock())
    assert [s for _, s in many] == [StageA.A, StageA.B] and never == []
    # frequency gates on the engine's step count
    e = Engine()
    every3 = []
    e.register_hook(hook(StageA.A, frequency=3, log=every3))
    for step in range(7):
        e.step_count = step
        e._call_hooks(StageA.A, MagicMock())
    assert len(every3) == 3


def test_context_and_stage_type():
    e = Engine()
    e.step_count = 42
    batch = MagicMock()
    ctx = e._build_context(batch)
    assert isinstance(ctx, HookContext) and ctx.batch is batch and ctx.global_rank == 0 and ctx.workflow is e
    e.model = MagicMock()
    assert e._build_context(batch).model is e.model
    d = DynamicsContext(batch=batch, step_count=5)
    assert d.step_count == 5 and d.batch is batch and d.model is None and d.converged_mask is None

    t = TypedEngine()
    t.register_hook(hook(StageA.A))
    with pytest.raises(TypeError, match="only accepts StageA"):
        t.register_hook(hook(StageX.X))
    Engine().register_hook(hook(StageX.X))  # no stage type: anything goes
    t.register_hook(hook(StageX.X, runs_on=lambda st: True))  # the hook decides: no check
    assert len(t.hooks) == 2

    class Both(HookRegistryMixin):
        _stage_type = (StageA, StageX)

        def __init__(self):
            self.step_count = 0
            self._init_hooks()

    class StageZ(Enum):
        Z = 0

    b = Both()
    b.register_hook(hook(StageA.A))
    b.register_hook(hook(StageX.X))
    with pytest.raises(TypeError, match=r"only accepts StageA \| StageX"):
        b.register_hook(hook(StageZ.Z))
