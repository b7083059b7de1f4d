"""``ConvergenceHook`` status migration and ``FusedStage`` on the host, over a Torch model: the
reference's own cases (test/dynamics/test_single_loop.py:158-860, 1410-1730) restated.  The stages
here move nothing (``BaseDynamics`` itself, or a subclass that records the masks it is given), so no
kernel is needed: what is checked is the control flow -- which systems each sub-stage gets, one model
evaluation per step, how converged systems migrate, when a run stops, which hooks fire.
"""

from collections import OrderedDict

import pytest
import torch

from nvalchemi_amd.data import AtomicData, Batch
from nvalchemi_amd.dynamics import BaseDynamics, ConvergenceHook, DynamicsStage, FusedStage
from nvalchemi_amd.hooks._context import DynamicsContext
from nvalchemi_amd.models import BaseModelMixin, ModelConfig


class ConstantForces(torch.nn.Module, BaseModelMixin):
    """Forces of modest size that do not depend on anything; counts its evaluations."""

    def __init__(self):
        super().__init__()
        self.model_config = ModelConfig(outputs=frozenset({"energy", "forces"}))
        self.forward_count = 0

    def forward(self, batch):
        self.forward_count += 1
        return OrderedDict(energy=torch.zeros(batch.num_graphs, 1), forces=torch.full((batch.num_nodes, 3), 0.5))


class Tracking(BaseDynamics):
    def __init__(self, model, **kw):
        super().__init__(model=model, **kw)
        self.updated_masks = []

    def _masked_pre_update(self, batch, mask):
        self.updated_masks.append(mask.clone())


def status_batch(n, status=None):
    data = [AtomicData(torch.randn(1, 3), torch.tensor([6])) for _ in range(n)]
    b = Batch.from_data_list(data)
    b["forces"] = torch.zeros(n, 3)
    b["energy"] = torch.zeros(n, 1)
    b["status"] = torch.zeros(n, 1, dtype=torch.long) if status is None else torch.as_tensor(status)
    return b


def migrate(batch, **kw):
    hook = ConvergenceHook.from_fmax(kw.pop("threshold", 0.05), source_status=0, target_status=1)
    hook(DynamicsContext(batch=batch, step_count=0), DynamicsStage.AFTER_STEP)
    return batch.status.view(-1).tolist()


def test_convergence_hook_moves_converged_systems_of_its_source_status_only():
    hook = ConvergenceHook()
    assert hook.frequency == 1 and hook.stage == DynamicsStage.AFTER_STEP and len(hook.criteria) == 1
    c = hook.criteria[0]
    assert (c.key, c.threshold, c.reduce_op) == ("forces", 0.05, "norm")
    assert hook.source_status is None and hook.target_status is None

    small = torch.tensor([[0.01, 0, 0], [0.02, 0, 0], [0.03, 0, 0]])
    b = status_batch(3, [0, 0, 0]); b.forces = small
    assert migrate(b) == [1, 1, 1]
    b = status_batch(3, [2, 2, 2]); b.forces = small
    assert migrate(b) == [2, 2, 2]
    b = status_batch(3, [0, 0, 0]); b.forces = torch.tensor([[0.1, 0, 0], [0.2, 0, 0], [0.3, 0, 0]])
    assert migrate(b) == [0, 0, 0]
    b = status_batch(4, [0, 2, 0, 2]); b.forces = torch.tensor([[0.01, 0, 0], [0.01, 0, 0], [0.1, 0, 0], [0.1, 0, 0]])
    assert migrate(b) == [1, 2, 0, 2]
    b = status_batch(3, [0, 0, 0]); b.forces = torch.tensor([[0.01, 0, 0], [0.05, 0, 0], [0.1, 0, 0]])
    assert migrate(b, threshold=0.2) == [1, 1, 1]
    # (B,) and (B, 1) status tensors alike, updated in place
    b = status_batch(3, [[0], [0], [0]]); b.forces = small
    before = b.status
    assert migrate(b) == [1, 1, 1] and before.view(-1).tolist() == [1, 1, 1]
    # without forces: a KeyError that names them; without a status: nothing to do
    b = status_batch(3)
    del b["forces"]
    with pytest.raises(KeyError, match="forces"):
        ConvergenceHook()(DynamicsContext(batch=b, step_count=0), DynamicsStage.AFTER_STEP)
    b = status_batch(3); b.forces = small
    del b["status"]
    ConvergenceHook()(DynamicsContext(batch=b, step_count=0), DynamicsStage.AFTER_STEP)


def test_fusing_stages_assigns_codes_and_checks_its_operands():
    m = ConstantForces()
    fused = BaseDynamics(model=m) + BaseDynamics(model=m)
    assert isinstance(fused, FusedStage) and [c for c, _ in fused.sub_stages] == [0, 1] and fused.exit_status == 2
    three = Tracking(m) + Tracking(m) + Tracking(m)
    assert [c for c, _ in three.sub_stages] == [0, 1, 2] and three.exit_status == 3
    grown = FusedStage(sub_stages=[(0, BaseDynamics(model=m))]) + BaseDynamics(model=m)
    assert [c for c, _ in grown.sub_stages] == [0, 1]
    assert FusedStage(sub_stages=[(0, BaseDynamics(model=m))], n_steps=100).n_steps == 100
    with pytest.raises(TypeError, match=r"Both operands of \+ must be BaseDynamics"):
        BaseDynamics(model=m) + object()
    with pytest.raises(TypeError, match="other must be a BaseDynamics instance"):
        FusedStage(sub_stages=[(0, BaseDynamics(model=m))]) + object()
    assert FusedStage.all_complete(status_batch(3, [2, 2, 2]), exit_status=2) is True
    assert FusedStage.all_complete(status_batch(3, [2, 1, 2]), exit_status=2) is False


def test_one_evaluation_per_step_and_every_sub_stage_gets_its_own_systems():
    m = ConstantForces()
    d0, d1 = Tracking(m), Tracking(m)
    fused = FusedStage(sub_stages=[(0, d0), (1, d1)])
    b = status_batch(4, [0, 1, 0, 1])
    fused.step(b)
    assert m.forward_count == 1 and fused.step_count == 1
    assert [x.tolist() for x in d0.updated_masks] == [[True, False, True, False]]
    assert [x.tolist() for x in d1.updated_masks] == [[False, True, False, True]]
    # a sub-stage without systems is skipped
    d0, d1 = Tracking(m), Tracking(m)
    FusedStage(sub_stages=[(0, d0), (1, d1)]).step(status_batch(3, [1, 1, 1]))
    assert d0.updated_masks == [] and len(d1.updated_masks) == 1


def test_converged_systems_move_to_the_next_stage_and_runs_stop_when_all_have_left():
    m = ConstantForces()
    loose = lambda: ConvergenceHook.from_fmax(1e6)  # noqa: E731  (everything counts as converged)
    fused = FusedStage(sub_stages=[(0, BaseDynamics(model=m, convergence_hook=loose())), (1, BaseDynamics(model=m))])
    b = status_batch(3)
    fused.step(b)
    assert b.status.view(-1).tolist() == [1, 1, 1]
    # a single stage moves them to the exit code; without a criterion it registers nothing
    single = FusedStage(sub_stages=[(0, BaseDynamics(model=m, convergence_hook=loose()))])
    b = status_batch(3)
    single.step(b)
    assert b.status.view(-1).tolist() == [single.exit_status] * 3
    plain = BaseDynamics(model=m)
    n_before = len([h for h in plain.hooks if isinstance(h, ConvergenceHook) and h.source_status is not None])
    FusedStage(sub_stages=[(0, plain)])
    assert len([h for h in plain.hooks if isinstance(h, ConvergenceHook) and h.source_status is not None]) == n_before
    # the hooks of successive stages fire one after the other: 0 -> 1 -> 2 within one step
    chain = FusedStage(sub_stages=[(0, BaseDynamics(model=m, convergence_hook=loose())),
                                   (1, BaseDynamics(model=m, convergence_hook=loose())), (2, BaseDynamics(model=m))])
    b = status_batch(3)
    chain.step(b)
    assert b.status.view(-1).tolist() == [2, 2, 2]
    # run: one evaluation before the loop, one per step; it ends when every system has the exit code,
    # whatever n_steps says
    m2 = ConstantForces()
    dyn = BaseDynamics(model=m2)
    dyn.register_hook(ConvergenceHook.from_fmax(1e6, source_status=0, target_status=1))
    fused = FusedStage(sub_stages=[(0, dyn)], n_steps=10000)
    fused.run(status_batch(3))
    assert fused.step_count == 1 and m2.forward_count == 2


def test_step_budget_and_criterion_both_graduate_and_are_reported_together():
    m = ConstantForces()
    dyn = BaseDynamics(model=m, n_steps=2, convergence_hook=ConvergenceHook(criteria={"key": "energy_change",
                                                                                     "threshold": 0.5}))
    fused = FusedStage(sub_stages=[(0, dyn)])
    b = status_batch(2, [0, 0])
    b.energy_change = torch.ones(2)
    b, left = fused.step(b)
    assert left is None
    b.energy_change = torch.tensor([1.0, 0.0])  # system 1 meets the criterion, system 0 runs out of steps
    b, left = fused.step(b)
    assert b.status.view(-1).tolist() == [fused.exit_status] * 2 and left.tolist() == [0, 1]
    assert b.n_steps_counter_0.view(-1).tolist() == [0, 1]


class Tracker:
    def __init__(self, stage, frequency=1):
        self.stage, self.frequency, self.calls = stage, frequency, []

    def __call__(self, ctx, stage):
        self.calls.append((stage, ctx.step_count))


def test_hooks_of_the_sub_stages_fire_at_their_stages():
    m = ConstantForces()
    stages = (DynamicsStage.BEFORE_STEP, DynamicsStage.BEFORE_PRE_UPDATE, DynamicsStage.AFTER_COMPUTE,
              DynamicsStage.AFTER_POST_UPDATE, DynamicsStage.AFTER_STEP, DynamicsStage.ON_CONVERGE)
    d0, d1 = BaseDynamics(model=m), BaseDynamics(model=m, convergence_hook=ConvergenceHook.from_fmax(1e6))
    hooks0 = {s: Tracker(s) for s in stages}
    hooks1 = {s: Tracker(s) for s in stages}
    for s in stages:
        d0.register_hook(hooks0[s])
        d1.register_hook(hooks1[s])
    every_other = Tracker(DynamicsStage.AFTER_STEP, frequency=2)
    d0.register_hook(every_other)
    fused = FusedStage(sub_stages=[(0, d0), (1, d1)])
    b = status_batch(3, [1, 1, 1])  # nothing for stage 0 to do: its hooks fire all the same
    for _ in range(4):
        fused.step(b)
        b["status"] = torch.ones(3, 1, dtype=torch.long)
    for s in stages[:5]:
        assert len(hooks0[s].calls) == 4 and len(hooks1[s].calls) == 4, s
    assert [c[1] for c in hooks0[DynamicsStage.AFTER_STEP].calls] == [0, 1, 2, 3]
    assert d0.step_count == 4 and d1.step_count == 4 and fused.step_count == 4
    assert [c[1] for c in every_other.calls] == [0, 2]
    # only the stage whose systems converged announces it
    assert len(hooks1[DynamicsStage.ON_CONVERGE].calls) == 4 and hooks0[DynamicsStage.ON_CONVERGE].calls == []


def test_device_type_and_the_stream_context_on_the_host():
    """``device_type`` follows what is available unless given; a fused stage wants one device type;
    without a GPU the stream context does nothing (test/dynamics/test_single_loop.py:863-1228)."""
    m = ConstantForces()
    auto = BaseDynamics(model=m)
    assert auto.device_type == ("cuda" if torch.cuda.is_available() else "cpu")
    a, b, c = (BaseDynamics(model=m, device_type=t) for t in ("cpu", "cpu", "cuda"))
    assert FusedStage(sub_stages=[(0, a), (1, b)]).device_type == "cpu"
    with pytest.raises(ValueError, match="must share the same device_type"):
        FusedStage(sub_stages=[(0, a), (1, c)])
    with pytest.raises(ValueError, match="device_type"):
        a + c
    fused = FusedStage(sub_stages=[(0, a), (1, b)])
    assert fused.stream is None
    with fused as entered:
        assert entered is fused and fused.stream is None and a.stream is None
        fused.step(status_batch(2, [0, 1]))
    assert fused.stream is None and fused._stream_ctx is None
