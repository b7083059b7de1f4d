"""In-flight batching on the host: ``refill_check`` and the sampler-driven ``FusedStage.run``
(nvalchemi/dynamics/base.py:1957-2083, 3162-3265) with the size-aware sampler and the host sink.

The cases restate the reference's own (test/dynamics/test_inflight.py:169-960) over a Torch model on
the CPU: selection, growth and bookkeeping are tensor bookkeeping and need no kernel.
"""

from collections import OrderedDict

import pytest
import torch

from nvalchemi_amd.data import AtomicData, Batch
from nvalchemi_amd.dynamics import BaseDynamics, ConvergenceHook, FusedStage, HostMemory, SizeAwareSampler
from nvalchemi_amd.models import BaseModelMixin, ModelConfig


class WellModel(torch.nn.Module, BaseModelMixin):
    """Harmonic well: forces = -positions."""

    def __init__(self):
        super().__init__()
        self.model_config = ModelConfig(outputs=frozenset({"energy", "forces"}))

    def forward(self, batch):
        e = torch.zeros(batch.num_graphs, dtype=batch.positions.dtype)
        e.index_add_(0, batch.batch_idx.long(), 0.5 * (batch.positions ** 2).sum(-1))
        return OrderedDict(energy=e.unsqueeze(-1), forces=-batch.positions.clone())


class Relax(BaseDynamics):
    """Steepest descent with a fixed step: positions move a tenth of the way down the forces."""

    __needs_keys__ = {"forces"}
    __provides_keys__ = {"positions"}

    def pre_update(self, batch):
        batch.positions.add_(0.1 * batch.forces)

    def post_update(self, batch):
        pass


class Dataset:
    def __init__(self, samples, scale=1.0, status=None):
        self.samples, self.scale, self.status = samples, scale, status

    def __len__(self):
        return len(self.samples)

    def get_metadata(self, k):
        return self.samples[k]

    def __getitem__(self, k):
        n, _ = self.samples[k]
        g = torch.Generator().manual_seed(k)
        d = AtomicData(self.scale * (1 + k) * torch.randn(n, 3, generator=g), torch.arange(1, n + 1),
                       forces=torch.zeros(n, 3), energy=torch.zeros(1, 1))
        if self.status is not None:
            d.add_system_property("status", torch.tensor([[self.status]], dtype=torch.long))
        return d, {}


def flat(t):
    return t.view(-1).tolist()


def test_refill_replaces_what_graduated_and_keeps_the_rest_in_order():
    model = WellModel()
    sampler = SizeAwareSampler(Dataset([(2, 0)] * 10), max_atoms=20, max_edges=10, max_batch_size=5)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    assert batch.num_graphs == 5 and flat(batch.system_id) == [0, 1, 2, 3, 4]
    kept_pos = batch.positions[[0, 1, 4, 5, 8, 9]].clone()
    batch["status"] = torch.tensor([[0], [1], [0], [1], [0]])
    result = dyn.refill_check(batch, exit_status=1)
    assert result is not batch and result.num_graphs == 5 and "status" in result
    assert flat(result.status) == [0] * 5 and flat(result.system_id) == [0, 2, 4, 5, 6]
    assert torch.equal(result.positions[:6], kept_pos) and result.num_nodes == 10 and len(sampler) == 3
    # nothing graduated: the very same batch comes back
    assert dyn.refill_check(result, exit_status=1) is result
    # everything graduated: all five slots refilled, three replacements left
    result["status"] = torch.ones(5, 1, dtype=torch.long)
    again = dyn.refill_check(result, exit_status=1)
    assert again.num_graphs == 3 and flat(again.system_id) == [7, 8, 9] and flat(again.status) == [0, 0, 0]
    assert sampler.exhausted and not dyn.done
    # the last ones leave: nothing is left, the run is over
    again["status"] = torch.ones(3, 1, dtype=torch.long)
    assert dyn.refill_check(again, exit_status=1) is None and dyn.done is True
    with pytest.raises(RuntimeError, match="requires a sampler"):
        BaseDynamics(model=model).refill_check(batch, exit_status=1)


def test_refill_keeps_system_ids_and_statuses_with_their_systems():
    model = WellModel()
    # a count limit of atoms: three single-atom systems in flight
    sampler = SizeAwareSampler(Dataset([(1, 0)] * 5), max_atoms=3)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    assert flat(batch.system_id) == [0, 1, 2]
    batch["status"] = torch.tensor([[0], [1], [2]])
    result = dyn.refill_check(batch, exit_status=2)
    assert flat(result.system_id) == [0, 1, 3] and flat(result.status) == [0, 1, 0]
    result["status"] = torch.tensor([[2], [1], [2]])
    result = dyn.refill_check(result, exit_status=2)
    assert flat(result.system_id) == [1, 4] and flat(result.status) == [1, 0]

    sampler = SizeAwareSampler(Dataset([(1, 0)] * 3), max_atoms=2)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    batch["status"] = torch.tensor([[1], [1]])
    result = dyn.refill_check(batch, exit_status=1)
    assert flat(result.system_id) == [2] and flat(result.status) == [0]

    # a status that the dataset gives its samples arrives with them
    sampler = SizeAwareSampler(Dataset([(1, 0)] * 5, status=1), max_atoms=3)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    assert flat(batch.status) == [0, 0, 0]  # the first batch starts at zero whatever the dataset says
    batch["status"] = torch.tensor([[0], [2], [1]])
    result = dyn.refill_check(batch, exit_status=2)
    assert flat(result.system_id) == [0, 2, 3] and flat(result.status) == [0, 1, 1]

    # fewer replacements than places: the batch shrinks
    sampler = SizeAwareSampler(Dataset([(2, 0)] * 6), max_atoms=20, max_edges=10, max_batch_size=5)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    assert len(sampler) == 1
    batch["status"] = torch.tensor([[1], [1], [1], [0], [0]])
    result = dyn.refill_check(batch, exit_status=1)
    assert result.num_graphs == 3 and flat(result.system_id) == [3, 4, 5] and flat(result.status) == [0, 0, 0]

    # the atom budget decides what can come in: 6 atoms in flight at most
    sampler = SizeAwareSampler(Dataset([(3, 0), (3, 0), (4, 0), (2, 0), (1, 0)]), max_atoms=6)
    dyn = BaseDynamics(model=model, sampler=sampler)
    batch = sampler.build_initial_batch()
    assert batch.num_nodes_list == [1, 2, 3]  # one per bin, smallest bins first
    batch["status"] = torch.tensor([[0], [1], [0]])
    result = dyn.refill_check(batch, exit_status=1)
    assert result.num_nodes_list == [1, 3] and len(sampler) == 2  # 2 atoms free: neither the 3 nor the 4 fits
    result["status"] = torch.tensor([[1], [1]])
    result = dyn.refill_check(result, exit_status=1)
    assert result.num_nodes_list == [4] and flat(result.system_id) == [3]  # largest first, then nothing else fits


def test_fused_stage_runs_a_dataset_through_a_batch_of_three_places():
    model = WellModel()
    hook = ConvergenceHook.from_fmax(0.05)
    n_total = 8
    sampler = SizeAwareSampler(Dataset([(2, 0)] * n_total, scale=0.3), max_atoms=6, max_batch_size=3)
    sink = HostMemory(capacity=20)
    seen_sizes, seen_ids = [], set()

    class Watch:
        frequency = 1
        stage = FusedStage._stage_type.BEFORE_STEP

        def __call__(self, ctx, stage):
            seen_sizes.append(ctx.batch.num_graphs)
            seen_ids.update(flat(ctx.batch.system_id))

    fused = FusedStage([(0, Relax(model=model, convergence_hook=hook))], sampler=sampler, refill_frequency=1,
                       sinks=[sink])
    fused.register_fused_hook(Watch())
    assert fused.run(None, n_steps=500) is None and fused.done and sampler.exhausted
    assert max(seen_sizes) == 3 and seen_ids == set(range(n_total))
    stored = sink.read()
    assert stored.num_graphs == n_total and sorted(flat(stored.system_id)) == list(range(n_total))
    assert flat(stored.status) == [1] * n_total
    # every stored system is relaxed to the criterion, and later samples (further out) took longer
    fmax = stored.forces.norm(dim=1).view(n_total, 2).max(dim=1).values
    assert bool((fmax <= 0.05).all())
    # a caller's batch instead of the sampler's first one; neither: an error
    sampler2 = SizeAwareSampler(Dataset([(2, 0)] * 4, scale=0.3), max_atoms=6, max_batch_size=3)
    first = sampler2.build_initial_batch()
    fused2 = FusedStage([(0, Relax(model=model, convergence_hook=hook))], sampler=sampler2, refill_frequency=2)
    assert fused2.run(first, n_steps=500) is None and fused2.done
    with pytest.raises(ValueError, match="No batch provided and no sampler configured"):
        FusedStage([(0, Relax(model=model, convergence_hook=hook))]).run(None, n_steps=3)


def test_refill_frequency_sets_how_often_places_are_checked():
    model = WellModel()
    hook = ConvergenceHook.from_fmax(0.05)

    def steps_with(freq):
        sampler = SizeAwareSampler(Dataset([(2, 0)] * 6, scale=0.3), max_atoms=4, max_batch_size=2)
        fused = FusedStage([(0, Relax(model=model, convergence_hook=hook))], sampler=sampler, refill_frequency=freq)
        fused.run(None, n_steps=2000)
        assert fused.done
        return fused.step_count

    quick, slow = steps_with(1), steps_with(7)
    assert slow > quick and slow % 7 == 0
