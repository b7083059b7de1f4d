"""CPU tests of the host-side mirror of the reference interfaces: Batch layout and key
routing, configs, hook registry gating and order, the step contract with a fake model,
status masking, convergence criteria.  They restate what the reference's own tests assert
(test/dynamics/test_base.py: RecordingHook :110, TestStepMasking :1003, frequency gating
:1497; test/models/test_lj_model.py; test/dynamics/test_ops.py::TestFireOptimizerState).
"""

from collections import OrderedDict

import pytest
import torch

from nvalchemi_amd.data import AtomicData, Batch
from nvalchemi_amd.dynamics import FIRE, NVE, BaseDynamics, ConvergenceHook, DynamicsStage
from nvalchemi_amd.dynamics._ops._bridge import _to_per_system
from nvalchemi_amd.dynamics._units import fs_to_internal_time
from nvalchemi_amd.models import (BaseModelMixin, LennardJonesModelWrapper, ModelConfig, NeighborConfig,
                                  NeighborListFormat)


def two_systems():
    d = []
    for n in (3, 5):
        d.append(AtomicData(torch.randn(n, 3), torch.full((n,), 6), cell=torch.eye(3) * 5,
                            pbc=torch.tensor([True, True, False]), forces=torch.zeros(n, 3),
                            energy=torch.zeros(1, 1)))
    return Batch.from_data_list(d)


class FakeModel(torch.nn.Module, BaseModelMixin):
    """Harmonic well: forces = -positions, energy = 0.5 sum r^2 per system."""

    def __init__(self):
        super().__init__()
        self.model_config = ModelConfig(outputs=frozenset({"energy", "forces"}))
        self.calls = 0

    def forward(self, batch):
        self.calls += 1
        e = torch.zeros(batch.num_graphs, dtype=batch.positions.dtype)
        e.index_add_(0, batch.batch_idx.long(), 0.5 * (batch.positions ** 2).sum(-1))
        return OrderedDict(energy=e.unsqueeze(-1), forces=-batch.positions.clone())


class RecordingHook:
    def __init__(self, stage, frequency=1, log=None):
        self.stage, self.frequency, self.log = stage, frequency, log if log is not None else []

    def __call__(self, ctx, stage):
        self.log.append((ctx.step_count, stage))


def test_batch_layout_and_lazy_index_tensors():
    b = two_systems()
    assert b.num_graphs == 2 and b.num_nodes == 8 and b.max_num_nodes == 5
    assert b.batch_idx.dtype == torch.int32 and b.batch_idx.tolist() == [0, 0, 0, 1, 1, 1, 1, 1]
    assert b.batch_ptr.dtype == torch.int32 and b.batch_ptr.tolist() == [0, 3, 8]
    assert b.cell.shape == (2, 3, 3) and b.pbc.shape == (2, 3) and b.pbc.dtype == torch.bool
    assert b.energy.shape == (2, 1) and b.velocities.shape == (8, 3) and float(b.velocities.abs().sum()) == 0
    assert b.atomic_masses.shape == (8,) and abs(float(b.atomic_masses[0]) - 12.011) < 1e-5
    assert b.edge_ptr.tolist() == [0] * 9
    assert getattr(b, "neighbor_matrix", None) is None
    with pytest.raises(AttributeError):
        b.neighbor_matrix


def test_batch_key_routing():
    b = two_systems()
    b["stress"] = torch.zeros(2, 3, 3)
    b.status = torch.zeros(2, 1, dtype=torch.long)
    b.my_unknown = torch.ones(2, 4)
    assert {"stress", "status", "my_unknown"} <= set(b._system_group.keys())
    assert b.status.dtype == torch.long
    b._atoms_group["neighbor_matrix"] = torch.zeros(8, 4, dtype=torch.int32)
    assert b.neighbor_matrix.shape == (8, 4)
    b.positions = torch.zeros(8, 3)
    assert "positions" in b._atoms_group and float(b.positions.abs().sum()) == 0
    b._neighbor_list_cutoff = 2.5
    assert b._neighbor_list_cutoff == 2.5 and "_neighbor_list_cutoff" not in b


def test_neighbor_list_index_key_is_offset_on_batching():
    d = [AtomicData(torch.zeros(2, 3), torch.ones(2, dtype=torch.long),
                    neighbor_list=torch.tensor([[0, 1], [1, 0]], dtype=torch.int32)) for _ in range(2)]
    b = Batch.from_data_list(d)
    assert b.neighbor_list.tolist() == [[0, 1], [1, 0], [2, 3], [3, 2]]
    assert b.num_edges == 4 and b.edge_ptr.tolist() == [0, 1, 2, 3, 4]


def test_atomic_data_validation():
    with pytest.raises(ValueError):
        AtomicData(torch.zeros(3, 2), torch.ones(3, dtype=torch.long))
    with pytest.raises(TypeError):
        AtomicData(torch.zeros(3, 3), torch.ones(3))
    with pytest.raises(ValueError):
        AtomicData(torch.zeros(3, 3), torch.ones(3, dtype=torch.long), forces=torch.zeros(2, 3))
    d = AtomicData(torch.zeros(3, 3, dtype=torch.float64), torch.ones(3, dtype=torch.long), cell=torch.eye(3))
    assert d.cell.dtype == torch.float64 and d.cell.shape == (1, 3, 3)


def test_neighbor_config_defaults_and_lj_model_config():
    nc = NeighborConfig(cutoff=3.0)
    assert nc.format == NeighborListFormat.COO and nc.half_list is False and nc.skin == 0.0
    lj = LennardJonesModelWrapper(epsilon=0.01, sigma=3.4, cutoff=8.5)
    cfg = lj.model_config
    assert cfg.neighbor_config.format == NeighborListFormat.MATRIX and cfg.neighbor_config.cutoff == 8.5
    assert cfg.active_outputs == {"energy", "forces"} and cfg.outputs == frozenset({"energy", "forces", "stress"})
    assert lj.input_data() == {"positions", "atomic_numbers", "neighbor_matrix", "num_neighbors"}
    assert lj.output_data() == {"energy", "forces"}
    hooks = lj.make_neighbor_hooks(max_neighbors=48)
    assert len(hooks) == 1 and hooks[0].stage == DynamicsStage.BEFORE_COMPUTE and hooks[0]._max_neighbors_override == 48
    with pytest.raises(KeyError):
        lj(two_systems())
    assert LennardJonesModelWrapper(0.01, 3.4, 8.5, switch_width=0.5).switch_width == 0.5
    with pytest.raises(ValueError):
        LennardJonesModelWrapper(0.01, 3.4, 8.5, switch_width=9.0)


def test_adapt_output_stress_is_minus_virial_over_volume():
    lj = LennardJonesModelWrapper(0.01, 3.4, 8.5)
    lj.model_config.active_outputs = {"energy", "forces", "stress"}
    b = two_systems()
    W = torch.arange(18, dtype=torch.float32).view(2, 3, 3)
    out = lj.adapt_output({"energy": torch.zeros(2, 1), "forces": torch.zeros(8, 3), "virial": W}, b)
    assert torch.allclose(out["stress"], -W / 125.0)


def test_hook_order_and_frequency_gating():
    log = []
    hooks = [RecordingHook(s, log=log) for s in DynamicsStage if s != DynamicsStage.ON_CONVERGE]
    every_other = RecordingHook(DynamicsStage.AFTER_STEP, frequency=2)
    dyn = BaseDynamics(FakeModel(), hooks=hooks + [every_other])
    b = two_systems()
    dyn.run(b, n_steps=3)
    assert [s for (k, s) in log if k == 0] == [DynamicsStage(i) for i in range(8)]
    assert [k for (k, s) in every_other.log] == [0, 2]
    assert dyn.step_count == 3 and dyn.model.calls == 3
    with pytest.raises(ValueError):
        dyn.register_hook(RecordingHook(DynamicsStage.AFTER_STEP, frequency=0))
    with pytest.raises(TypeError):
        dyn.register_hook(RecordingHook(None))
    with pytest.raises(TypeError):
        BaseDynamics(torch.nn.Linear(1, 1))
    with pytest.raises(ValueError):
        BaseDynamics(FakeModel()).run(b)


def test_compute_copies_into_existing_batch_tensors_only():
    dyn = BaseDynamics(FakeModel())
    b = two_systems()
    f_before = b.forces
    out = dyn.compute(b)
    assert b.forces is f_before and torch.equal(b.forces, -b.positions)
    assert b.energy.shape == (2, 1) and torch.allclose(b.energy, out["energy"])

    class Needs(BaseDynamics):
        __needs_keys__ = {"stress"}

    with pytest.raises(RuntimeError):
        Needs(FakeModel()).compute(b)


class Drift(BaseDynamics):
    """pre_update moves everything; used to see which systems the step protects."""

    def pre_update(self, batch):
        batch.positions += 1.0
        batch.cell += 1.0


def test_step_masking_preserves_graduated_systems():
    b = two_systems()
    b.status = torch.tensor([[0], [1]])
    p0, c0 = b.positions.clone(), b.cell.clone()
    Drift(FakeModel()).step(b)
    assert torch.equal(b.positions[:3], p0[:3] + 1) and torch.equal(b.positions[3:], p0[3:])
    assert torch.equal(b.cell[0], c0[0] + 1) and torch.equal(b.cell[1], c0[1])
    b2 = two_systems()
    b2.status = torch.tensor([[0], [1]])
    p0 = b2.positions.clone()
    Drift(FakeModel(), exit_status=2).step(b2)
    assert torch.equal(b2.positions, p0 + 1)


def test_convergence_criteria_and_status_migration():
    b = two_systems()
    b.forces[:3] = 0.01
    b.forces[3:] = 1.0
    hook = ConvergenceHook.from_fmax(0.05)
    assert hook.evaluate(b).tolist() == [0]
    b.forces[:] = 1.0
    assert hook.evaluate(b) is None
    both = ConvergenceHook(criteria=[{"key": "forces", "threshold": 2.0, "reduce_op": "norm"},
                                     {"key": "energy", "threshold": -1.0}])
    assert both.num_criteria == 2 and both.evaluate(b) is None
    b.energy[1] = -2.0
    assert both.evaluate(b).tolist() == [1]
    with pytest.raises(KeyError):
        ConvergenceHook(criteria={"key": "nope", "threshold": 1.0}).evaluate(b)
    with pytest.raises(TypeError):
        ConvergenceHook(criteria=3)
    b.status = torch.tensor([[0], [0]])
    mig = ConvergenceHook(criteria={"key": "energy", "threshold": -1.0}, source_status=0, target_status=1)
    dyn = BaseDynamics(FakeModel(), hooks=[mig])
    mig(dyn._build_context(b), DynamicsStage.AFTER_STEP)
    assert b.status.view(-1).tolist() == [0, 1]
    # run() stops early once every system has converged
    done = BaseDynamics(FakeModel(), convergence_hook={"criteria": {"key": "energy", "threshold": 1e9}})
    done.run(two_systems(), n_steps=10)
    assert done.step_count == 1


def test_integrator_state_shapes_and_units():
    b = two_systems()
    nve = NVE(FakeModel(), dt=0.5)
    nve._init_state(b)
    assert nve._state.dt.shape == (2,) and torch.allclose(nve._state.dt, torch.tensor(0.5 / 10.180505710759414))
    assert fs_to_internal_time(10.180505710759414) == pytest.approx(1.0)
    fire = FIRE(FakeModel(), dt=2.0)
    fire._init_state(b)
    s = fire._state
    for k in ("dt", "dt_max", "dt_min", "alpha", "alpha_start", "f_alpha", "maxstep", "f_dec", "f_inc", "vf", "vv", "ff"):
        assert getattr(s, k).shape == (2,) and getattr(s, k).dtype == torch.float32, k
    for k in ("n_min", "uphill_flag", "n_steps_positive"):
        assert getattr(s, k).dtype == torch.int32, k
    assert s.dt.tolist() == [2.0, 2.0] and s.dt_max.tolist() == [20.0, 20.0] and torch.allclose(s.dt_min, torch.tensor(0.04))
    assert s.n_min.tolist() == [5, 5] and s.alpha.tolist() == pytest.approx([0.1, 0.1])
    with pytest.raises(NotImplementedError):
        FIRE(FakeModel(), dt=1.0, uphill=True)
    assert _to_per_system(torch.tensor([3.0]), 4, "cpu", torch.float32).tolist() == [3.0] * 4
    with pytest.raises(ValueError):
        _to_per_system(torch.ones(3), 4, "cpu", torch.float32)


def test_estimate_max_neighbors_is_a_multiple_of_16_and_monotone():
    from nvalchemi_amd._neighbor_ops import ceil16, estimate_max_neighbors

    ks = [estimate_max_neighbors(rc) for rc in (1.0, 2.5, 5.0, 6.0, 8.5)]
    assert all(k % 16 == 0 and k >= 16 for k in ks) and ks == sorted(ks)
    assert ceil16(1) == 16 and ceil16(16) == 16 and ceil16(17) == 32


def test_strategy_helpers_of_the_neighbor_hook():
    """The two helpers the reference hook imports unconditionally
    (nvalchemi/hooks/neighbor_list.py:63-65): a strategy name and its base method."""
    from nvalchemi_amd._neighbor_ops import neighbor_list_strategy_run_args, suggest_neighbor_list_method

    ptr = torch.tensor([0, 5, 9], dtype=torch.int32)
    name = suggest_neighbor_list_method(ptr, torch.eye(3).repeat(2, 1, 1) * 10, torch.ones(2, 3, dtype=torch.bool), 3.0,
                                        half_fill=False, return_neighbor_list=False, positions_dtype=torch.float32)
    base, extra = neighbor_list_strategy_run_args(name)
    assert base.endswith("cell_list") and extra == {}
    assert neighbor_list_strategy_run_args("batch_cell_list_pair_centric")[0] == "batch_cell_list"
    with pytest.raises(ValueError):
        neighbor_list_strategy_run_args("no_such_strategy")
    # float32 and float64 positions are both served (as in the reference); anything else is refused
    assert suggest_neighbor_list_method(ptr, torch.eye(3).repeat(2, 1, 1), torch.ones(2, 3, dtype=torch.bool), 3.0,
                                        positions_dtype=torch.float64) == name
    with pytest.raises(TypeError):
        suggest_neighbor_list_method(ptr, torch.eye(3).repeat(2, 1, 1), torch.ones(2, 3, dtype=torch.bool), 3.0,
                                     positions_dtype=torch.float16)


def test_batch_index_select_append_and_trim():
    """Selecting, appending and trimming systems (nvalchemi/data/batch.py:816-874, 987-1038,
    1138-1178): segments gathered in the order asked, ``neighbor_list`` re-based, system rows
    following, the receiver of ``append`` growing in place."""
    from nvalchemi_amd.data import AtomicData, Batch

    g = torch.Generator().manual_seed(0)
    data = []
    for n in (3, 5, 2, 4):
        nl = torch.tensor([[0, 1], [1, 0], [n - 1, 0]], dtype=torch.int32)
        data.append(AtomicData(torch.rand(n, 3, generator=g), torch.full((n,), n), cell=torch.eye(3) * n,
                               pbc=torch.ones(3, dtype=torch.bool), neighbor_list=nl,
                               energy=torch.full((1, 1), float(n))))
    b = Batch.from_data_list(data)
    s = b.index_select([2, 0])
    assert s.num_graphs == 2 and s.batch_ptr.tolist() == [0, 2, 5] and s.atomic_numbers.tolist() == [2, 2, 3, 3, 3]
    assert s.neighbor_list.tolist() == [[0, 1], [1, 0], [1, 0], [2, 3], [3, 2], [4, 2]]
    assert s.energy.view(-1).tolist() == [2.0, 3.0] and s.num_edges_per_graph.tolist() == [3, 3]
    assert torch.equal(s.positions[2:5], b.positions[0:3]) and torch.equal(s.cell[0], b.cell[2])
    s.append(b.index_select([3]))
    assert s.num_graphs == 3 and s.batch_ptr.tolist() == [0, 2, 5, 9] and s.neighbor_list[-3:].tolist() == [[5, 6], [6, 5], [8, 5]]
    assert s.batch_idx.tolist() == [0, 0, 1, 1, 1, 2, 2, 2, 2]
    assert b[1:3].num_nodes_list == [5, 2] and isinstance(b[0], AtomicData) and b[-1].num_nodes == 4
    assert b[torch.tensor([True, False, False, True])].num_nodes_list == [3, 4]
    assert b.trim(torch.tensor([True, True, False, False])).num_nodes_list == [2, 4]
    assert b.trim(torch.ones(4, dtype=torch.bool)) is None
    with pytest.raises(ValueError):
        b.append(b)
    with pytest.raises(IndexError):
        b.index_select([])
    with pytest.raises(IndexError):
        b.index_select(torch.tensor([0.5]))
    with pytest.raises(ValueError):
        b.trim()


def test_fixed_capacity_batches_and_host_sink_on_the_host():
    """The bookkeeping of ``Batch.empty`` / ``zero`` / ``empty_like`` (nvalchemi/data/batch.py:569-737,
    1583-1616) and the ``HostMemory`` sink (nvalchemi/dynamics/sinks.py:537-670) need no kernel; the
    masked copies do, and refuse host tensors instead of copying some other way."""
    from nvalchemi_amd import _lib
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.dynamics import DataSink, GPUBuffer, HostMemory

    g = torch.Generator().manual_seed(1)
    data = [AtomicData(torch.rand(n, 3, generator=g), torch.full((n,), n), cell=torch.eye(3) * n,
                       pbc=torch.ones(3, dtype=torch.bool), energy=torch.full((1, 1), float(n)),
                       neighbor_list=torch.tensor([[0, n - 1], [n - 1, 0]])) for n in (3, 5, 2)]
    b = Batch.from_data_list(data)
    buf = Batch.empty(num_systems=4, num_nodes=20, num_edges=8, template=b)
    assert buf.num_graphs == 0 and buf.system_capacity == 4 and buf.num_nodes == 0 and buf.num_edges == 0
    assert buf.positions.shape == (20, 3) and buf.cell.shape == (4, 3, 3) and buf.neighbor_list.shape == (8, 2)
    assert buf.atomic_numbers.dtype == b.atomic_numbers.dtype and buf.batch_ptr.tolist() == [0]
    assert buf._atoms_group._ptr_store().shape[0] == 6 and buf.num_nodes_list == []
    buf.zero()
    assert buf.num_graphs == 0 and buf.system_capacity == 4
    like = Batch.empty_like(b)
    assert like.num_graphs == 0 and like.system_capacity == 0 and sorted(like.keys()) == sorted(b.keys())
    with pytest.raises(_lib.KernelLibraryError):
        buf.put(b, torch.ones(3, dtype=torch.bool))
    with pytest.raises(_lib.KernelLibraryError):
        b.defrag(copied_mask=torch.tensor([True, False, False]))
    with pytest.raises(ValueError, match="defrag requires copied_mask or a prior put"):
        Batch.from_data_list(data).defrag()

    with pytest.raises(TypeError):
        DataSink()
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="requires an available GPU"):
            GPUBuffer(capacity=1, max_atoms=1, max_edges=0)
    sink = HostMemory(capacity=3)
    sink.write(b, mask=torch.tensor([False, True, True]))
    assert len(sink) == 2 and not sink.is_full
    with pytest.raises(RuntimeError, match="Buffer is full"):
        sink.write(b)
    out = sink.drain()
    assert len(sink) == 0 and out.num_nodes_list == [5, 2] and out.neighbor_list.tolist() == [[0, 4], [4, 0], [5, 6], [6, 5]]
    assert torch.equal(out.positions, b.positions[3:]) and out.energy.view(-1).tolist() == [5.0, 2.0]
    got = b.to_data_list()
    assert [d.num_nodes for d in got] == [3, 5, 2] and got[1].neighbor_list.tolist() == [[0, 4], [4, 0]]
    b.append_data([data[0]])
    assert b.num_nodes_list == [3, 5, 2, 3]
    with pytest.raises(ValueError, match="No data provided"):
        b.append_data([])


def test_state_of_the_thermostats_and_of_fire2_and_the_rows_made_for_newcomers():
    """Per-system state of the other integrators (restating test/dynamics/test_state_management.py:249-530):
    shapes, dtypes, internal units, and ``_make_new_state`` for systems that join a running batch."""
    from nvalchemi_amd.dynamics import FIRE2, NVTLangevin, NVTNoseHoover

    b = two_systems()
    FS = 10.180505710759414
    kB = 8.617333262e-5
    lang = NVTLangevin(FakeModel(), dt=1.0, temperature=300.0, friction=0.1)
    lang._init_state(b)
    s = lang._state
    assert s.dt.shape == s.temperature.shape == s.friction.shape == (2,) and s.num_graphs == 2
    assert torch.allclose(s.temperature, torch.tensor(300.0 * kB)) and torch.allclose(s.friction, torch.tensor(0.1 * FS))
    assert lang._make_new_state(3, b).friction.shape == (3,)

    for M_new, C in ((1, 3), (4, 5)):
        nhc = NVTNoseHoover(FakeModel(), dt=1.0, temperature=torch.tensor([100.0, 300.0]), thermostat_time=50.0,
                            chain_length=C)
        nhc._init_state(b)
        s = nhc._state
        assert s.dt.shape == s.temperature.shape == s.nhc_ndof.shape == (2,)
        assert s.nhc_eta.shape == s.nhc_eta_dot.shape == s.nhc_Q.shape == (2, C) and s.num_graphs == 2
        assert s.nhc_ndof.tolist() == [9.0, 15.0] and not s.nhc_eta.any() and not s.nhc_eta_dot.any()
        kT, tau = torch.tensor([100.0, 300.0]) * kB, 50.0 / FS
        assert torch.allclose(s.nhc_Q[:, 1], kT * tau * tau) and torch.allclose(s.nhc_Q[:, 0], s.nhc_ndof * kT * tau * tau)
        fresh = NVTNoseHoover(FakeModel(), dt=1.0, temperature=300.0, thermostat_time=50.0,
                              chain_length=C)._make_new_state(M_new, b)
        assert fresh.nhc_eta.shape == (M_new, C) and fresh.nhc_Q.shape == (M_new, C) and fresh.num_graphs == M_new
        assert fresh.nhc_ndof.tolist() == [12.0] * M_new  # the batch's mean system size: 8 atoms in 2 systems
    with pytest.raises(ValueError, match="yoshida_order"):
        NVTNoseHoover(FakeModel(), dt=1.0, temperature=300.0, thermostat_time=50.0, yoshida_order=4)

    f2 = FIRE2(FakeModel(), dt=0.05)
    f2._init_state(b)
    s = f2._state
    assert s.dt.tolist() == pytest.approx([0.05, 0.05]) and s.alpha.tolist() == pytest.approx([0.09, 0.09])
    assert s.nsteps_inc.dtype == torch.int32 and s.nsteps_inc.tolist() == [0, 0] and s.num_graphs == 2
    for k in ("vf", "v_sumsq", "f_sumsq"):
        assert getattr(s, k).shape == (2,)
    assert (f2.delaystep, f2.dtgrow, f2.dtshrink, f2.alphashrink, f2.tmax, f2.tmin, f2.maxstep) == \
        (60, 1.05, 0.75, 0.985, 0.08, 0.005, 0.1)
    assert f2._make_new_state(3, b).alpha.tolist() == pytest.approx([0.09] * 3)
    # the kernels behind them refuse host tensors
    from nvalchemi_amd import _lib

    b.velocities = torch.zeros(8, 3)
    for dyn in (nhc, f2):
        with pytest.raises(_lib.KernelLibraryError):
            dyn.pre_update(b)
