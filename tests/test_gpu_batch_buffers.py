"""Fixed-capacity batches and data sinks on the GPU: ``Batch.empty / put / defrag / zero / trim``
(nvalchemi/data/batch.py:569-1038) and ``GPUBuffer`` / ``HostMemory``
(nvalchemi/dynamics/sinks.py), the callers of the masked-copy kernels.

The cases restate the reference's own (test/data/test_batch.py::TestBatchPutDefrag,
test/dynamics/test_sinks.py::TestGPUBuffer, ::TestHostMemory) and add what those leave open:
the values that arrive, checked bit for bit against the source systems taken one by one.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _system(n, seed, *, with_cell=True, edges=0):
    from nvalchemi_amd.data import AtomicData

    g = torch.Generator().manual_seed(seed)
    kw = dict(forces=torch.randn(n, 3, generator=g), energy=torch.randn(1, 1, generator=g),
              velocities=torch.randn(n, 3, generator=g), atomic_masses=torch.rand(n, generator=g) + 1.0)
    if with_cell:
        kw["cell"] = torch.eye(3) * (5.0 + seed) + 0.1 * torch.randn(3, 3, generator=g)
        kw["pbc"] = torch.tensor([True, seed % 2 == 0, True])
        kw["system_id"] = torch.full((1, 1), 100 + seed, dtype=torch.long)
    if edges:
        kw["neighbor_list"] = torch.randint(0, n, (edges, 2), generator=g)
        kw["neighbor_list_shifts"] = torch.randint(-1, 2, (edges, 3), generator=g, dtype=torch.int32)
        kw["shifts"] = torch.randn(edges, 3, generator=g)
    return AtomicData(torch.randn(n, 3, generator=g), torch.randint(1, 90, (n,), generator=g), **kw)


def _batch(sizes, seed0=0, **kw):
    from nvalchemi_amd.data import Batch

    systems = [_system(n, seed0 + k, **kw) for k, n in enumerate(sizes)]
    return Batch.from_data_list(systems, device=DEV), systems


def _same_system(got, want, keys=None):
    """Every key of ``want`` (an AtomicData on the host) is in ``got`` with the same bits."""
    for k in (keys if keys is not None else want.keys()):
        a, b = getattr(got, k).cpu(), getattr(want, k)
        assert a.dtype == b.dtype and a.shape == b.shape, (k, a.dtype, b.dtype, a.shape, b.shape)
        assert torch.equal(a, b), k


# ---- test_batch.py::TestBatchPutDefrag -------------------------------------------------------------
def test_put_leaves_the_copied_mask_on_the_source_or_in_the_argument():
    buffer, _ = _batch([2, 2])
    src, _ = _batch([2, 2], 5)
    buffer.put(src, torch.tensor([False, False]))
    assert src._copied_mask.shape == (2,) and int(src._copied_mask.sum()) == 0
    one, _ = _batch([2], 9)
    copied = torch.zeros(1, dtype=torch.bool, device=DEV)
    buffer.put(one, torch.tensor([False]), copied_mask=copied)
    assert copied.shape == (1,) and int(copied.sum()) == 0
    with pytest.raises(ValueError, match="mask shape"):
        buffer.put(one, torch.tensor([True, False]))


def test_a_batch_without_headroom_takes_nothing():
    buffer, _ = _batch([2, 2])
    before = buffer.positions.clone()
    src, _ = _batch([2, 2], 5)
    copied = torch.ones(2, dtype=torch.bool, device=DEV)
    buffer.put(src, torch.tensor([True, True]), copied_mask=copied)
    assert int(copied.sum()) == 0 and buffer.num_graphs == 2
    assert torch.equal(buffer.positions, before)
    # a mask on the host is updated all the same
    copied_host = torch.ones(2, dtype=torch.bool)
    buffer.put(src, torch.tensor([True, True]), copied_mask=copied_host)
    assert int(copied_host.sum()) == 0


def test_defrag_drops_the_marked_systems_and_keeps_the_rest_bit_for_bit():
    batch, systems = _batch([2, 3, 1, 4], edges=5)
    cap_rows = batch.positions.shape[0]
    batch.defrag(copied_mask=torch.tensor([True, False, True, False]))
    assert batch.num_graphs == 2 and batch.num_nodes_list == [3, 4] and batch.num_nodes == 7
    assert batch.num_edges_list == [5, 5] and batch.num_edges == 10
    assert len(batch.num_nodes_per_graph) == 2 and int(batch.num_nodes_per_graph.sum()) == 7
    assert batch.batch_idx.tolist() == [0] * 3 + [1] * 4 and batch.batch_ptr.tolist() == [0, 3, 7]
    # the storage keeps its size, the rows behind the kept ones are zero
    assert batch.positions.shape[0] == cap_rows and not batch.positions[7:].any()
    assert not batch.atomic_numbers[7:].any() and not batch.cell[2:].any()
    _same_system(batch.get_data(0), systems[1])
    _same_system(batch.get_data(1), systems[3])
    with pytest.raises(ValueError, match="defrag requires copied_mask or a prior put"):
        batch.defrag()
    with pytest.raises(ValueError, match="copied_mask shape"):
        batch.defrag(copied_mask=torch.tensor([True, False, True, False]))
    # a second pass over the compacted storage
    batch.defrag(copied_mask=torch.tensor([True, False]))
    assert batch.num_graphs == 1 and batch.num_nodes == 4
    _same_system(batch.get_data(0), systems[3])
    # selection and growth work on the compacted storage
    more, more_sys = _batch([2], 40, edges=5)
    batch.append(more)
    assert batch.num_nodes_list == [4, 2] and batch.positions.shape[0] == 6
    _same_system(batch.get_data(0), systems[3])
    _same_system(batch.get_data(1), more_sys[0])


def test_put_into_an_empty_buffer_then_defrag_or_trim_of_the_source():
    from nvalchemi_amd.data import Batch

    batch, systems = _batch([3, 5, 4, 3], edges=6)
    buffer = Batch.empty(num_systems=4, num_nodes=50, num_edges=40, template=systems[0], device=DEV)
    assert buffer.num_graphs == 0 and buffer.system_capacity == 4 and buffer.num_nodes == 0
    buffer.put(batch, torch.tensor([True, False, True, False]))
    assert batch._copied_mask.tolist() == [True, False, True, False]
    assert buffer.num_graphs == 2 and buffer.num_nodes_list == [3, 4] and buffer.num_edges_list == [6, 6]
    assert buffer.positions.shape[0] == 50 and buffer.system_capacity == 4
    _same_system(buffer.get_data(0), systems[0])
    _same_system(buffer.get_data(1), systems[2])
    # every system-level key of a system sits in the same slot
    assert torch.equal(buffer.system_id[:2].cpu().view(-1), torch.tensor([100, 102]))
    assert torch.equal(buffer.cell[1].cpu(), systems[2].cell[0]) and not buffer.cell[2:].any()
    tight = buffer.index_select([1, 0])
    assert tight.positions.shape[0] == 7
    _same_system(tight.get_data(0), systems[2])

    trimmed = batch.trim()
    assert trimmed.num_graphs == 2 and trimmed.num_nodes == 8 and trimmed.positions.shape[0] == 8
    _same_system(trimmed.get_data(0), systems[1])
    batch.defrag()
    assert batch.num_graphs == 2 and batch.num_nodes == 8 and len(batch.num_nodes_list) == 2
    assert "_copied_mask" not in batch.__dict__
    expanded = torch.repeat_interleave(torch.ones(2, dtype=torch.bool, device=DEV),
                                       batch.num_nodes_per_graph.to(torch.long))
    assert len(expanded) == batch.num_nodes
    _same_system(batch.get_data(0), systems[1])
    _same_system(batch.get_data(1), systems[3])

    # a put cuts the boundaries to the segments in use: without new headroom nothing more goes in
    copied = torch.zeros(2, dtype=torch.bool, device=DEV)
    buffer.put(batch, torch.tensor([True, True]), copied_mask=copied)
    assert int(copied.sum()) == 0 and buffer.num_graphs == 2

    buffer.zero()
    assert buffer.num_graphs == 0 and buffer.system_capacity == 4 and buffer.positions.shape[0] == 50
    assert not buffer.positions.any() and not buffer.atomic_numbers.any() and not buffer.cell.any()


def test_only_the_systems_that_fit_on_every_level_move():
    from nvalchemi_amd.data import Batch

    batch, systems = _batch([3, 5, 4, 3])
    # room for 8 atoms: systems 0 and 1 fit, 2 does not, 3 would fit by size but comes behind 2
    buffer = Batch.empty(num_systems=4, num_nodes=8, num_edges=0, template=systems[0], device=DEV)
    buffer.put(batch, torch.ones(4, dtype=torch.bool))
    assert batch._copied_mask.tolist() == [True, True, False, False]
    assert buffer.num_graphs == 2 and buffer.num_nodes == 8
    _same_system(buffer.get_data(1), systems[1])
    # two free system slots only: the occupied one is skipped, the mask of slots is updated
    batch2, systems2 = _batch([1, 1, 1], 20)
    small = Batch.empty(num_systems=3, num_nodes=30, num_edges=0, template=systems2[0], device=DEV)
    slots = torch.tensor([True, False, False], device=DEV)
    small.put(batch2, torch.ones(3, dtype=torch.bool), dest_mask=slots)
    assert batch2._copied_mask.tolist() == [True, True, False] and small.num_graphs == 2
    assert slots.tolist() == [True, True, True]
    assert small.system_id.cpu().view(-1).tolist() == [0, 120, 121]
    assert torch.equal(small.cell[2].cpu(), systems2[1].cell[0]) and small.pbc[1].cpu().tolist() == [True, True, True]
    # a source of more systems than the boundaries have headroom for moves nothing
    two = Batch.empty(num_systems=2, num_nodes=30, num_edges=0, template=systems2[0], device=DEV)
    two.put(batch2, torch.ones(3, dtype=torch.bool))
    assert batch2._copied_mask.tolist() == [False, False, False] and two.num_graphs == 0
    with pytest.raises(ValueError, match="non-negative"):
        Batch.empty(num_systems=-1, num_nodes=1, num_edges=0)
    default = Batch.empty(num_systems=3, num_nodes=10, num_edges=0, device=DEV)
    assert sorted(k for k in default.keys() if k in ("positions", "atomic_numbers", "energy")) == \
        ["atomic_numbers", "energy", "positions"]
    assert Batch.empty_like(batch).num_graphs == 0


# ---- test_sinks.py::TestGPUBuffer -------------------------------------------------------------------
def test_gpu_buffer_round_trip_accumulation_and_limits():
    from nvalchemi_amd.dynamics import GPUBuffer

    buf = GPUBuffer(capacity=6, max_atoms=5, max_edges=8, device="cuda")
    assert buf.capacity == 6 and buf.device.type == "cuda" and len(buf) == 0 and not buf.is_full
    with pytest.raises(RuntimeError, match="empty"):
        buf.read()
    with pytest.raises(RuntimeError, match="empty"):
        buf.drain()
    with pytest.raises(RuntimeError, match="GPU device"):
        GPUBuffer(capacity=1, max_atoms=1, max_edges=0, device="cpu")

    b1, s1 = _batch([2, 5], edges=4)
    b2, s2 = _batch([3, 1, 4], 10, edges=4)
    buf.write(b1)
    assert len(buf) == 2
    buf.write(b2, mask=torch.tensor([True, False, True]))
    assert len(buf) == 4 and not buf.is_full
    buf.write(b2, mask=torch.tensor([False, False, False]))
    assert len(buf) == 4
    with pytest.raises(ValueError, match="mask length"):
        buf.write(b2, mask=torch.tensor([True]))
    got = buf.read()
    assert got.num_graphs == 4 and got.num_nodes_list == [2, 5, 3, 4] and got.positions.shape[0] == 14
    for k, want in enumerate((s1[0], s1[1], s2[0], s2[2])):
        _same_system(got.get_data(k), want)
    # reading does not consume
    assert len(buf) == 4
    with pytest.raises(RuntimeError, match="Buffer is full"):
        buf.write(b2)
    big, _ = _batch([6], 30, edges=4)
    with pytest.raises(RuntimeError, match="Atom capacity exceeded"):
        buf.write(big)
    many, _ = _batch([2], 31, edges=9)
    with pytest.raises(RuntimeError, match="Edge capacity exceeded"):
        buf.write(many)
    buf.write(b1)
    assert buf.is_full and len(buf) == 6
    full = buf.read()
    assert full.num_graphs == 6
    _same_system(full.get_data(5), s1[1])

    drained = buf.drain()
    assert drained.num_graphs == 6 and len(buf) == 0
    # the storage is kept and zeroed, and takes new systems
    assert buf._buffer.system_capacity == 6 and not buf._buffer.positions.any()
    buf.write(b2)
    assert len(buf) == 3
    _same_system(buf.read().get_data(1), s2[1])


# ---- test_sinks.py::TestHostMemory ------------------------------------------------------------------
def test_host_memory_keeps_systems_on_the_host():
    from nvalchemi_amd.dynamics import HostMemory

    sink = HostMemory(capacity=4)
    assert sink.capacity == 4 and len(sink) == 0
    with pytest.raises(RuntimeError, match="empty"):
        sink.read()
    b, s = _batch([2, 3, 1], edges=3)
    sink.write(b, mask=torch.tensor([True, False, True]))
    assert len(sink) == 2
    sink.write(b, mask=torch.tensor([False, False, False]))
    assert len(sink) == 2
    with pytest.raises(ValueError, match="mask length"):
        sink.write(b, mask=torch.tensor([True]))
    with pytest.raises(RuntimeError, match="Buffer is full"):
        sink.write(b)
    got = sink.read()
    assert got.device.type == "cpu" and got.positions.device.type == "cpu" and got.num_nodes_list == [2, 1]
    _same_system(got.get_data(0), s[0])
    _same_system(got.get_data(1), s[2])
    # the stored systems do not alias the batch they came from
    b.positions.zero_()
    _same_system(sink.read().get_data(0), s[0])
    sink.write(b, mask=torch.tensor([False, True, True]))
    assert sink.is_full
    sink.zero()
    assert len(sink) == 0


def test_fused_stage_writes_finished_systems_to_its_sinks_in_order():
    """Systems that leave an in-flight batch go to the first sink with room
    (nvalchemi/dynamics/base.py:878-901, 1999-2000): what the sinks hold is what the step hook saw
    leave, bit for bit, whichever sink it went to."""
    from nvalchemi_amd.data import AtomicData
    from nvalchemi_amd.dynamics import (FIRE, ConvergenceHook, FusedStage, GPUBuffer, HostMemory,
                                        SizeAwareSampler)
    from nvalchemi_amd.models import LennardJonesModelWrapper
    from _systems import fcc_boxes

    P, C, pb, ptr = fcc_boxes(seed=9, n_boxes=6, reps=2, a=5.4, jitter=0.0)
    rng = np.random.default_rng(4)
    for s, amp in enumerate((0.02, 0.2, 0.05, 0.12, 0.03, 0.3)):
        P[ptr[s]:ptr[s + 1]] += rng.normal(0, amp, (ptr[s + 1] - ptr[s], 3)).astype(np.float32)

    def system(s):
        a0, a1 = int(ptr[s]), int(ptr[s + 1])
        n = a1 - a0
        return AtomicData(torch.from_numpy(P[a0:a1]), torch.full((n,), 18), atomic_masses=torch.full((n,), 39.95),
                          forces=torch.zeros(n, 3), energy=torch.zeros(1, 1), velocities=torch.zeros(n, 3),
                          cell=torch.from_numpy(C[s]), pbc=torch.from_numpy(pb[s])).to(DEV)

    class Dataset:
        """The dataset protocol of the sampler over a list of systems."""

        def __len__(self):
            return 6

        def get_metadata(self, k):
            return int(ptr[k + 1] - ptr[k]), 0

        def __getitem__(self, k):
            return system(k), {}

    n_atoms = int(ptr[1] - ptr[0])
    model = LennardJonesModelWrapper(epsilon=0.0104, sigma=3.4, cutoff=5.0)
    relax = FIRE(model, dt=1.0, convergence_hook=ConvergenceHook.from_fmax(0.02))
    sinks = [GPUBuffer(capacity=8, max_atoms=n_atoms, max_edges=0, device=DEV), HostMemory(capacity=10)]
    # room for three systems by atoms, four by count: the atom budget is what binds
    sampler = SizeAwareSampler(Dataset(), max_atoms=3 * n_atoms + 5, max_batch_size=4)
    left = {}

    class Collect:
        frequency = 1
        stage = FusedStage._stage_type.AFTER_STEP

        def __call__(self, ctx, stage):
            b = ctx.batch
            for k in torch.where(b.status.view(-1) >= 1)[0].tolist():
                sid = int(b.system_id.view(-1)[k])
                a0, a1 = int(b.batch_ptr[k]), int(b.batch_ptr[k + 1])
                left.setdefault(sid, (b.positions[a0:a1].cpu(), b.forces[a0:a1].cpu(), b.energy[k].cpu()))

    fused = FusedStage([(0, relax)], hooks=model.make_neighbor_hooks(), sampler=sampler, refill_frequency=1,
                       sinks=sinks)
    fused.register_fused_hook(Collect())
    out = fused.run(None, n_steps=2000)
    assert out is None and fused.done and sampler.exhausted and sorted(left) == list(range(6))
    assert len(sinks[0]) == 6 and len(sinks[1]) == 0
    # the batch carried the hook's neighbor matrix; the buffer does not allocate room for it
    assert "neighbor_matrix" not in sinks[0]._buffer and "positions" in sinks[0]._buffer
    seen = []
    for sink in sinks[:1]:
        stored = sink.read()
        for k in range(stored.num_graphs):
            d = stored.get_data(k)
            sid = int(d.system_id)
            seen.append(sid)
            pos, frc, en = left[sid]
            assert torch.equal(d.positions.cpu(), pos) and torch.equal(d.forces.cpu(), frc)
            assert torch.equal(d.energy.cpu().view(-1), en.view(-1))
            assert torch.equal(d.atomic_numbers.cpu(), torch.full((n_atoms,), 18))
            assert int(d.status) >= 1
    assert sorted(seen) == list(range(6))
    # the first sink that is not full takes the whole write -- or refuses it
    stored = sinks[0].read()
    order = FusedStage([(0, relax)], sinks=[GPUBuffer(capacity=3, max_atoms=n_atoms, max_edges=0, device=DEV),
                                            HostMemory(capacity=3)])
    pick = lambda *ids: torch.tensor([k in ids for k in range(6)], device=DEV)
    order._overflow_to_sinks(stored, mask=pick(0, 4))
    assert [len(s) for s in order.sinks] == [2, 0]
    with pytest.raises(RuntimeError, match="Buffer is full"):
        order._overflow_to_sinks(stored, mask=pick(1, 2))
    order._overflow_to_sinks(stored, mask=pick(5))
    order._overflow_to_sinks(stored, mask=pick(1, 2))
    assert [len(s) for s in order.sinks] == [3, 2]
    assert order.sinks[0].read().system_id.view(-1).tolist() == [seen[0], seen[4], seen[5]]
    assert order.sinks[1].read().system_id.view(-1).tolist() == [seen[1], seen[2]]
    with pytest.raises(RuntimeError, match="Buffer is full"):
        order._overflow_to_sinks(stored, mask=pick(0, 3))
    order._overflow_to_sinks(stored, mask=pick(3))
    with pytest.raises(RuntimeError, match="All sinks are full"):
        order._overflow_to_sinks(stored, mask=pick(0))


# ---- test_level_storage.py: put / defrag / fit mask of one storage group ----------------------------
def _col(values):
    return torch.tensor([[float(v)] for v in values], device=DEV)


def test_uniform_group_put_defrag_and_fit_mask():
    """test/data/test_level_storage.py:283-452 restated for ``UniformGroup``."""
    from nvalchemi_amd.data import UniformGroup

    src = UniformGroup({"a": _col([1, 2, 3, 4])}, 4, DEV)
    dest = UniformGroup({"a": torch.zeros(4, 1, device=DEV)}, 4, DEV)
    dest.put(src, torch.tensor([True, False, True, False], device=DEV))
    assert dest["a"].view(-1).tolist() == [1.0, 3.0, 0.0, 0.0] and dest["a"].shape == (4, 1)
    assert src._copied_mask.tolist() == [True, False, True, False]
    src.defrag()
    assert len(src) == 2 and src["a"].view(-1).tolist() == [2.0, 4.0, 0.0, 0.0] and not hasattr(src, "_copied_mask")

    src = UniformGroup({"a": _col([1, 2])}, 2, DEV)
    dest = UniformGroup({"a": torch.zeros(2, 1, device=DEV)}, 2, DEV)
    copied = torch.zeros(2, dtype=torch.bool, device=DEV)
    dest.put(src, torch.tensor([True, True], device=DEV), copied_mask=copied)
    assert bool(copied.all()) and dest["a"].view(-1).tolist() == [1.0, 2.0]
    src.defrag(copied_mask=copied)
    assert len(src) == 0 and src["a"].shape == (2, 1)

    # only what fits: one empty slot, the first masked row takes it
    src = UniformGroup({"a": _col([1, 2, 3])}, 3, DEV)
    dest = UniformGroup({"a": torch.zeros(3, 1, device=DEV)}, 3, DEV)
    copied = torch.zeros(3, dtype=torch.bool, device=DEV)
    slots = torch.tensor([True, True, False], device=DEV)
    dest.put(src, torch.ones(3, dtype=torch.bool, device=DEV), copied_mask=copied, dest_mask=slots)
    assert copied.tolist() == [True, False, False] and float(dest["a"][2]) == 1.0 and slots.tolist() == [True] * 3

    # the fit mask says beforehand what put will move
    src = UniformGroup({"a": _col([1, 2, 3, 4])}, 4, DEV)
    dest = UniformGroup({"a": torch.zeros(4, 1, device=DEV)}, 4, DEV)
    fit = torch.zeros(4, dtype=torch.bool, device=DEV)
    dest.compute_put_per_system_fit_mask(src, torch.tensor([True, False, True, False], device=DEV), None, fit)
    assert fit.tolist() == [True, False, True, False]
    dest.put(src, fit)
    assert dest["a"].view(-1).tolist()[:2] == [1.0, 3.0]
    src = UniformGroup({"a": _col([1, 2, 3])}, 3, DEV)
    dest = UniformGroup({"a": torch.zeros(3, 1, device=DEV)}, 3, DEV)
    fit = torch.ones(3, dtype=torch.bool, device=DEV)
    dest.compute_put_per_system_fit_mask(src, torch.ones(3, dtype=torch.bool, device=DEV),
                                         torch.tensor([True, True, False], device=DEV), fit)
    assert fit.tolist() == [True, False, False]
    # several keys of one row land in one slot
    src = UniformGroup({"a": _col([1, 2, 3]), "b": 10 * _col([1, 2, 3])}, 3, DEV)
    dest = UniformGroup({"a": torch.zeros(3, 1, device=DEV), "b": torch.zeros(3, 1, device=DEV)}, 3, DEV)
    dest.put(src, torch.tensor([False, True, True], device=DEV))
    assert dest["a"].view(-1).tolist() == [2.0, 3.0, 0.0] and dest["b"].view(-1).tolist() == [20.0, 30.0, 0.0]
    with pytest.raises(ValueError, match="at least one common attribute"):
        dest.put(UniformGroup({"c": _col([1])}, 1, DEV), torch.tensor([True], device=DEV))


def test_segmented_group_put_defrag_and_fit_mask():
    """test/data/test_level_storage.py:737-930 restated for ``SegmentedGroup``."""
    from nvalchemi_amd.data import SegmentedGroup

    rows = lambda *v: torch.tensor([[float(x), 0.0] for x in v], device=DEV)  # noqa: E731
    src = SegmentedGroup({"x": rows(1, 2, 3, 4, 5)}, [2, 3], DEV)
    dest = SegmentedGroup({"x": torch.zeros(15, 2, device=DEV)}, [10], DEV, batch_ptr_capacity=5)
    dest.put(src, torch.tensor([True, True], device=DEV))
    assert len(dest) == 3 and dest.num_elements() == 15 and dest["x"].shape == (15, 2)
    assert torch.equal(dest["x"][10:15], src["x"]) and not dest["x"][:10].any()
    assert dest.batch_ptr.tolist() == [0, 10, 12, 15] and dest.lengths_list() == [10, 2, 3]
    assert bool(src._copied_mask.all())
    src.defrag()
    assert len(src) == 0 and src.num_elements() == 0 and src["x"].shape == (5, 2) and not src["x"].any()

    src = SegmentedGroup({"x": _col([1, 2, 3])}, [1, 2], DEV)
    dest = SegmentedGroup({"x": torch.zeros(10, 1, device=DEV)}, [0], DEV, batch_ptr_capacity=5)
    copied = torch.zeros(2, dtype=torch.bool, device=DEV)
    dest.put(src, torch.tensor([True, False], device=DEV), copied_mask=copied)
    assert copied.tolist() == [True, False] and len(dest) == 2 and float(dest["x"][0]) == 1.0
    src.defrag(copied_mask=copied)
    assert len(src) == 1 and src.num_elements() == 2 and src["x"].view(-1).tolist() == [2.0, 3.0, 0.0]
    assert src.batch_idx.tolist() == [0, 0]

    # the fit mask, with and without headroom in the boundaries
    src = SegmentedGroup({"x": _col([1, 2, 3, 4, 5])}, [2, 3], DEV)
    dest = SegmentedGroup({"x": torch.zeros(15, 1, device=DEV)}, [10], DEV, batch_ptr_capacity=5)
    fit = torch.zeros(2, dtype=torch.bool, device=DEV)
    dest.compute_put_per_system_fit_mask(src, torch.tensor([True, True], device=DEV), None, fit)
    assert fit.tolist() == [True, True]
    dest.put(src, fit)
    assert len(dest) == 3 and torch.equal(dest["x"][10:15], src["x"])
    tight = SegmentedGroup({"x": torch.zeros(10, 1, device=DEV)}, [0], DEV)
    fit = torch.ones(1, dtype=torch.bool, device=DEV)
    tight.compute_put_per_system_fit_mask(SegmentedGroup({"x": _col([1, 2])}, [2], DEV),
                                          torch.tensor([True], device=DEV), None, fit)
    assert fit.tolist() == [False]

    # room for the first segment only
    src = SegmentedGroup({"x": _col([1, 2, 3, 4, 5])}, [2, 3], DEV)
    dest = SegmentedGroup({"x": torch.zeros(12, 1, device=DEV)}, [10], DEV, batch_ptr_capacity=5)
    copied = torch.zeros(2, dtype=torch.bool, device=DEV)
    dest.put(src, torch.tensor([True, True], device=DEV), copied_mask=copied)
    assert copied.tolist() == [True, False] and dest["x"].view(-1).tolist()[10:] == [1.0, 2.0] and len(dest) == 2
