"""``SizeAwareSampler`` (nvalchemi/dynamics/sampler.py:36-641): host logic, no kernel.

The cases are the reference's own (test/dynamics/test_sampler.py:110-1085), restated over the same
kind of mock dataset, with the expectations tightened to the exact samples where the stated
algorithm (round-robin over ascending bins for the first batch, largest bin first for budgeted
replacements, the slot's bin downwards for a slot replacement) fixes them.
"""

import random

import pytest
import torch

from nvalchemi_amd.data import AtomicData
from nvalchemi_amd.dynamics.sampler import SizeAwareSampler


class MockDataset:
    def __init__(self, samples):
        self.samples = samples
        self.loaded = []

    def __len__(self):
        return len(self.samples)

    def get_metadata(self, index):
        return self.samples[index]

    def __getitem__(self, index):
        n, e = self.samples[index]
        self.loaded.append(index)
        data = AtomicData(torch.randn(n, 3), torch.arange(1, n + 1, dtype=torch.long))
        if e > 0:
            data.neighbor_list = torch.stack([torch.randint(0, n, (e,)), torch.randint(0, n, (e,))], dim=1)
        return data, {}


def make(samples, **kw):
    ds = MockDataset(samples)
    return ds, SizeAwareSampler(dataset=ds, **kw)


def test_construction_and_validation():
    ds, s = make([(10, 20), (15, 30), (8, 16), (12, 24), (5, 10)], max_atoms=100, max_edges=200, max_batch_size=10)
    assert len(s) == 5 and not s.exhausted and (s.max_atoms, s.max_edges, s.max_batch_size) == (100, 200, 10)
    assert ds.loaded == []  # the scan reads sizes only
    with pytest.raises(RuntimeError, match="exceeding max_atoms=40"):
        make([(10, 20), (50, 30)], max_atoms=40, max_edges=100, max_batch_size=4)
    with pytest.raises(RuntimeError, match="exceeding max_edges=25"):
        make([(10, 20), (10, 30)], max_atoms=40, max_edges=25, max_batch_size=4)
    make([(10, 20), (5000, 30)], max_atoms=None, max_edges=100, max_batch_size=4)
    make([(10, 20), (10, 3000)], max_atoms=100, max_edges=None, max_batch_size=4)
    for bad in (0, -1):
        with pytest.raises(ValueError, match="max_batch_size must be >= 1"):
            make([(1, 1)], max_atoms=10, max_batch_size=bad)
    with pytest.raises(ValueError, match="At least one of max_atoms or max_batch_size"):
        make([(1, 1)])
    make([(1, 1)], max_batch_size=2)
    make([(1, 1)], max_atoms=2)
    with pytest.raises(ValueError, match="bin_width must be >= 1"):
        make([(1, 1)], max_atoms=10, bin_width=0)
    for bad in (0.0, -0.5, 1.5):
        with pytest.raises(ValueError, match="max_gpu_memory_fraction"):
            make([(1, 1)], max_atoms=10, max_gpu_memory_fraction=bad)
    make([(1, 1)], max_atoms=10, max_gpu_memory_fraction=1.0)

    class NoLen:
        def __getitem__(self, i): ...
        def get_metadata(self, i): ...

    class NoGet:
        def __len__(self): return 0
        def get_metadata(self, i): ...

    class NoMeta:
        def __len__(self): return 0
        def __getitem__(self, i): ...

    for cls, what in ((NoLen, "__len__"), (NoGet, "__getitem__"), (NoMeta, "get_metadata")):
        with pytest.raises(TypeError, match=what):
            SizeAwareSampler(dataset=cls(), max_atoms=10)
    if not torch.cuda.is_available():
        assert s._estimate_max_atoms_from_gpu() is None


def test_first_batch_round_robin_over_bins():
    # atoms limit: bins 10, 20, 30 give one each -> 60 > 55 at the third, so 10 + 20; second round: nothing fits
    ds, s = make([(10, 5), (20, 10), (30, 15), (40, 20), (50, 25)], max_atoms=55, max_edges=1000, max_batch_size=10)
    b = s.build_initial_batch()
    assert b.num_nodes_list == [10, 20] and ds.loaded == [0, 1] and len(s) == 3
    assert b.status.shape == (2, 1) and b.status.dtype == torch.long and not b.status.any()
    assert b.system_id.view(-1).tolist() == [0, 1]
    # edges limit: one bin, samples in order while their edges fit: 10 + 20 = 30, then 30 and 40 and 50 do not
    ds, s = make([(5, 10), (5, 20), (5, 30), (5, 40), (5, 50)], max_atoms=1000, max_edges=55, max_batch_size=10)
    assert s.build_initial_batch().num_edges_list == [10, 20] and ds.loaded == [0, 1]
    # count limit
    ds, s = make([(5, 10)] * 10, max_atoms=1000, max_edges=1000, max_batch_size=3)
    assert s.build_initial_batch().num_graphs == 3 and len(s) == 7
    # all three at once: bins ascending 6, 8 -> two systems
    ds, s = make([(10, 20), (15, 30), (8, 16), (12, 24), (6, 12)], max_atoms=30, max_edges=60, max_batch_size=2)
    assert s.build_initial_batch().num_nodes_list == [6, 8]
    # every size is represented; order: one per bin per round
    ds, s = make([(15, 30), (12, 24), (5, 10), (5, 10), (5, 10), (12, 24)], max_atoms=100, max_edges=200,
                 max_batch_size=10)
    assert s.build_initial_batch().num_nodes_list == [5, 12, 15, 5, 12, 5] and s.exhausted
    # a tight budget still mixes sizes: 5 + 12, then 15 does not fit, next round nothing fits
    ds, s = make([(5, 10), (5, 10), (5, 10), (12, 24), (15, 30)], max_atoms=20, max_edges=100, max_batch_size=10)
    assert s.build_initial_batch().num_nodes_list == [5, 12]
    ds, s = make([(5, 10)], max_atoms=100, max_edges=100, max_batch_size=10)
    s.build_initial_batch()
    with pytest.raises(RuntimeError, match="no samples available"):
        s.build_initial_batch()
    # a wide bin holds everything
    ds, s = make([(5, 10), (10, 20), (15, 30), (20, 40), (25, 50)], max_atoms=1000, max_edges=1000,
                 max_batch_size=10, bin_width=100)
    assert s.build_initial_batch().num_nodes_list == [5, 10, 15, 20, 25]


def test_slot_replacement_searches_from_the_slots_bin_downwards():
    samples = [(10, 20), (15, 30), (8, 16), (12, 24), (5, 10)]
    ds, s = make(samples, max_atoms=100, max_edges=100, max_batch_size=2)
    assert s.build_initial_batch().num_nodes_list == [5, 8]
    r = s.request_replacement(num_atoms=15, num_edges=30)
    assert r.num_nodes == 15 and int(r.system_id) == 2 and r.level_of("system_id") == "system"
    assert s.request_replacement(num_atoms=11, num_edges=30).num_nodes == 10
    assert s.request_replacement(num_atoms=11, num_edges=30) is None
    assert s.request_replacement(num_atoms=12, num_edges=23) is None  # the edges do not fit
    assert s.request_replacement(num_atoms=12, num_edges=24).num_nodes == 12 and s.exhausted
    assert s.request_replacement(num_atoms=100, num_edges=100) is None

    ds, s = make([(20, 40)] * 3, max_atoms=100, max_edges=100, max_batch_size=1)
    s.build_initial_batch()
    assert s.request_replacement(num_atoms=5, num_edges=10) is None and len(s) == 2

    ds, s = make([(30, 60), (25, 50), (15, 30), (5, 10)], max_atoms=100, max_edges=100, max_batch_size=1, bin_width=10)
    assert s.build_initial_batch().num_nodes == 5
    assert s.request_replacement(num_atoms=20, num_edges=40).num_nodes == 15

    ds, s = make([(5, 10), (5, 10), (10, 20)], max_atoms=100, max_edges=100, max_batch_size=1)
    s.build_initial_batch()
    assert len(s) == 2
    assert s.request_replacement(num_atoms=10, num_edges=20).num_nodes == 10 and len(s) == 1
    assert s.request_replacement(num_atoms=10, num_edges=20).num_nodes == 5 and len(s) == 0 and s.exhausted

    ds, s = make([(1, 2), (2, 4), (3, 6), (4, 8), (5, 10)], max_atoms=100, max_edges=100, max_batch_size=1)
    assert s.build_initial_batch().num_nodes == 1
    for want in (2, 3, 4, 5):
        assert s.request_replacement(num_atoms=want, num_edges=100).num_nodes == want


def test_budgeted_replacements_take_the_largest_first():
    ds, s = make([(5, 0), (10, 0), (20, 0), (50, 0)], max_atoms=200, max_batch_size=10)
    got = s.request_replacements_budget(atom_budget=60, max_count=5)
    assert [r.num_nodes for r in got] == [50, 10] and [int(r.system_id) for r in got] == [0, 1]
    assert [r.num_nodes for r in s.request_replacements_budget(atom_budget=60)] == [20, 5] and s.exhausted
    assert s.request_replacements_budget() == []
    ds, s = make([(5, 0)] * 20, max_atoms=200, max_batch_size=20)
    assert len(s.request_replacements_budget(atom_budget=100, max_count=3)) == 3 and ds.loaded == [0, 1, 2]
    assert s.request_replacements_budget(atom_budget=100, max_count=0) == []
    ds, s = make([(10, 0)] * 10, max_atoms=200, max_batch_size=20)
    assert len(s.request_replacements_budget(atom_budget=35)) == 3
    ds, s = make([(50, 0), (5, 0)], max_atoms=100, max_batch_size=10)
    assert [r.num_nodes for r in s.request_replacements_budget(atom_budget=55)] == [50, 5]
    ds, s = make([(5, 4), (5, 9), (6, 3)], max_atoms=100, max_batch_size=10)
    assert [(r.num_nodes, r.neighbor_list.shape[0]) for r in s.request_replacements_budget(edge_budget=8)] == \
        [(6, 3), (5, 4)]


def test_vectorised_slot_replacements_take_the_lowest_fitting_index():
    ds, s = make([(10, 20), (15, 30), (8, 16), (12, 24), (5, 10)], max_atoms=100, max_edges=100, max_batch_size=1)
    assert s.build_initial_batch().num_nodes == 5
    got = s.request_replacements(torch.tensor([12, 12, 9, 4]), torch.tensor([100, 100, 100, 100]))
    assert [None if r is None else r.num_nodes for r in got] == [10, 8, None, None]
    assert len(s) == 2 and sorted(s) == [1, 3]
    # the host-side searches see what the vectorised one handed out, and the other way round
    assert s.request_replacement(num_atoms=12, num_edges=100).num_nodes == 12
    got = s.request_replacements(torch.tensor([20]), torch.tensor([29]))
    assert got == [None]
    assert s.request_replacements(torch.tensor([20]), torch.tensor([30]))[0].num_nodes == 15 and s.exhausted


def test_iteration_length_and_shuffle():
    ds, s = make([(5, 10), (15, 30), (5, 10), (25, 50)], max_atoms=100, max_edges=100, max_batch_size=1, bin_width=10)
    assert list(s) == [0, 2, 1, 3] and len(s) == 4
    s.build_initial_batch()
    assert list(s) == [2, 1, 3] and len(s) == 3 and not s.exhausted
    orders = set()
    for _ in range(3):
        orders.add(tuple(make([(5, 10)] * 10, max_atoms=100, max_batch_size=1, bin_width=10)[1]))
    assert orders == {tuple(range(10))}
    # shuffling permutes inside a bin only, by Python's generator: the same seed, the same order
    samples = [(5, 10)] * 6 + [(25, 10)] * 6
    seen = []
    for seed in (0, 1, 0):
        random.seed(seed)
        seen.append(list(make(samples, max_atoms=100, max_batch_size=1, bin_width=10, shuffle=True)[1]))
    assert seen[0] == seen[2] and seen[0] != seen[1]
    for order in seen:
        assert sorted(order[:6]) == list(range(6)) and sorted(order[6:]) == list(range(6, 12))
    random.seed(0)
    expect = [list(range(6)), list(range(6, 12))]
    for members in expect:
        random.shuffle(members)
    assert seen[0] == expect[0] + expect[1]
