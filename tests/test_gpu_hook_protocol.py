"""The reference's own behavioural cases for ``NeighborListHook``, restated against this package
(test/hooks/test_neighbor_list_hook.py: ``TestShapeInvalidation`` :539-608, ``TestAdaptiveK``
:946-1029, ``TestStaleCOOEntries`` :1031-1100, with its builders ``_line_batch`` :63-90 and
``_pbc_wrap_batch`` :91-104).  Same inputs, same expected results; buffers that only the
reference's implementation has (staging copies) are not asserted."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CUTOFF = 2.5


def cfg(cutoff=CUTOFF, fmt=None, half_list=False):
    from nvalchemi_amd.models.base import NeighborConfig, NeighborListFormat

    return NeighborConfig(cutoff=cutoff, format=fmt or NeighborListFormat.MATRIX, half_list=half_list)


def ctx(batch):
    from nvalchemi_amd.hooks._context import HookContext

    return HookContext(batch=batch)


def stage():
    from nvalchemi_amd.dynamics import DynamicsStage

    return DynamicsStage.BEFORE_COMPUTE


def line_batch(pbc=False, n_graphs=1, cell_size=20.0):
    from nvalchemi_amd.data import AtomicData, Batch

    data = []
    for _ in range(n_graphs):
        kw = {}
        if pbc:
            kw["cell"] = torch.eye(3) * cell_size
            kw["pbc"] = torch.tensor([True, True, True])
        data.append(AtomicData(torch.tensor([[0.0, 0, 0], [1.5, 0, 0], [5.0, 0, 0]]), torch.tensor([1, 1, 1]), **kw))
    return Batch.from_data_list(data, device=DEV)


def random_batch(n):
    from nvalchemi_amd.data import AtomicData, Batch

    return Batch.from_data_list([AtomicData(torch.rand(n, 3), torch.ones(n, dtype=torch.long))], device=DEV)


def hook(**kw):
    from nvalchemi_amd.hooks import NeighborListHook

    config = kw.pop("config", None) or cfg()
    return NeighborListHook(config, stage=stage(), **kw)


def is_neighbor(nm, nn, i, j):
    return j in nm[i, : int(nn[i])].tolist()


def test_line_and_wrap_batches_give_the_reference_topology():
    from nvalchemi_amd.data import AtomicData, Batch

    b = line_batch()
    hook()(ctx(b), stage())
    assert is_neighbor(b.neighbor_matrix, b.num_neighbors, 0, 1) and is_neighbor(b.neighbor_matrix, b.num_neighbors, 1, 0)
    assert int(b.num_neighbors[2]) == 0 and "neighbor_matrix_shifts" not in b
    two = line_batch(n_graphs=2)
    hook()(ctx(two), stage())
    assert is_neighbor(two.neighbor_matrix, two.num_neighbors, 3, 4) and not is_neighbor(two.neighbor_matrix, two.num_neighbors, 1, 3)
    w = Batch.from_data_list([AtomicData(torch.tensor([[0.1, 0, 0], [2.9, 0, 0]]), torch.tensor([1, 1]),
                                         cell=torch.eye(3) * 3.0, pbc=torch.tensor([True, True, True]))], device=DEV)
    hook()(ctx(w), stage())
    assert is_neighbor(w.neighbor_matrix, w.num_neighbors, 0, 1)
    k = w.neighbor_matrix[0, : int(w.num_neighbors[0])].tolist().index(1)
    assert w.neighbor_matrix_shifts[0, k].tolist() == [-1, 0, 0]
    assert w._neighbor_list_cutoff == CUTOFF


def test_shape_changes_reallocate_and_reset_the_skin_reference():
    h = hook()
    small = line_batch()
    h(ctx(small), stage())
    assert h._alloc_N == 3 and h._alloc_B == 1
    matrix = h._neighbor_matrix
    h(ctx(small), stage())
    assert h._neighbor_matrix is matrix  # same shape: the same buffers
    h(ctx(random_batch(5)), stage())
    assert h._alloc_N == 5 and h._neighbor_matrix.shape[0] == 5
    h(ctx(line_batch(n_graphs=2)), stage())
    assert h._alloc_B == 2 and h._alloc_N == 6
    s = hook(skin=0.5)
    s(ctx(small), stage())
    assert s._ref_positions is not None and s._ref_positions.shape == (3, 3)
    s(ctx(random_batch(5)), stage())
    assert s._ref_positions is not None and s._ref_positions.shape == (5, 3)


def test_adaptive_k():
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.neighbors import compute_neighbors

    three = Batch.from_data_list([AtomicData(torch.tensor([[0.0, 0, 0], [1.0, 0, 0], [2.0, 0, 0]]),
                                             torch.tensor([1, 1, 1]))], device=DEV)
    h = hook(config=cfg(cutoff=100.0))
    h(ctx(three), stage())
    assert h._max_neighbors <= 16  # non-periodic: capped at ceil16(largest system)
    pair = Batch.from_data_list([AtomicData(torch.tensor([[0.0, 0, 0], [1.0, 0, 0]]), torch.tensor([1, 1]),
                                            cell=torch.eye(3) * 3.0, pbc=torch.tensor([True, True, True]))], device=DEV)
    h = hook(config=cfg(cutoff=6.0))
    h(ctx(pair), stage())
    assert h._max_neighbors > 1 and int(h._num_neighbors.max()) < h._max_neighbors  # images: no cap
    four = Batch.from_data_list([AtomicData(torch.tensor([[0.0, 0, 0], [1.0, 0, 0], [2.0, 0, 0], [3.0, 0, 0]]),
                                            torch.ones(4, dtype=torch.long))], device=DEV)
    h = hook(config=cfg(cutoff=5.0), max_neighbors=100)
    h(ctx(four), stage())
    assert h._max_neighbors < 100 and h._neighbor_matrix.shape[1] == h._max_neighbors
    assert int(h._num_neighbors.max()) <= 3
    b = Batch.from_data_list([AtomicData(torch.tensor([[0.0, 0, 0], [1.0, 0, 0], [2.0, 0, 0]]), torch.tensor([1, 1, 1]),
                                         forces=torch.zeros(3, 3), energy=torch.zeros(1, 1))], device=DEV)
    compute_neighbors(b, cutoff=100.0)
    assert b.neighbor_matrix.shape[1] <= 16


def test_shrinking_neighbors_leave_no_stale_coo_edges():
    from nvalchemi_amd.hooks import NeighborListHook
    from nvalchemi_amd.models.base import NeighborListFormat

    h = NeighborListHook(cfg(fmt=NeighborListFormat.COO), skin=1.0, stage=stage())
    b = line_batch()
    h(ctx(b), stage())
    before = {tuple(r) for r in b.neighbor_list.cpu().tolist()}
    b.positions[1, 0] = 4.0  # 4.0 from atom 0 (beyond cutoff + skin), 1.0 from atom 2; moved 2.5 > skin / 2
    h(ctx(b), stage())
    after = {tuple(r) for r in b.neighbor_list.cpu().tolist()}
    assert (0, 1) in before and (1, 0) in before
    assert (0, 1) not in after and (1, 0) not in after and (1, 2) in after and (2, 1) in after
    counts = torch.bincount(b.neighbor_list[:, 0].cpu().long(), minlength=b.num_nodes)
    assert torch.equal(counts, h._num_neighbors.cpu().long())


def test_a_cell_too_thin_for_the_search_is_refused_not_truncated():
    """The search looks at 32 periodic images per axis and direction at most.  A cell thinner than
    cutoff / 32 used to give a truncated list with an OK status; the build now reports it in its
    status bits, and the callers that wait for the device anyway raise."""
    from nvalchemi_amd import _lib
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.neighbors import compute_neighbors

    thin = Batch.from_data_list([AtomicData(torch.tensor([[0.0, 0, 0], [0.01, 0.5, 0.5]]), torch.tensor([1, 1]),
                                            cell=torch.diag(torch.tensor([0.05, 4.0, 4.0])),
                                            pbc=torch.tensor([True, True, True]))], device=DEV)
    with pytest.raises(ValueError, match="thinner than cutoff / 32"):
        compute_neighbors(thin, cutoff=2.0)
    with pytest.raises(ValueError, match="thinner than cutoff / 32"):
        hook(config=cfg(cutoff=2.0))(ctx(thin), stage())
    # a cell of ordinary proportions clears the bit of the last build; the accumulated bits keep it until read
    ok = line_batch(pbc=True)
    compute_neighbors(ok, cutoff=2.5)
    st = _lib.nl_status(ok.num_nodes, ok.num_graphs, ok.positions.device).tolist()
    assert st[0] == 0


def test_rows_that_overflow_after_the_first_build_leave_a_flag():
    """After its first build the reference's hook never compares counts with K again
    (nvalchemi/hooks/neighbor_list.py:351-355).  The kernels count past K on the device and leave a
    bit in the workspace; ``overflowed()`` reads it."""
    from nvalchemi_amd.data import AtomicData, Batch

    g = torch.Generator().manual_seed(3)
    pos = torch.rand(64, 3, generator=g) * 6.0
    b = Batch.from_data_list([AtomicData(pos, torch.ones(64, dtype=torch.long), cell=torch.eye(3) * 6.0,
                                         pbc=torch.tensor([True, True, True]))], device=DEV)
    h = hook(config=cfg(cutoff=2.5))
    h(ctx(b), stage())
    assert not h.overflowed()
    K = h._max_neighbors
    # squeeze every atom into a corner of the cell: every row now wants 63 neighbors or more
    b.positions.mul_(0.05)
    h(ctx(b), stage())
    if int(h._num_neighbors.max()) > K:
        assert h.overflowed()
        assert not h.overflowed()  # (read and cleared)
    h(ctx(b), stage())
    assert h.overflowed() == (int(h._num_neighbors.max()) > K)


def test_status_bits_survive_a_regrown_workspace(monkeypatch):
    """The accumulated status bits live in the header of the per-stream workspace.  A larger build makes the
    package replace that buffer: the new one takes the old header over, so an overflow recorded through the
    smaller buffer is still reported afterwards."""
    from nvalchemi_amd import _lib

    monkeypatch.setattr(_lib, "workspaces", _lib._Workspaces())
    dev = torch.device(DEV)

    def build(n, K, box):
        g = torch.Generator().manual_seed(n)
        pos = (torch.rand(n, 3, generator=g) * box).to(dev)
        cell = (torch.eye(3) * box).reshape(1, 3, 3).to(dev)
        pbc = torch.ones(1, 3, dtype=torch.bool, device=dev)
        ptr = torch.tensor([0, n], dtype=torch.int32, device=dev)
        bidx = torch.zeros(n, dtype=torch.int32, device=dev)
        nm = torch.full((n, K), n, dtype=torch.int32, device=dev)
        nn = torch.zeros(n, dtype=torch.int32, device=dev)
        sh = torch.zeros(n, K, 3, dtype=torch.int32, device=dev)
        _lib.nl_build(pos, cell, pbc, ptr, bidx, None, 2.5, K, False, 0, nm, nn, sh)
        return nn

    _lib.nl_status(64, 1, dev, clear=True)
    nn = build(64, 4, 4.0)  # 64 atoms in a 4 A box: far more than 4 neighbors each
    assert int(nn.max()) > 4
    small = _lib.workspaces.get(dev, "nl", 1).numel()
    nn = build(20000, 64, 60.0)  # a dilute box through a much larger workspace: no overflow of its own
    assert int(nn.max()) <= 64
    assert _lib.workspaces.get(dev, "nl", 1).numel() > small
    st = _lib.nl_status(20000, 1, dev).tolist()
    assert st[0] == 0 and st[1] & 2  # NVAMD_NL_STATUS_ROW_OVERFLOW of the earlier build
