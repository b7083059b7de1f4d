"""HIP neighbor filters against the numpy oracle, through the package's mirror of
nvalchemi/models/_ops/neighbor_filter.py: the reference's cases, random periodic batches (lists
built with a skin and filtered to the bare cutoff must equal lists built at the bare cutoff), rows
wider than one wavefront, and prepare_neighbors_for_model on a batch."""

import numpy as np
import pytest
import torch

import oracle
from _systems import periodic_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return None if a is None else torch.as_tensor(np.ascontiguousarray(a), device=DEV)


def N_(t):
    return None if t is None else t.cpu().numpy()


def canonical(nm, nn, sh):
    K = nm.shape[1]
    ii, kk = np.nonzero(np.arange(K)[None, :] < nn[:, None])
    rows = np.concatenate([ii[:, None], nm[ii, kk][:, None], sh[ii, kk]], axis=1).astype(np.int64)
    return rows[np.lexsort(rows.T[::-1])]


def test_reference_cases():
    from nvalchemi_amd.models._ops import neighbor_filter as nf

    pos = np.array([[0.0, 0, 0], [1.0, 0, 0], [3.0, 0, 0], [5.0, 0, 0]], dtype=np.float32)
    nm = np.array([[1, 2, 4], [0, 2, 4], [0, 1, 4], [4, 4, 4]], dtype=np.int32)
    nn = np.array([2, 2, 2, 0], dtype=np.int32)
    sh = np.zeros((4, 3, 3), np.int32)
    sh[..., 0] = np.arange(12).reshape(4, 3)
    for rc in (0.1, 1.5, 2.5, 10.0):
        for shifts in (None, sh):
            got = nf.filter_neighbor_matrix(T(pos), rc, T(nm), T(nn), 4, neighbor_matrix_shifts=T(shifts))
            want = oracle.filter_neighbor_matrix(pos, rc, nm, nn, 4, neighbor_matrix_shifts=shifts)
            for g, w in zip(got, want):
                assert (g is None and w is None) or np.array_equal(N_(g), w)
    # the image pair through a 5 A cell, single cell and per-system cells
    pos = np.array([[0.0, 0, 0], [4.5, 0, 0], [0.0, 0, 0], [1.0, 0, 0]], dtype=np.float32)
    cells = np.stack([5.0 * np.eye(3), 10.0 * np.eye(3)]).astype(np.float32)
    nm = np.array([[1, 4], [0, 4], [3, 4], [2, 4]], dtype=np.int32)
    sh = np.zeros((4, 2, 3), np.int32)
    sh[0, 0], sh[1, 0] = [-1, 0, 0], [1, 0, 0]
    bi = np.array([0, 0, 1, 1], np.int32)
    _, cnt, _ = nf.filter_neighbor_matrix(T(pos), 2.0, T(nm), torch.ones(4, dtype=torch.int32, device=DEV), 4,
                                          cell=T(cells), neighbor_matrix_shifts=T(sh), batch_idx=T(bi))
    assert cnt.tolist() == [1, 1, 1, 1]
    _, cnt, _ = nf.filter_neighbor_matrix(T(pos[:2]), 2.0, T(np.array([[1, 2], [0, 2]], np.int32)),
                                          torch.ones(2, dtype=torch.int32, device=DEV), 2, cell=T(cells[0]),
                                          neighbor_matrix_shifts=T(sh[:2]))
    assert cnt.tolist() == [1, 1]
    with pytest.raises(ValueError):
        nf.filter_neighbor_matrix(T(pos), 2.0, T(nm), torch.ones(4, dtype=torch.int32, device=DEV), 4, cell=T(cells),
                                  neighbor_matrix_shifts=T(sh))
    # COO
    nl = np.array([[0, 1], [0, 2], [1, 0], [1, 2], [2, 0], [2, 1]], dtype=np.int32)
    ptr = np.array([0, 2, 4, 6, 6], dtype=np.int32)
    chain = np.array([[0.0, 0, 0], [1.0, 0, 0], [3.0, 0, 0], [5.0, 0, 0]], dtype=np.float32)
    for rc in (0.1, 1.5, 2.5, 10.0):
        got = nf.filter_neighbor_list(T(chain), rc, T(nl), T(ptr))
        want = oracle.filter_neighbor_list(chain, rc, nl, ptr)
        assert np.array_equal(N_(got[0]), want[0]) and np.array_equal(N_(got[1]), want[1]) and got[2] is None


@pytest.mark.parametrize("name,kw,rc_list,rc,K", [
    ("liquid", dict(n_systems=4, n_lo=100, n_hi=400, density=0.8), 3.0, 2.5, 160),
    ("triclinic, unwrapped", dict(n_systems=5, n_lo=10, n_hi=120, density=0.05, triclinic=True, spread=1.5), 7.0, 5.0, 160),
    ("rows wider than a wavefront", dict(n_systems=2, n_lo=200, n_hi=300, density=0.9), 3.6, 3.0, 288),
])
def test_filtering_a_skin_list_gives_the_bare_list(name, kw, rc_list, rc, K):
    from nvalchemi_amd.models._ops import neighbor_filter as nf

    P, C, pb, ptr = periodic_batch(seed=91, **kw)
    bi = oracle.batch_idx_from_ptr(ptr)
    N = len(P)
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc_list, K)
    assert nn.max() < K
    got = nf.filter_neighbor_matrix(T(P), rc, T(nm), T(nn), N, cell=T(C), neighbor_matrix_shifts=T(sh), batch_idx=T(bi))
    want = oracle.filter_neighbor_matrix(P, rc, nm, nn, N, cell=C, neighbor_matrix_shifts=sh, batch_idx=bi)
    for g, w in zip(got, want):
        assert np.array_equal(N_(g), w), name
    bare = oracle.nl_cell(P, C, pb, ptr, rc, K)
    assert np.array_equal(canonical(N_(got[0]), N_(got[1]), N_(got[2])), canonical(bare[0], bare[1], bare[2]))
    # the same through COO: matrix -> list, then the list filter
    nl, eptr, nls = nf.neighbor_matrix_to_list(T(nm), T(nn), N, T(sh))
    w_nl, w_ptr, w_sh = oracle.neighbor_matrix_to_list(nm, nn, N, sh)
    assert np.array_equal(N_(nl), w_nl) and np.array_equal(N_(eptr), w_ptr) and np.array_equal(N_(nls), w_sh)
    f_nl, f_ptr, f_sh = nf.filter_neighbor_list(T(P), rc, nl, eptr, cell=T(C), neighbor_list_shifts=nls, batch_idx=T(bi))
    o_nl, o_ptr, o_sh = oracle.filter_neighbor_list(P, rc, w_nl, w_ptr, cell=C, neighbor_list_shifts=w_sh, batch_idx=bi)
    assert np.array_equal(N_(f_nl), o_nl) and np.array_equal(N_(f_ptr), o_ptr) and np.array_equal(N_(f_sh), o_sh)
    l2, p2, s2 = nf.neighbor_matrix_to_list(*got[:2], N, got[2])
    assert np.array_equal(N_(l2), o_nl) and np.array_equal(N_(p2), o_ptr) and np.array_equal(N_(s2), o_sh)


def test_prepare_neighbors_for_model_on_a_batch():
    """A batch whose list was built at 6 A serves a 4 A model in both formats; without the stamp,
    or with an equal cutoff, nothing is filtered (nvalchemi/models/_ops/neighbor_filter.py:336-338)."""
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.models._ops.neighbor_filter import prepare_neighbors_for_model
    from nvalchemi_amd.models.base import NeighborListFormat
    from nvalchemi_amd.neighbors import compute_neighbors

    P, C, pb, ptr = periodic_batch(seed=93, n_systems=3, n_lo=30, n_hi=80, density=0.06)
    data = [AtomicData(torch.from_numpy(P[a:b]), torch.full((b - a,), 18), cell=torch.from_numpy(C[s]),
                       pbc=torch.from_numpy(pb[s])) for s, (a, b) in enumerate(zip(ptr[:-1], ptr[1:]))]
    batch = Batch.from_data_list(data, device=DEV)
    compute_neighbors(batch, cutoff=6.0, format=NeighborListFormat.MATRIX)
    N = len(P)
    bare = oracle.nl_cell(P, C, pb, ptr, 4.0, 128)
    out = prepare_neighbors_for_model(batch, 4.0, NeighborListFormat.MATRIX, N)
    assert set(out) == {"neighbor_matrix", "num_neighbors", "neighbor_matrix_shifts"}
    assert np.array_equal(canonical(N_(out["neighbor_matrix"]), N_(out["num_neighbors"]), N_(out["neighbor_matrix_shifts"])),
                          canonical(*bare))
    coo = prepare_neighbors_for_model(batch, 4.0, NeighborListFormat.COO, N)
    assert set(coo) == {"neighbor_list", "edge_ptr", "neighbor_list_shifts"}
    assert coo["neighbor_list"].shape == (int(bare[1].sum()), 2) and int(coo["edge_ptr"][-1]) == int(bare[1].sum())
    same = prepare_neighbors_for_model(batch, 6.0, NeighborListFormat.MATRIX, N)
    assert same["neighbor_matrix"] is batch.neighbor_matrix
    object.__setattr__(batch, "_neighbor_list_cutoff", None)
    assert prepare_neighbors_for_model(batch, 4.0, NeighborListFormat.MATRIX, N)["neighbor_matrix"] is batch.neighbor_matrix
    empty = Batch.from_data_list(data, device=DEV)
    with pytest.raises(RuntimeError):
        prepare_neighbors_for_model(empty, 4.0, NeighborListFormat.MATRIX, N)
    with pytest.raises(RuntimeError):
        prepare_neighbors_for_model(empty, 4.0, NeighborListFormat.COO, N)
