"""Pins the oracle's neighbor functions (CPU only).

Known answers restate, as facts, the hand geometries of the reference's tests
(test/hooks/test_neighbor_list_hook.py:65-105,630-719 and
test/models/test_neighbor_filter.py:182-215); the rest are lattice coordination numbers,
invariants and brute force.
"""

import numpy as np
import pytest

import oracle
from _systems import fcc_boxes, molecules_batch, periodic_batch, ptr_from_counts


def _edges(*rows):
    return oracle.canonical_edges(np.array(rows, dtype=np.int64).reshape(-1, 5))


LINE = np.array([[0.0, 0, 0], [1.5, 0, 0], [5.0, 0, 0]], dtype=np.float32)


def test_line_three_atoms_non_periodic():
    e = oracle.nl_brute(LINE, None, None, [0, 3], 2.5)
    assert np.array_equal(e, _edges([0, 1, 0, 0, 0], [1, 0, 0, 0, 0]))


def test_line_three_atoms_big_periodic_cell():
    cell = np.eye(3, dtype=np.float32)[None] * 20.0
    e = oracle.nl_brute(LINE, cell, np.ones((1, 3), bool), [0, 3], 2.5)
    assert np.array_equal(e, _edges([0, 1, 0, 0, 0], [1, 0, 0, 0, 0]))


def test_two_graphs_do_not_mix():
    pos = np.concatenate([LINE, LINE])
    e = oracle.nl_brute(pos, None, None, [0, 3, 6], 2.5)
    assert np.array_equal(e, _edges([0, 1, 0, 0, 0], [1, 0, 0, 0, 0], [3, 4, 0, 0, 0], [4, 3, 0, 0, 0]))


def test_neighbor_only_through_periodic_image():
    pos = np.array([[0.1, 0, 0], [2.9, 0, 0]], dtype=np.float32)
    cell = np.eye(3, dtype=np.float32)[None] * 3.0
    e = oracle.nl_brute(pos, cell, np.ones((1, 3), bool), [0, 2], 2.5)
    assert np.array_equal(e, _edges([0, 1, -1, 0, 0], [1, 0, 1, 0, 0]))
    assert len(oracle.nl_brute(pos, None, None, [0, 2], 2.5)) == 0
    # pbc switched off on x only: the image is not used
    pbc = np.array([[False, True, True]])
    assert len(oracle.nl_brute(pos, cell, pbc, [0, 2], 2.5)) == 0


def test_shift_sign_convention():
    # atom0 at 0, atom1 at 4.5, cell 5: row 0 sees atom 1 through (-1,0,0), row 1 through (+1,0,0)
    pos = np.array([[0.0, 0, 0], [4.5, 0, 0]], dtype=np.float32)
    cell = np.eye(3, dtype=np.float32)[None] * 5.0
    e = oracle.nl_brute(pos, cell, np.ones((1, 3), bool), [0, 2], 2.0)
    assert np.array_equal(e, _edges([0, 1, -1, 0, 0], [1, 0, 1, 0, 0]))


def test_strict_less_than_cutoff():
    pos = np.array([[0.0, 0, 0], [2.5, 0, 0]], dtype=np.float32)
    assert len(oracle.nl_brute(pos, None, None, [0, 2], 2.5)) == 0
    assert len(oracle.nl_brute(pos, None, None, [0, 2], 2.5000001)) == 2


def test_fcc_coordination_shells():
    # perfect FCC a=3.6: shells at a/sqrt2 (12), a (6), a*sqrt(1.5) (24), a*sqrt2 (12),
    # a*sqrt(2.5) (24); a*sqrt3 = 6.235 is outside 6.0
    P, C, pb, ptr = fcc_boxes(seed=0, n_boxes=1, reps=4, a=3.6, jitter=0.0)
    for rc, z in ((3.0, 12), (4.0, 18), (5.0, 42), (5.5, 54), (6.0, 78)):
        e = oracle.nl_brute(P, C, pb, ptr, rc)
        counts = np.bincount(e[:, 0], minlength=len(P))
        assert np.all(counts == z), (rc, counts.min(), counts.max())


def test_self_images_in_a_small_cell():
    pos = np.zeros((1, 3), dtype=np.float32) + 0.3
    cell = np.eye(3, dtype=np.float32)[None] * 2.0
    pb = np.ones((1, 3), bool)
    e = oracle.nl_brute(pos, cell, pb, [0, 1], 2.5)
    assert len(e) == 6 and np.all(e[:, 0] == 0) and np.all(e[:, 1] == 0)
    assert np.all(np.abs(e[:, 2:]).sum(1) == 1)
    assert len(oracle.nl_brute(pos, cell, pb, [0, 1], 3.0)) == 18  # + 12 face diagonals
    h = oracle.nl_brute(pos, cell, pb, [0, 1], 2.5, half=True)
    assert len(h) == 3


@pytest.mark.parametrize("triclinic", [False, True])
def test_symmetry_and_no_self_pair(triclinic):
    P, C, pb, ptr = periodic_batch(3, 3, 5, 40, 0.05, triclinic=triclinic, spread=1.5)
    e = oracle.nl_brute(P, C, pb, ptr, 5.0)
    assert len(e) > 0
    assert not np.any((e[:, 0] == e[:, 1]) & np.all(e[:, 2:] == 0, axis=1))
    rev = e.copy()
    rev[:, 0], rev[:, 1] = e[:, 1], e[:, 0]
    rev[:, 2:] = -e[:, 2:]
    assert np.array_equal(oracle.canonical_edges(rev), e)
    bi = oracle.batch_idx_from_ptr(ptr)
    assert np.array_equal(bi[e[:, 0]], bi[e[:, 1]])
    half = oracle.nl_brute(P, C, pb, ptr, 5.0, half=True)
    assert 2 * len(half) == len(e)


def test_lattice_translation_of_atoms_moves_only_the_shifts():
    rng = np.random.default_rng(5)
    n, L = 30, 8.0
    P = (rng.integers(0, 8 * 1024, (n, 3)) / 1024.0).astype(np.float32)  # dyadic, exact
    C = np.eye(3, dtype=np.float32)[None] * L
    pb = np.ones((1, 3), bool)
    e0 = oracle.nl_brute(P, C, pb, [0, n], 3.0)
    k = rng.integers(-2, 3, (n, 3))
    P2 = (P.astype(np.float64) + k * L).astype(np.float32)
    assert np.array_equal(P2.astype(np.float64), P.astype(np.float64) + k * L)
    e1 = oracle.nl_brute(P2, C, pb, [0, n], 3.0)
    # r_j + k_j L - (r_i + k_i L) + S' L = r_j - r_i + S L  =>  S' = S - k_j + k_i
    exp = e0.copy()
    exp[:, 2:] = e0[:, 2:] - k[e0[:, 1]] + k[e0[:, 0]]
    assert np.array_equal(oracle.canonical_edges(exp), e1)


def _numpy_brute(P, C, pb, ptr, rc, qmax=3):
    out = []
    q = np.stack(np.meshgrid(*[np.arange(-qmax, qmax + 1)] * 3, indexing="ij"), -1).reshape(-1, 3)
    for s in range(len(ptr) - 1):
        a0, a1 = ptr[s], ptr[s + 1]
        H = C[s].astype(np.float64)
        qs = q[np.all((q == 0) | pb[s][None, :], axis=1)]
        T = qs @ H
        R = P[a0:a1].astype(np.float64)
        for i in range(a1 - a0):
            d = R[None, :, :] - R[i][None, None, :] + T[:, None, :]
            ok = (d * d).sum(-1) < rc * rc
            for si, j in zip(*np.nonzero(ok)):
                if j == i and not qs[si].any():
                    continue
                out.append([a0 + i, a0 + j, *qs[si]])
    return oracle.canonical_edges(np.array(out).reshape(-1, 5))


@pytest.mark.parametrize("triclinic", [False, True])
def test_brute_matches_independent_numpy_enumeration(triclinic):
    P, C, pb, ptr = periodic_batch(11, 2, 6, 14, 0.03, triclinic=triclinic)
    pb[1] = [True, False, True]
    assert np.array_equal(oracle.nl_brute(P, C, pb, ptr, 4.0), _numpy_brute(P, C, pb, ptr, 4.0))


CASES = [
    dict(seed=1, n_systems=5, n_lo=20, n_hi=300, density=0.05, triclinic=False, rc=5.0),
    dict(seed=2, n_systems=6, n_lo=8, n_hi=200, density=0.0764, triclinic=True, rc=5.0),
    dict(seed=3, n_systems=4, n_lo=8, n_hi=40, density=0.0764, triclinic=True, rc=6.0, spread=2.0),
    dict(seed=4, n_systems=3, n_lo=50, n_hi=400, density=0.1, triclinic=False, rc=6.0,
         pbc=[True, True, False]),
    dict(seed=5, n_systems=3, n_lo=1, n_hi=3, density=0.2, triclinic=True, rc=4.0),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"seed{c['seed']}")
@pytest.mark.parametrize("half", [False, True])
def test_cell_list_equals_brute_force(case, half):
    c = dict(case)
    rc = c.pop("rc")
    P, C, pb, ptr = periodic_batch(**c)
    ref = oracle.nl_brute(P, C, pb, ptr, rc, half=half)
    K = int(np.bincount(ref[:, 0], minlength=len(P)).max()) + 1
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, K, half=half)
    assert np.array_equal(oracle.matrix_to_edges(nm, nn, sh), ref)
    assert np.array_equal(nn, np.bincount(ref[:, 0], minlength=len(P)))
    cols = np.arange(K)[None, :]
    assert np.all(nm[cols >= nn[:, None]] == len(P))
    assert np.all(sh[cols >= nn[:, None]] == 0)


def test_cell_list_non_periodic_molecules_and_overflow_counts():
    P, Z, M, ptr = molecules_batch(seed=0)
    ref = oracle.nl_brute(P, None, None, ptr, 5.0)
    nm, nn, sh = oracle.nl_cell(P, None, None, ptr, 5.0, 32)
    assert np.array_equal(oracle.matrix_to_edges(nm, nn, sh), ref)
    # K too small: counts keep the true totals, rows hold the first K found
    nm2, nn2, _ = oracle.nl_cell(P, None, None, ptr, 5.0, 4)
    assert np.array_equal(nn2, nn) and nn2.max() >= 4 and nm2.shape == (len(P), 4)


def test_empty_and_single_atom_systems():
    pos = np.array([[0.0, 0, 0], [1.0, 0, 0], [9.0, 9, 9]], dtype=np.float32)
    ptr = ptr_from_counts([0, 2, 0, 1])
    e = oracle.nl_brute(pos, None, None, ptr, 2.0)
    assert np.array_equal(e, _edges([0, 1, 0, 0, 0], [1, 0, 0, 0, 0]))
    nm, nn, sh = oracle.nl_cell(pos, None, None, ptr, 2.0, 4)
    assert np.array_equal(oracle.matrix_to_edges(nm, nn, sh), e)
