"""CPU checks that pin the oracle's Verlet-skin displacement test and periodic wrap.

Skin test: the cases of the reference's own tests of ``batch_neighbor_list_rebuild_inplace``
(test/hooks/test_neighbor_list_hook.py:166-246), restated, plus what the geometry fixes (a
displacement of a whole lattice vector is no displacement under the minimum-image convention).
Wrap: the documented formula (nvalchemi/hooks/periodic.py:159-163) against plain numpy, the
per-axis masking of :111-113, and invariants (result inside the cell, equal modulo the lattice).
"""

import numpy as np

import oracle
from _systems import periodic_batch


def _idx(counts):
    return np.repeat(np.arange(len(counts)), counts).astype(np.int32)


def test_flags_are_cleared_and_unmoved_atoms_do_not_flag():
    ref = np.zeros((4, 3), np.float32)
    flags, _ = oracle.rebuild_check(ref, ref.copy(), _idx([4]), 1, 0.5)
    assert not flags.any()
    rng = np.random.default_rng(0)
    ref = rng.normal(size=(6, 3)).astype(np.float32)
    flags, _ = oracle.rebuild_check(ref, ref.copy(), _idx([3, 3]), 2, 0.1)
    assert not flags.any()


def test_displacement_above_and_below_the_threshold():
    ref = np.zeros((3, 3), np.float32)
    cur = ref.copy()
    cur[1, 0] = 1.0
    flags, _ = oracle.rebuild_check(ref, cur, _idx([3]), 1, 0.5)
    assert flags[0]
    cur = ref.copy()
    cur[0, 0] = 0.1
    flags, _ = oracle.rebuild_check(ref, cur, _idx([3]), 1, 0.5)
    assert not flags[0]


def test_only_the_system_that_moved_is_flagged():
    ref = np.zeros((6, 3), np.float32)
    cur = ref.copy()
    cur[4, 0] = 1.0
    flags, _ = oracle.rebuild_check(ref, cur, _idx([3, 3]), 2, 0.5)
    assert flags.tolist() == [False, True]


def test_reference_is_refreshed_only_for_flagged_systems():
    ref = np.zeros((6, 3), np.float32)
    cur = ref.copy()
    cur[0, 0] = 1.0     # system 0: above
    cur[1, 1] = 0.2     # system 0: below, refreshed together with its system
    cur[4, 2] = 0.1     # system 1: below
    flags, new_ref = oracle.rebuild_check(ref, cur, _idx([3, 3]), 2, 0.5, update_reference=True)
    assert flags.tolist() == [True, False]
    assert np.array_equal(new_ref[:3], cur[:3])
    assert np.array_equal(new_ref[3:], ref[3:])
    flags, same = oracle.rebuild_check(ref, cur, _idx([3, 3]), 2, 0.5, update_reference=False)
    assert np.array_equal(same, ref)


def test_a_lattice_translation_is_no_displacement_on_periodic_axes_only():
    cell = np.array([[[4.0, 0, 0], [1.0, 5.0, 0], [0, 0, 6.0]]], np.float32)
    ref = np.array([[0.5, 0.5, 0.5]], np.float32)
    cur = (ref + cell[0, 1] - cell[0, 0]).astype(np.float32)  # moved by a1 - a0
    flags, _ = oracle.rebuild_check(ref, cur, _idx([1]), 1, 0.01, cell=cell, pbc=np.array([[1, 1, 1]]))
    assert not flags[0]
    flags, _ = oracle.rebuild_check(ref, cur, _idx([1]), 1, 0.01, cell=cell, pbc=np.array([[1, 0, 1]]))
    assert flags[0]      # the a1 part is a real displacement when axis 1 is not periodic
    flags, _ = oracle.rebuild_check(ref, cur, _idx([1]), 1, 0.01)
    assert flags[0]      # no cell: plain displacement


def test_wrap_matches_the_documented_formula_and_lands_inside_the_cell():
    P, C, pb, ptr = periodic_batch(seed=3, n_systems=5, n_lo=5, n_hi=40, density=0.05, triclinic=True, spread=2.5)
    bi = oracle.batch_idx_from_ptr(ptr)
    W = oracle.wrap_positions(P, C, pb, bi)
    for s in range(len(ptr) - 1):
        sl = slice(ptr[s], ptr[s + 1])
        H = C[s].astype(np.float64)
        frac = P[sl].astype(np.float64) @ np.linalg.inv(H)
        expect = (frac % 1.0) @ H
        assert np.allclose(W[sl], expect, rtol=0, atol=2e-6 * np.abs(H).max())
        fw = W[sl].astype(np.float64) @ np.linalg.inv(H)
        assert (fw > -1e-5).all() and (fw < 1 + 1e-5).all()
        shift = (W[sl].astype(np.float64) - P[sl]) @ np.linalg.inv(H)
        assert np.allclose(shift, np.round(shift), atol=1e-4)  # moved by whole lattice vectors


def test_wrap_keeps_the_cartesian_components_of_non_periodic_axes():
    cell = (np.eye(3) * 10).astype(np.float32)[None]
    pos = np.array([[11.0, -1.0, 25.0], [3.0, 4.0, 5.0]], np.float32)
    bi = np.zeros(2, np.int32)
    assert np.allclose(oracle.wrap_positions(pos, cell, np.array([[1, 1, 0]]), bi), [[1, 9, 25], [3, 4, 5]])
    assert np.array_equal(oracle.wrap_positions(pos, cell, np.array([[0, 0, 0]]), bi), pos)
    # a sheared cell with one open axis: the open axis keeps its old Cartesian component even
    # though wrapping the other two changes what lies along it (the reference masks Cartesian
    # components, nvalchemi/hooks/periodic.py:111-113)
    cell = np.array([[[10.0, 0, 0], [0, 10.0, 0], [3.0, 0, 10.0]]], np.float32)
    pos = np.array([[1.0, 2.0, 12.0]], np.float32)
    out = oracle.wrap_positions(pos, cell, np.array([[0, 1, 1]]), np.zeros(1, np.int32))
    assert out[0, 0] == pos[0, 0]
    assert np.allclose(out[0, 1:], [2.0, 2.0], atol=1e-5)
