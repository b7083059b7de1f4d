"""The float64 restatement (oracle/f64.py) pinned: against the float32 oracle on inputs that float32
holds exactly (the two must then agree: to the bit for neighbor sets, to float32 rounding for the
rest), against closed forms evaluated in double, and on pairs that only double resolves."""

import numpy as np

import oracle
from oracle import f64
from _systems import periodic_batch, ptr_from_counts, sheared_fcc_boxes


def test_neighbor_sets_equal_the_float32_oracle_on_float32_inputs():
    for seed, tri, pbc in [(0, False, None), (1, True, None), (2, True, [True, False, True]), (3, False, [False, False, False])]:
        P, C, pb, ptr = periodic_batch(seed, 3, 5, 40, 0.05, triclinic=tri, pbc=pbc, spread=0.3)
        for half in (False, True):
            want = oracle.nl_brute(P, C, pb, ptr, 4.0, half=half)
            got = f64.nl_brute(P.astype(np.float64), C.astype(np.float64), pb, ptr, 4.0, half=half)
            assert np.array_equal(got, want), (seed, half)
    # a cell narrower than the cutoff: several images of the same pair, self images
    P = np.array([[0.1, 0.2, 0.3], [1.0, 1.1, 0.9]], dtype=np.float32)
    C = (np.eye(3) * 2.0).astype(np.float32)[None]
    pb = np.ones((1, 3), bool)
    ptr = ptr_from_counts([2])
    assert np.array_equal(f64.nl_brute(P.astype(np.float64), C.astype(np.float64), pb, ptr, 3.0), oracle.nl_brute(P, C, pb, ptr, 3.0))


def test_pairs_that_only_double_resolves():
    rc = 3.0
    for eps, inside in [(-1e-12, True), (1e-12, False), (-1e-9, True), (1e-9, False)]:
        P = np.array([[0.0, 0.0, 0.0], [rc * (1.0 + eps), 0.0, 0.0]])
        assert np.float32(P[1, 0]) == np.float32(rc)  # float32 cannot tell them apart
        e = f64.nl_brute(P, None, None, ptr_from_counts([2]), rc)
        assert (len(e) == 2) == inside
    # across a periodic boundary, with the shift that brings the pair together
    L = 10.0
    P = np.array([[0.25, 5.0, 5.0], [L - 2.75 + 1e-11, 5.0, 5.0]])
    e = f64.nl_brute(P, np.eye(3)[None] * L, np.ones((1, 3), bool), ptr_from_counts([2]), rc)
    assert e.tolist() == [[0, 1, -1, 0, 0], [1, 0, 1, 0, 0]]
    P[1, 0] -= 2e-11
    assert len(f64.nl_brute(P, np.eye(3)[None] * L, np.ones((1, 3), bool), ptr_from_counts([2]), rc)) == 0


def _dimer(r, eps=0.7, sig=1.3, rc=5.0, **kw):
    P = np.array([[0.0, 0.0, 0.0], [r, 0.0, 0.0]])
    nm = np.array([[1], [0]], dtype=np.int32)
    nn = np.array([1, 1], dtype=np.int32)
    return f64.lj_matrix(P, np.eye(3)[None] * 100.0, nm, None, nn, np.zeros(2, np.int32), 2, eps, sig, rc, **kw)


def test_lennard_jones_closed_forms_in_double():
    eps, sig = 0.7, 1.3
    out = _dimer(sig)
    assert abs(out["energy"][0]) < 1e-15 and abs(out["forces"][0, 0] + 24 * eps / sig) < 1e-12
    rm = 2 ** (1 / 6) * sig
    out = _dimer(rm)
    assert abs(out["energy"][0] + eps) < 1e-15 and np.abs(out["forces"]).max() < 1e-13
    # F = -dE/dr to 1e-9 (central difference in double), with and without the switch
    for sw in (0.0, 1.5):
        for r in (1.2, 1.7, 3.9, 4.6):
            hstep = 1e-6
            dE = (_dimer(r + hstep, switch_width=sw)["energy"][0] - _dimer(r - hstep, switch_width=sw)["energy"][0]) / (2 * hstep)
            f1 = _dimer(r, switch_width=sw)["forces"][1, 0]
            assert abs(f1 + dE) < 1e-8 * max(1.0, abs(dE)), (sw, r)
    assert _dimer(5.0)["energy"][0] == 0.0 and _dimer(4.999999)["energy"][0] != 0.0  # strict cutoff, no shift


def test_lennard_jones_equals_the_float32_oracle_to_float32_rounding():
    P, C, pb, ptr = sheared_fcc_boxes(seed=2, n_boxes=2, reps=3)
    bi = oracle.batch_idx_from_ptr(ptr)
    for half in (False, True):
        nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, 2.5, 96, half=half)
        a = oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), 1.0, 1.0, 2.5, half=half, virial=True)
        b = f64.lj_matrix(P.astype(np.float64), C.astype(np.float64), nm, sh, nn, bi, len(P), 1.0, 1.0, 2.5, half=half, virial=True)
        for k in ("atomic_energies", "forces", "energy", "virials"):
            scale = np.abs(b[k]).max()
            assert np.abs(a[k] - b[k]).max() <= 2e-6 * scale, (half, k)
        assert np.abs(b["forces"].sum(0)).max() < 1e-10 * np.abs(b["forces"]).max() * len(P)


def test_velocity_verlet_in_double():
    # one harmonic oscillator (F = -k x): the discrete map has the closed form x_n = cos(n theta) with
    # cos(theta) = 1 - k dt^2 / (2 m) when v_0 = 0
    k, m, dt = 2.0, 1.5, 0.05
    x = np.array([[1.0, 0.0, 0.0]])
    v = np.zeros((1, 3))
    bi = np.zeros(1, np.int32)
    theta = np.arccos(1.0 - k * dt * dt / (2 * m))
    F = -k * x
    for n in range(1, 200):
        f64.vv_pre(x, v, F, np.array([m]), np.array([dt]), bi)
        F = -k * x
        f64.vv_post(v, F, np.array([m]), np.array([dt]), bi)
        assert abs(x[0, 0] - np.cos(n * theta)) < 1e-12
    # and the float32 oracle on the same float32 inputs, to its rounding
    rng = np.random.default_rng(0)
    P, V, Fo = (rng.normal(size=(50, 3)).astype(np.float32) for _ in range(3))
    M = rng.uniform(1, 20, 50).astype(np.float32)
    bi = np.repeat(np.arange(5, dtype=np.int32), 10)
    dts = rng.uniform(0.1, 1.0, 5).astype(np.float32)
    act = np.array([1, 0, 1, 1, 0], np.uint8)
    P32, V32 = P.copy(), V.copy()
    oracle.vv_pre(P32, V32, Fo, M, dts, bi, active=act)
    P64, V64 = P.astype(np.float64), V.astype(np.float64)
    f64.vv_pre(P64, V64, Fo.astype(np.float64), M.astype(np.float64), dts.astype(np.float64), bi, active=act)
    assert np.abs(P32 - P64).max() < 1e-6 and np.abs(V32 - V64).max() < 1e-6
    assert np.array_equal(P64[10:20], P[10:20].astype(np.float64))  # inactive system untouched


def _fire_state(M, dtype):
    full = lambda v, t=dtype: np.full(M, v, dtype=t)  # noqa: E731
    return {"alpha": full(0.1), "dt": full(0.01), "alpha_start": full(0.1), "f_alpha": full(0.99), "dt_min": full(0.0002),
            "dt_max": full(0.1), "maxstep": full(0.2), "f_dec": full(0.5), "f_inc": full(1.1), "vf": full(0), "vv": full(0),
            "ff": full(0), "n_steps_positive": np.zeros(M, np.int32), "n_min": np.full(M, 5, np.int32)}


def test_fire_equals_the_float32_oracle_to_float32_rounding_and_goes_downhill():
    rng = np.random.default_rng(1)
    N, M = 40, 4
    x0 = rng.normal(size=(N, 3)).astype(np.float32)
    P = (x0 + rng.normal(scale=0.3, size=(N, 3))).astype(np.float32)
    bi = np.repeat(np.arange(M, dtype=np.int32), N // M)
    mass = rng.uniform(1, 3, N).astype(np.float32)
    kk = np.float32(3.0)
    P32, V32 = P.copy(), np.zeros_like(P)
    P64, V64 = P.astype(np.float64), np.zeros((N, 3))
    s32, s64 = _fire_state(M, np.float32), _fire_state(M, np.float64)
    e0 = 0.5 * 3.0 * ((P64 - x0) ** 2).sum()
    for _ in range(60):
        oracle.fire_step(P32, V32, (-kk * (P32 - x0)).astype(np.float32), mass, s32, bi)
        f64.fire_step(P64, V64, -3.0 * (P64 - x0.astype(np.float64)), mass.astype(np.float64), s64, bi)
    assert np.array_equal(s32["n_steps_positive"], s64["n_steps_positive"])
    assert np.allclose(s32["dt"], s64["dt"], rtol=1e-5) and np.allclose(s32["alpha"], s64["alpha"], rtol=1e-5)
    assert np.abs(P32 - P64).max() < 5e-5
    assert 0.5 * 3.0 * ((P64 - x0) ** 2).sum() < 1e-3 * e0


def test_fmax_in_double():
    f = np.array([[3.0, 4.0, 0.0], [0.0, 0.0, 1e-200], [1.0, 2.0, 2.0]])
    out = f64.fmax(f, np.array([0, 0, 2], np.int32), 3)
    assert out[0] == 5.0 and out[1] == -np.inf and out[2] == 3.0


def _skin_case(seed=7):
    """Three triclinic boxes with mixed periodic flags, float32-exact values: a reference, a current
    configuration with a few atoms pushed across faces, one system left as it was."""
    P, C, pb, ptr = periodic_batch(seed, 3, 30, 60, 0.05, triclinic=True)
    pb = pb.copy()
    pb[1] = [1, 0, 1]
    bi = oracle.batch_idx_from_ptr(ptr)
    rng = np.random.default_rng(seed)
    cur = P.copy()
    moved = bi != 2
    cur[moved] += rng.normal(0, 0.08, (int(moved.sum()), 3)).astype(np.float32)
    cur[0] += (2 * C[0][0] - C[0][1]).astype(np.float32)  # a lattice translation: no displacement on periodic axes
    return P, cur, C, pb, ptr, bi


def test_skin_test_in_double_equals_the_float32_oracle_on_float32_inputs():
    P, cur, C, pb, ptr, bi = _skin_case()
    B = len(ptr) - 1
    for cell, pbc in ((None, None), (C, pb)):
        for thr in (0.05, 0.2, 0.5):
            f32, ref32 = oracle.rebuild_check(P, cur, bi, B, thr, update_reference=True, cell=cell, pbc=pbc)
            ref64 = P.astype(np.float64)
            got = f64.rebuild_check(ref64, cur.astype(np.float64), bi, B, thr, update_reference=True,
                                    cell=None if cell is None else cell.astype(np.float64), pbc=pbc)
            assert np.array_equal(got.astype(bool), f32)
            assert np.array_equal(ref64, ref32.astype(np.float64))  # the same systems were refreshed
    # with the cell, the lattice translation of atom 0 does not flag system 0 at a threshold above the jitter
    assert f64.rebuild_check(P.astype(np.float64), cur.astype(np.float64), bi, B, 0.6, cell=C.astype(np.float64), pbc=pb)[0] == 0
    assert f64.rebuild_check(P.astype(np.float64), cur.astype(np.float64), bi, B, 0.6)[0] == 1


def test_skin_test_resolves_what_only_double_resolves():
    """A displacement of threshold (1 +- 1e-12): float32 cannot tell either from the threshold."""
    ref = np.zeros((2, 3))
    thr = 0.25
    for eps, want in ((+1e-12, 1), (-1e-12, 0)):
        cur = ref.copy()
        cur[1] = np.array([0.6, 0.0, 0.8]) * thr * (1 + eps)
        assert f64.rebuild_check(ref.copy(), cur, [0, 0], 1, thr)[0] == want


def test_wrap_in_double():
    P, cur, C, pb, ptr, bi = _skin_case(9)
    far = (cur.astype(np.float64) * 3.0 - 5.0)  # well outside the cells
    W = f64.wrap_positions(far, C.astype(np.float64), pb, bi)
    for s in range(len(ptr) - 1):
        a, b = ptr[s], ptr[s + 1]
        H = C[s].astype(np.float64)
        moved = (W[a:b] - far[a:b]) @ np.linalg.inv(H)
        if pb[s].all():
            frac = W[a:b] @ np.linalg.inv(H)
            assert frac.min() > -1e-12 and frac.max() < 1 + 1e-12          # inside the cell
            assert np.abs(moved - np.round(moved)).max() < 1e-9            # moved by whole lattice vectors
    # float32-exact inputs: the float32 oracle's result is this one rounded once
    W32 = oracle.wrap_positions(cur, C, pb, bi)
    W64 = f64.wrap_positions(cur.astype(np.float64), C.astype(np.float64), pb, bi)
    assert np.array_equal(W64.astype(np.float32), W32)
    # an open system is left alone; a Cartesian component whose flag is clear is kept
    pb0 = pb.copy()
    pb0[2] = 0
    W0 = f64.wrap_positions(far, C.astype(np.float64), pb0, bi)
    assert np.array_equal(W0[ptr[2]:ptr[3]], far[ptr[2]:ptr[3]])
    assert np.array_equal(W[ptr[1]:ptr[2], 1], far[ptr[1]:ptr[2], 1])
