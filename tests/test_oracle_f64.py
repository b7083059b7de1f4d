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


# ---- Langevin, Nose-Hoover chain, FIRE 2.0 in double ------------------------------------------------------------
def _thermostat_case(seed, n_systems=3, n_lo=4, n_hi=9):
    """Per-atom and per-system arrays that float32 holds exactly (multiples of 2^-10)."""
    g = np.random.default_rng(seed)
    counts = g.integers(n_lo, n_hi, n_systems)
    ptr = ptr_from_counts(counts)
    bidx = oracle.batch_idx_from_ptr(ptr)
    N = int(ptr[-1])
    q = lambda a: np.round(a * 1024.0) / 1024.0  # noqa: E731
    return dict(N=N, M=n_systems, bidx=bidx, pos=q(g.normal(size=(N, 3)) * 3.0), vel=q(g.normal(size=(N, 3)) * 0.2),
                frc=q(g.normal(size=(N, 3))), masses=q(g.uniform(1.0, 20.0, N)), dt=q(g.uniform(0.05, 0.2, n_systems)),
                kT=q(g.uniform(0.02, 0.05, n_systems)), friction=q(g.uniform(0.1, 2.0, n_systems)))


def test_langevin_in_double_equals_the_float32_oracle_to_float32_rounding_and_its_closed_forms():
    c = _thermostat_case(5)
    active = np.array([1, 0, 1], dtype=np.uint8)
    for act in (None, active):
        p32, v32 = c["pos"].astype(np.float32), c["vel"].astype(np.float32)
        oracle.langevin_half_step(p32, v32, c["frc"], c["masses"], c["dt"], c["kT"], c["friction"], 77, c["bidx"], act)
        p64, v64 = c["pos"].copy(), c["vel"].copy()
        f64.langevin_half_step(p64, v64, c["frc"], c["masses"], c["dt"], c["kT"], c["friction"], 77, c["bidx"], act)
        assert np.abs(p64 - p32).max() < 2e-6 and np.abs(v64 - v32).max() < 2e-6
        if act is not None:
            off = act[c["bidx"]] == 0
            assert np.array_equal(p64[off], c["pos"][off]) and np.array_equal(v64[off], c["vel"][off])
            assert off.any() and not np.array_equal(p64[~off], c["pos"][~off])
    # no friction: c1 = 1, c2 = 0, the noise drops out: a kick of dt/2 and two drifts of dt/2 with the kicked velocity
    zero = np.zeros(c["M"])
    p, v = c["pos"].copy(), c["vel"].copy()
    f64.langevin_half_step(p, v, c["frc"], c["masses"], c["dt"], c["kT"], zero, 3, c["bidx"])
    h = c["dt"][c["bidx"]][:, None]
    vk = c["vel"] + (c["frc"] / c["masses"][:, None]) * (0.5 * h)
    assert np.abs(v - vk).max() < 1e-15 and np.abs(p - (c["pos"] + vk * h)).max() < 1e-14
    # no forces, no temperature: the velocity decays by exp(-gamma dt)
    p, v = c["pos"].copy(), c["vel"].copy()
    f64.langevin_half_step(p, v, np.zeros_like(c["frc"]), c["masses"], c["dt"], zero, c["friction"], 3, c["bidx"])
    decay = np.exp(-c["friction"] * c["dt"])[c["bidx"]][:, None]
    assert np.abs(v - c["vel"] * decay).max() < 1e-15
    assert np.abs(p - (c["pos"] + 0.5 * h * c["vel"] * (1.0 + decay))).max() < 1e-14
    # the noise has the amplitude sqrt(kT/m (1 - c1^2)) and the deviates of the float32 oracle
    p, v = np.zeros((c["N"], 3)), np.zeros((c["N"], 3))
    f64.langevin_half_step(p, v, np.zeros_like(c["frc"]), c["masses"], c["dt"], c["kT"], c["friction"], 9, c["bidx"])
    xi = np.array([oracle.langevin_normals(9, i)[:3] for i in range(c["N"])])
    amp = np.sqrt(c["kT"][c["bidx"]] / c["masses"] * (1.0 - np.exp(-2.0 * c["friction"] * c["dt"])[c["bidx"]]))
    assert np.abs(v - amp[:, None] * xi).max() < 1e-14


def test_the_chain_in_double_equals_the_float32_oracle_to_float32_rounding_and_its_closed_forms():
    c = _thermostat_case(6, n_systems=4)
    M, bidx = c["M"], c["bidx"]
    ndof = 3.0 * np.bincount(bidx, minlength=M)
    g = np.random.default_rng(1)
    for C, order in [(1, 1), (3, 3), (4, 5)]:
        Q = oracle.nhc_masses(c["kT"], np.full(M, 0.5), ndof, C).astype(np.float64)
        eta0 = np.round(g.normal(size=(M, C)) * 64.0) / 1024.0
        eta_dot0 = np.round(g.normal(size=(M, C)) * 64.0) / 1024.0
        active = np.array([1, 1, 0, 1], dtype=np.uint8)
        for act in (None, active):
            v32, e32, d32 = c["vel"].astype(np.float32), eta0.astype(np.float32), eta_dot0.astype(np.float32)
            k32, s32 = oracle.nhc_chain_update(v32, c["masses"], e32, d32, Q, c["kT"], c["dt"], ndof, bidx, active=act,
                                               yoshida_order=order)
            v64, e64, d64 = c["vel"].copy(), eta0.copy(), eta_dot0.copy()
            k64, s64 = f64.nhc_chain_update(v64, c["masses"], e64, d64, Q, c["kT"], c["dt"], ndof, bidx, active=act,
                                            yoshida_order=order)
            live = np.ones(M, bool) if act is None else act.astype(bool)
            assert np.abs(v64 - v32).max() < 1e-6 and np.abs(e64 - e32).max() < 1e-6 and np.abs(d64 - d32).max() < 1e-5
            assert np.allclose(k64, k32, rtol=1e-6) and np.allclose(s64[live], s32[live], rtol=1e-6)
            if act is not None:
                assert np.array_equal(v64[bidx == 2], c["vel"][bidx == 2]) and np.array_equal(e64[2], eta0[2])
    # a chain at rest with the kinetic energy at its target: the first link feels no force
    vel = c["vel"].copy()
    k2 = np.bincount(bidx, weights=c["masses"] * (vel * vel).sum(1), minlength=M)
    kT = k2 / ndof
    Q = oracle.nhc_masses(kT, np.full(M, 0.5), ndof, 3).astype(np.float64)
    eta, eta_dot = np.zeros((M, 3)), np.zeros((M, 3))
    # (G_1 = 0 exactly when ke2 is supplied as ndof kT; G_k = -kT / Q_k for the links above: they do move)
    _, scale = f64.nhc_chain_update(vel, c["masses"], eta, eta_dot, Q, kT, c["dt"], ndof, bidx, ke2=ndof * kT,
                                    yoshida_order=1)
    assert np.all(eta_dot[:, 1:] < 0.0) and np.abs(eta_dot[:, 0]).max() < 1e-3  # (the first link only through the second)
    # one link, one weight: u' = u + G d/4 twice around s = exp(-u d/2), with KE2 scaled by s^2 in between
    Q1 = oracle.nhc_masses(c["kT"], np.full(M, 0.5), ndof, 1).astype(np.float64)
    vel = c["vel"].copy()
    k2 = np.bincount(bidx, weights=c["masses"] * (vel * vel).sum(1), minlength=M)
    eta, eta_dot = np.zeros((M, 1)), np.full((M, 1), 0.125)
    _, scale = f64.nhc_chain_update(vel, c["masses"], eta, eta_dot, Q1, c["kT"], c["dt"], ndof, bidx, yoshida_order=1)
    d = c["dt"]
    u1 = 0.125 + (k2 - ndof * c["kT"]) / Q1[:, 0] * d / 4
    s = np.exp(-u1 * d / 2)
    u2 = u1 + (k2 * s * s - ndof * c["kT"]) / Q1[:, 0] * d / 4
    assert np.abs(scale - s).max() < 1e-15 and np.abs(eta_dot[:, 0] - u2).max() < 1e-14
    assert np.abs(eta[:, 0] - u1 * d / 2).max() < 1e-16 and np.abs(vel - c["vel"] * s[bidx][:, None]).max() < 1e-15
    # the drift
    p = c["pos"].copy()
    f64.nhc_position_update(p, c["vel"], c["dt"], bidx, np.array([1, 0, 1, 1], dtype=np.uint8))
    want = c["pos"] + c["vel"] * c["dt"][bidx][:, None]
    assert np.array_equal(p[bidx != 1], want[bidx != 1]) and np.array_equal(p[bidx == 1], c["pos"][bidx == 1])


def test_fire2_in_double_equals_the_float32_oracle_to_float32_rounding_and_its_uphill_form():
    c = _thermostat_case(8, n_systems=4, n_lo=5, n_hi=12)
    M, bidx = c["M"], c["bidx"]
    # systems 0 and 2 uphill (v against F), 1 and 3 downhill
    vel = c["vel"].copy()
    sign = np.where(np.isin(bidx, [0, 2]), -1.0, 1.0)[:, None]
    vel = sign * np.abs(vel) * np.sign(c["frc"] + 1e-30)
    active = np.array([1, 1, 1, 0], dtype=np.uint8)
    for act in (None, active):
        for maxstep in (0.1, 0.004):
            a32, d32, n32 = np.full(M, 0.09, np.float32), np.full(M, 0.03125, np.float32), np.array([60, 61, 3, 7], np.int32)
            p32, v32 = c["pos"].astype(np.float32), vel.astype(np.float32)
            o32 = oracle.fire2_step(p32, v32, c["frc"], bidx, a32, d32, n32, active=act, maxstep=maxstep)
            a64, d64, n64 = np.full(M, 0.09), np.full(M, 0.03125), np.array([60, 61, 3, 7], np.int32)
            p64, v64 = c["pos"].copy(), vel.copy()
            o64 = f64.fire2_step(p64, v64, c["frc"], bidx, a64, d64, n64, active=act, maxstep=maxstep)
            assert np.abs(p64 - p32).max() < 2e-6 and np.abs(v64 - v32).max() < 2e-6
            assert np.array_equal(n64, n32) and np.allclose(a64, a32, rtol=1e-6) and np.allclose(d64, d32, rtol=1e-6)
            for k in ("vf", "v_sumsq", "f_sumsq"):
                assert np.allclose(o64[k], o32[k], rtol=1e-6), k
            live = np.ones(M, bool) if act is None else act.astype(bool)
            assert np.allclose(o64["max_norm"][live], o32["max_norm"][live], rtol=1e-5)
            assert n64[0] == 0 and n64[1] == 62 and (act is not None or n64[3] == 8)
    # P <= 0 in double: half a step back with the old velocity, then a plain kick and drift from rest
    a, d, n = np.full(M, 0.2), np.full(M, 0.0625), np.full(M, 9, np.int32)
    p, v = c["pos"].copy(), vel.copy()
    f64.fire2_step(p, v, c["frc"], bidx, a, d, n, maxstep=1e9, dtshrink=0.5, tmin=0.0)
    up = np.isin(bidx, [0, 2])
    assert np.array_equal(d, np.where(np.isin(np.arange(M), [0, 2]), 0.03125, 0.0625)) and a[0] == 0.09 and n[0] == 0
    want_v = 0.03125 * c["frc"][up]
    assert np.abs(v[up] - want_v).max() < 1e-17
    assert np.abs(p[up] - (c["pos"][up] - 0.03125 * vel[up] + 0.03125 * want_v)).max() < 1e-15
