"""GPU parity of the float64 forms (through the C ABI) against the float64 oracle (oracle/f64.py).

The reference's ops take float32 or float64 arrays (nvalchemi/dynamics/_ops/_bridge.py, _ops/fire.py:281-287,
models/_ops/lj.py:116-216).  Bars: neighbor data bit-exact as canonical sets (the decision is made in
double on the float64 positions); velocity Verlet bit for bit (one rounding per operation on both
sides); energies, forces, virials and the FIRE step to 1e-12 relative to the largest term (the sums
run in another order on the device: rounding of a double sum, nothing else)."""

import numpy as np
import pytest
import torch

import oracle
from oracle import f64
from _systems import fcc_boxes, periodic_batch, ptr_from_counts, sheared_fcc_boxes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def build(P, C, pb, ptr, rc, K, half=False, sort_path=None):
    from nvalchemi_amd import _lib

    N, B = len(P), len(ptr) - 1
    bi = oracle.batch_idx_from_ptr(ptr)
    nm = torch.full((N, K), N, dtype=torch.int32, device=DEV)
    nn = torch.zeros(N, dtype=torch.int32, device=DEV)
    sh = torch.zeros((N, K, 3), dtype=torch.int32, device=DEV) if C is not None else None
    _lib.nl_build(T(P, F64), None if C is None else T(C, F64), None if C is None else T(pb), T(ptr), T(bi), None, rc, K,
                  half, 1, nm, nn, sh, sort_path=sort_path)
    torch.cuda.synchronize()
    return nm.cpu().numpy(), nn.cpu().numpy(), None if sh is None else sh.cpu().numpy(), bi


@pytest.mark.parametrize("sort_path", [1, 2], ids=["per_system", "global"])
@pytest.mark.parametrize("half", [False, True])
def test_neighbor_build_on_float64_positions(sort_path, half):
    rng = np.random.default_rng(7)
    for seed, tri, pbc, spread in [(0, False, None, 0.0), (1, True, None, 0.5), (2, True, [True, False, True], 0.0)]:
        P32, C32, pb, ptr = periodic_batch(seed, 4, 5, 60, 0.05, triclinic=tri, pbc=pbc, spread=spread)
        # genuinely double positions: float32 values plus something float32 cannot hold
        P = P32.astype(np.float64) + rng.uniform(-1e-9, 1e-9, P32.shape)
        C = C32.astype(np.float64) * (1.0 + 1e-10)
        want = f64.nl_brute(P, C, pb, ptr, 4.0, half=half)
        nm, nn, sh, _ = build(P, C, pb, ptr, 4.0, 160, half=half, sort_path=sort_path)
        assert int(nn.max()) < 160
        assert np.array_equal(oracle.matrix_to_edges(nm, nn, sh), want), (seed, half)


def test_pairs_that_only_double_resolves_are_decided_in_double():
    rc, L = 3.0, 10.0
    cell = np.eye(3)[None] * L
    pb = np.ones((1, 3), bool)
    ptr = ptr_from_counts([2])
    for eps, inside in [(-1e-12, True), (1e-12, False)]:
        P = np.array([[1.0, 5.0, 5.0], [1.0 + rc * (1.0 + eps), 5.0, 5.0]])
        nm, nn, sh, _ = build(P, cell, pb, ptr, rc, 16)
        assert nn.tolist() == ([1, 1] if inside else [0, 0])
    P = np.array([[0.25, 5.0, 5.0], [L - 2.75 + 1e-11, 5.0, 5.0]])  # through the boundary
    nm, nn, sh, _ = build(P, cell, pb, ptr, rc, 16)
    assert nn.tolist() == [1, 1] and sh[0, 0].tolist() == [-1, 0, 0] and sh[1, 0].tolist() == [1, 0, 0]
    P[1, 0] -= 2e-11
    assert build(P, cell, pb, ptr, rc, 16)[1].tolist() == [0, 0]


def gpu_lj(P, C, nm, sh, nn, bi, eps, sig, rc, half=False, virial=False, switch_width=0.0):
    from nvalchemi_amd import _lib

    N, B = len(P), len(C)
    e = torch.empty(N, dtype=F64, device=DEV)
    f = torch.empty((N, 3), dtype=F64, device=DEV)
    w = torch.empty((B, 9), dtype=F64, device=DEV) if virial else None
    es = torch.empty(B, dtype=F64, device=DEV)
    _lib.lj_energy_forces(T(P, F64), T(C, F64), T(nm), None if sh is None else T(sh), T(nn), T(bi), N, eps, sig, rc,
                          switch_width, half, e, f, w, es)
    torch.cuda.synchronize()
    out = {"atomic_energies": e.cpu().numpy(), "forces": f.cpu().numpy(), "energy": es.cpu().numpy()}
    if virial:
        out["virials"] = w.cpu().numpy()
    return out


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("switch_width", [0.0, 1.0])
def test_lennard_jones_on_float64_positions(half, switch_width):
    rng = np.random.default_rng(3)
    for P32, C32, pb, ptr, rc, eps, sig in [
        (*sheared_fcc_boxes(seed=5, n_boxes=3, reps=3), 2.5, 1.0, 1.0),
        (*periodic_batch(9, 5, 8, 200, 0.0764, triclinic=True), 5.0, 0.01, 2.5),
    ]:
        P = P32.astype(np.float64) + rng.uniform(-1e-9, 1e-9, P32.shape)
        C = C32.astype(np.float64)
        nm, nn, sh, bi = build(P, C, pb, ptr, rc, 256, half=half)
        assert int(nn.max()) < 256
        want = f64.lj_matrix(P, C, nm, sh, nn, bi, len(P), eps, sig, rc, half=half, virial=True, switch_width=switch_width)
        got = gpu_lj(P, C, nm, sh, nn, bi, eps, sig, rc, half=half, virial=True, switch_width=switch_width)
        for k in want:
            # (a double sum in another order: rounding relative to the largest term of the sum)
            scale = np.abs(want[k]).max() if k != "forces" else None
            if k == "forces":
                scale = max(np.abs(want[k]).max(), 1.0)
            assert np.abs(got[k] - want[k]).max() <= 1e-11 * scale, (half, switch_width, k, np.abs(got[k] - want[k]).max())


def test_velocity_verlet_fire_and_fmax_on_float64_arrays():
    from nvalchemi_amd import _lib

    rng = np.random.default_rng(11)
    N, M = 777, 9
    counts = rng.multinomial(N, np.ones(M) / M)
    counts[3] = 0
    counts[0] += N - counts.sum()
    bi = np.repeat(np.arange(M, dtype=np.int32), counts)
    P, V, F = (rng.normal(size=(N, 3)) for _ in range(3))
    mass = rng.uniform(1, 30, N)
    dt = rng.uniform(0.1, 1.0, M)
    act = (rng.random(M) < 0.6)
    for active in (None, act):
        Pd, Vd = T(P), T(V)
        _lib.vv_position_update(Pd, Vd, T(F), T(mass), T(dt), T(bi), None if active is None else T(active))
        Pr, Vr = P.copy(), V.copy()
        f64.vv_pre(Pr, Vr, F, mass, dt, bi, active)
        assert np.array_equal(Pd.cpu().numpy(), Pr) and np.array_equal(Vd.cpu().numpy(), Vr)
        _lib.vv_velocity_finalize(Vd, T(F * 0.5), T(mass), T(dt), T(bi), None if active is None else T(active))
        f64.vv_post(Vr, F * 0.5, mass, dt, bi, active)
        assert np.array_equal(Vd.cpu().numpy(), Vr)
    fm = torch.empty(M, dtype=F64, device=DEV)
    _lib.segment_fmax(T(F), T(bi), fm)
    assert np.array_equal(fm.cpu().numpy(), f64.fmax(F, bi, M))
    # FIRE: twelve steps on a quadratic bowl, half of the systems frozen
    full = lambda v: np.full(M, v)  # noqa: E731
    st = {"alpha": full(0.1), "dt": full(0.02), "alpha_start": full(0.1), "f_alpha": full(0.99), "dt_min": full(0.0004),
          "dt_max": full(0.2), "maxstep": full(0.15), "f_dec": full(0.5), "f_inc": full(1.1), "vf": full(0.0), "vv": full(0.0),
          "ff": full(0.0), "n_steps_positive": np.zeros(M, np.int32), "n_min": np.full(M, 3, np.int32)}
    sd = {k: T(v) for k, v in st.items()}
    up = torch.zeros(M, dtype=torch.int32, device=DEV)
    Pd, Vd = T(P), T(V * 0.1)
    Pr, Vr = P.copy(), V * 0.1
    x0 = rng.normal(size=(N, 3))
    for _ in range(12):
        Fr = -2.0 * (Pr - x0)
        _lib.fire_step(Pd, Vd, T(Fr), T(mass), sd["alpha"], sd["dt"], sd["alpha_start"], sd["f_alpha"], sd["dt_min"], sd["dt_max"],
                       sd["maxstep"], sd["n_steps_positive"], sd["n_min"], sd["f_dec"], sd["f_inc"], up, sd["vf"], sd["vv"],
                       sd["ff"], T(bi), True, T(act))
        f64.fire_step(Pr, Vr, Fr, mass, st, bi, act)
        assert np.abs(Pd.cpu().numpy() - Pr).max() < 1e-12 and np.abs(Vd.cpu().numpy() - Vr).max() < 1e-12
        Pd.copy_(T(Pr)); Vd.copy_(T(Vr))  # (both sides continue from the same state)
    assert np.array_equal(sd["n_steps_positive"].cpu().numpy(), st["n_steps_positive"])
    assert np.allclose(sd["dt"].cpu().numpy(), st["dt"], rtol=1e-14) and np.allclose(sd["alpha"].cpu().numpy(), st["alpha"], rtol=1e-14)
    assert np.allclose(sd["vf"].cpu().numpy(), st["vf"], rtol=1e-12, atol=1e-12)


def test_a_float64_batch_runs_through_the_package_api():
    """NVE on a float64 batch: 20 steps against the float64 oracle loop (build, pair kernel, integrator)."""
    from nvalchemi_amd.data import AtomicData, Batch
    from nvalchemi_amd.dynamics import FIRE, NVE
    from nvalchemi_amd.models import LennardJonesModelWrapper

    P32, C32, pb, ptr = fcc_boxes(seed=4, n_boxes=2, reps=3, a=1.5496, jitter=0.03)
    P, C = P32.astype(np.float64), C32.astype(np.float64)
    N = len(P)
    bi = oracle.batch_idx_from_ptr(ptr)

    def make():
        data = []
        for s in range(len(ptr) - 1):
            a0, a1 = int(ptr[s]), int(ptr[s + 1])
            data.append(AtomicData(torch.from_numpy(P[a0:a1]), torch.full((a1 - a0,), 18), atomic_masses=torch.ones(a1 - a0, dtype=F64),
                                   cell=torch.from_numpy(C[s]), pbc=torch.from_numpy(pb[s]),
                                   forces=torch.zeros(a1 - a0, 3, dtype=F64), energy=torch.zeros(1, 1, dtype=F64)))
        return Batch.from_data_list(data, device=DEV)

    model = LennardJonesModelWrapper(epsilon=1.0, sigma=1.0, cutoff=2.2)
    batch = make()
    assert batch.positions.dtype == F64
    dyn = NVE(model, dt=0.05, hooks=model.make_neighbor_hooks())
    dyn.run(batch, n_steps=20)
    assert batch.positions.dtype == F64 and batch.forces.dtype == F64
    # the same loop with the oracle: forces of the start, then 20 x (half kick + drift, build, forces, half kick)
    h = np.full(len(ptr) - 1, float(dyn._state.dt[0]))
    Pr, Vr = P.copy(), np.zeros_like(P)
    M = np.ones(N)

    def forces(Pn):
        e = f64.nl_brute(Pn, C, pb, ptr, 2.2)
        K = 96
        nm = np.full((N, K), N, np.int32); nn = np.zeros(N, np.int32); sh = np.zeros((N, K, 3), np.int32)
        for i, j, sx, sy, sz in e:
            nm[i, nn[i]] = j; sh[i, nn[i]] = (sx, sy, sz); nn[i] += 1
        return f64.lj_matrix(Pn, C, nm, sh, nn, bi, N, 1.0, 1.0, 2.2)

    Fr = np.zeros_like(P)  # (the dynamics does not prime the forces: the first kick sees zeros)
    for _ in range(20):
        f64.vv_pre(Pr, Vr, Fr, M, h, bi)
        out = forces(Pr)
        Fr = out["forces"]
        f64.vv_post(Vr, Fr, M, h, bi)
    assert np.abs(batch.positions.cpu().numpy() - Pr).max() < 1e-10
    assert np.abs(batch.forces.cpu().numpy() - Fr).max() < 1e-9 * max(1.0, np.abs(Fr).max())
    assert np.abs(batch.energy.cpu().numpy().ravel() - out["energy"]).max() < 1e-10 * np.abs(out["energy"]).max()
    # and FIRE accepts the same batch
    b2 = make()
    e0 = None
    relax = FIRE(model, dt=0.005, hooks=model.make_neighbor_hooks())
    for k in range(30):
        relax.step(b2)
        if k == 0:
            e0 = b2.energy.clone()
    assert b2.energy.dtype == F64 and bool((b2.energy < e0).all())
    # ... and so do FIRE 2.0 and the two thermostats: every array stays float64, the relaxation goes downhill, the
    # thermostats heat a lattice at rest towards their temperature
    from nvalchemi_amd.dynamics import FIRE2, NVTLangevin, NVTNoseHoover

    b3 = make()
    relax2 = FIRE2(model, dt=0.005, hooks=model.make_neighbor_hooks())
    for k in range(30):
        relax2.step(b3)
        if k == 0:
            e0 = b3.energy.clone()
    assert b3.positions.dtype == F64 and b3.energy.dtype == F64 and bool((b3.energy < e0).all())
    for make_dyn in (lambda: NVTLangevin(model, dt=0.05, temperature=3000.0, friction=0.5, hooks=model.make_neighbor_hooks()),
                     lambda: NVTNoseHoover(model, dt=0.05, temperature=3000.0, thermostat_time=2.0,
                                           hooks=model.make_neighbor_hooks())):
        b4 = make()
        dyn4 = make_dyn()
        dyn4.run(b4, n_steps=40)
        assert b4.positions.dtype == F64 and b4.velocities.dtype == F64 and dyn4._state.dt.dtype == F64
        v = b4.velocities
        assert bool(torch.isfinite(v).all()) and float((v * v).sum()) > 0.0


def test_skin_test_and_wrap_on_float64_arrays():
    """The Verlet-skin displacement test and the periodic wrap on float64 arrays against the float64 oracle:
    flags and refreshed references to the bit, wrapped positions to the bit (both sides compute in double, one
    operation at a time), and a displacement of threshold (1 +- 1e-12) on the right side."""
    from nvalchemi_amd import _lib
    from nvalchemi_amd.hooks.periodic import wrap_positions_into_cell

    P, C, pb, ptr = periodic_batch(7, 3, 30, 60, 0.05, triclinic=True)
    pb = pb.copy()
    pb[1] = [1, 0, 1]
    bi = oracle.batch_idx_from_ptr(ptr)
    B = len(ptr) - 1
    rng = np.random.default_rng(7)
    P64 = P.astype(np.float64) + rng.normal(0, 1e-9, P.shape)       # values float32 does not hold
    C64 = C.astype(np.float64) * (1 + 1e-10)
    cur = P64.copy()
    moved = bi != 2
    cur[moved] += rng.normal(0, 0.08, (int(moved.sum()), 3))
    cur[0] += 2 * C64[0][0] - C64[0][1]
    for cell, pbc in ((None, None), (C64, pb)):
        for thr in (0.05, 0.2, 0.6):
            ref = P64.copy()
            want = f64.rebuild_check(ref, cur, bi, B, thr, update_reference=True, cell=cell, pbc=pbc)
            ref_t, flags = T(P64), torch.ones(B, dtype=torch.bool, device=DEV)
            _lib.nl_rebuild_check(ref_t, T(cur), T(bi), flags, thr, True, None if cell is None else T(C64),
                                  None if pbc is None else T(pb).bool())
            assert np.array_equal(flags.cpu().numpy(), want.astype(bool))
            assert np.array_equal(ref_t.cpu().numpy(), ref)
    thr = 0.25
    for eps, want in ((+1e-12, True), (-1e-12, False)):
        c2 = np.zeros((2, 3))
        c2[1] = np.array([0.6, 0.0, 0.8]) * thr * (1 + eps)
        flags = torch.zeros(1, dtype=torch.bool, device=DEV)
        _lib.nl_rebuild_check(T(np.zeros((2, 3))), T(c2), T(np.zeros(2, dtype=np.int32)), flags, thr, False)
        assert bool(flags[0]) == want
    far = cur * 3.0 - 5.0
    want = f64.wrap_positions(far, C64, pb, bi)
    got = wrap_positions_into_cell(T(far), T(C64), T(pb).bool(), T(bi))
    assert got.dtype == torch.float64 and np.array_equal(got.cpu().numpy(), want)


def test_thermostats_and_fire2_on_float64_arrays():
    """The Langevin half step, the Nose-Hoover chain and its drift, and FIRE 2.0 on float64 arrays against the float64
    oracle.  Bars: the drift bit for bit; the rest to 1e-12 relative to the largest value (exp, log, sin and cos differ
    by a rounding between the device's library and the host's; the device sums in another order), the integer
    counters exactly."""
    from nvalchemi_amd import _lib

    rng = np.random.default_rng(21)
    N, M = 901, 7
    counts = rng.multinomial(N, np.ones(M) / M)
    counts[4] = 0
    counts[0] += N - counts.sum()
    bi = np.repeat(np.arange(M, dtype=np.int32), counts)
    P, V, F = rng.normal(size=(N, 3)) * 3.0, rng.normal(size=(N, 3)) * 0.05, rng.normal(size=(N, 3))  # (m v^2 about kT)
    mass = rng.uniform(1, 30, N)
    dt, kT, gamma = rng.uniform(0.05, 0.3, M), rng.uniform(0.02, 0.05, M), rng.uniform(0.1, 2.0, M)
    act = np.array([1, 0, 1, 1, 1, 0, 1], dtype=np.uint8)
    close = lambda got, want, tol=1e-12: np.abs(got.cpu().numpy() - want).max() <= tol * max(1.0, np.abs(want).max())  # noqa: E731

    for active in (None, act):
        a_t = None if active is None else T(active)
        # Langevin
        Pd, Vd = T(P), T(V)
        _lib.langevin_half_step(Pd, Vd, T(F), T(mass), T(dt), T(kT), T(gamma), (1 << 40) + 12345, T(bi), a_t)
        Pr, Vr = P.copy(), V.copy()
        f64.langevin_half_step(Pr, Vr, F, mass, dt, kT, gamma, (1 << 40) + 12345, bi, active)
        assert Pd.dtype == F64 and close(Pd, Pr) and close(Vd, Vr)
        if active is not None:
            off = active[bi] == 0
            assert np.array_equal(Pd.cpu().numpy()[off], P[off]) and np.array_equal(Vd.cpu().numpy()[off], V[off])
        # the chain, computing the kinetic energy and taking it from the caller
        ndof = 3.0 * np.maximum(counts, 1)
        for C, order in ((1, 1), (3, 3), (5, 5)):
            Q = oracle.nhc_masses(kT, np.full(M, 0.4), ndof, C).astype(np.float64)
            eta0, eta_dot0 = rng.normal(size=(M, C)) * 0.05, rng.normal(size=(M, C)) * 0.05
            for supplied in (False, True):
                Vd, e_d, d_d = T(V), T(eta0), T(eta_dot0)
                k2_in = rng.uniform(0.5, 2.0, M) * ndof * kT
                k2_d = T(k2_in) if supplied else torch.zeros(M, dtype=F64, device=DEV)
                sc_d = torch.ones(M, dtype=F64, device=DEV)
                _lib.nhc_chain_update(Vd, T(mass), e_d, d_d, T(Q), T(kT), T(dt), T(ndof), k2_d, sc_d, T(bi),
                                      compute_ke=not supplied, yoshida_order=order, active=a_t)
                Vr, e_r, d_r = V.copy(), eta0.copy(), eta_dot0.copy()
                k2_r, sc_r = f64.nhc_chain_update(Vr, mass, e_r, d_r, Q, kT, dt, ndof, bi, ke2=k2_in if supplied else None,
                                                  active=active, yoshida_order=order)
                live = np.ones(M, bool) if active is None else active.astype(bool)
                assert close(Vd, Vr) and close(e_d, e_r) and close(d_d, d_r), (C, order, supplied)
                assert np.allclose(k2_d.cpu().numpy()[live], k2_r[live], rtol=1e-12)
                assert np.allclose(sc_d.cpu().numpy()[live], sc_r[live], rtol=1e-12)
        # the drift
        Pd = T(P)
        _lib.nhc_position_update(Pd, T(V), T(dt), T(bi), a_t)
        Pr = P.copy()
        f64.nhc_position_update(Pr, V, dt, bi, active)
        assert np.array_equal(Pd.cpu().numpy(), Pr)

    # FIRE 2.0: fifteen steps on a quadratic bowl, from velocities that point uphill in some systems; one system
    # frozen; a maxstep that binds in the first steps
    x0 = rng.normal(size=(N, 3))
    Vs = np.where(np.isin(bi, [1, 3])[:, None], 0.1 * (P - x0), V)  # (systems 1 and 3 start against their forces)
    alpha_r, dt_r, n_r = np.full(M, 0.09), np.full(M, 0.02), np.zeros(M, np.int32)
    alpha_d, dt_d, n_d = T(alpha_r), T(dt_r), T(n_r)
    outs = {k: torch.zeros(M, dtype=F64, device=DEV) for k in ("vf", "v_sumsq", "f_sumsq", "max_norm")}
    Pd, Vd, Pr, Vr = T(P), T(Vs), P.copy(), Vs.copy()
    frozen = np.array([1, 1, 1, 1, 1, 1, 0], dtype=np.uint8)
    par = dict(delaystep=4, dtgrow=1.1, dtshrink=0.5, alphashrink=0.99, alpha0=0.09, tmax=0.1, tmin=0.001, maxstep=0.05)
    for step in range(15):
        Fr = -2.0 * (Pr - x0)
        _lib.fire2_step(Pd, Vd, T(Fr), T(bi), alpha_d, dt_d, n_d, outs["vf"], outs["v_sumsq"], outs["f_sumsq"],
                        outs["max_norm"], active=T(frozen), **par)
        want = f64.fire2_step(Pr, Vr, Fr, bi, alpha_r, dt_r, n_r, active=frozen, **par)
        assert close(Pd, Pr) and close(Vd, Vr), step
        assert np.array_equal(n_d.cpu().numpy(), n_r), step
        assert np.allclose(dt_d.cpu().numpy(), dt_r, rtol=1e-14) and np.allclose(alpha_d.cpu().numpy(), alpha_r, rtol=1e-14)
        for k in ("vf", "v_sumsq", "f_sumsq"):
            assert np.allclose(outs[k].cpu().numpy(), want[k], rtol=1e-12, atol=1e-12), (k, step)
        has_atoms = (counts > 0) & (frozen != 0)
        assert np.allclose(outs["max_norm"].cpu().numpy()[has_atoms], want["max_norm"][has_atoms], rtol=1e-12)
        Pd.copy_(T(Pr)); Vd.copy_(T(Vr))  # (both sides continue from the same state)
    assert n_r.max() > par["delaystep"] and (n_r[[1, 3]] < 15).all()  # (both branches and the growth were met)
    assert np.array_equal(Pr[bi == 6], P[bi == 6])
