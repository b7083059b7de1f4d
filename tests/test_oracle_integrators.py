"""Pins the oracle's integrators (CPU only).

Velocity Verlet: literal one-step values from the reference's docstring formulas
(nvalchemi/dynamics/_ops/velocity_verlet.py:63-64,112), the closed form of the discrete
harmonic oscillator and time reversibility.  FIRE: the order of the step is the one the
reference's own sentences give (MD integration first, then velocity mixing, then the parameter
update, with the sums of entry: nvalchemi/dynamics/_ops/fire.py:270-272,
nvalchemi/dynamics/_dynamics_coordinator.py:296-340), and each sentence is a check with literal
numbers that another order fails; what no sentence decides (the sub-step of the integration, the
norm of the clamp, P = 0, > against >= at n_min) is the restatement's choice and stays unpinned
against the reference, whose kernel is in a library that the tree does not hold.  The invariants
(dt bounds, counters, descent to the minimum) are checked on top.  fmax: literal cases of
nvalchemi/dynamics/base.py:304-349.
"""

import numpy as np
import pytest

import oracle


def test_vv_literal_single_step():
    r = np.array([[1.0, 0, 0]], dtype=np.float32)
    v = np.array([[2.0, 0, 0]], dtype=np.float32)
    F = np.array([[3.0, 0, 0]], dtype=np.float32)
    m = np.array([4.0], dtype=np.float32)
    dt = np.array([0.5], dtype=np.float32)
    oracle.vv_pre(r, v, F, m, dt, [0])
    # r + v dt + 1/2 (F/m) dt^2 = 1 + 1 + 0.09375 ; v + 1/2 (F/m) dt = 2 + 0.1875
    assert r[0, 0] == np.float32(2.09375) and v[0, 0] == np.float32(2.1875)
    oracle.vv_post(v, np.array([[-1.0, 0, 0]], dtype=np.float32), m, dt, [0])
    assert v[0, 0] == np.float32(2.125)


def test_vv_per_system_dt_and_active_mask():
    r = np.zeros((3, 3), dtype=np.float32)
    v = np.ones((3, 3), dtype=np.float32)
    F = np.zeros((3, 3), dtype=np.float32)
    m = np.ones(3, dtype=np.float32)
    dt = np.array([0.5, 2.0, 1.0], dtype=np.float32)
    oracle.vv_pre(r, v, F, m, dt, [0, 1, 2], active=[1, 1, 0])
    assert np.array_equal(r[:, 0], np.array([0.5, 2.0, 0.0], dtype=np.float32))


def test_vv_harmonic_oscillator_closed_form_and_reversibility():
    k, m0, h, n = 2.0, 1.5, 0.05, 400
    r = np.array([[1.0, -0.5, 0.25]], dtype=np.float32)
    v = np.zeros((1, 3), dtype=np.float32)
    r0 = r.copy()
    m = np.array([m0], dtype=np.float32)
    dt = np.array([h], dtype=np.float32)
    F = (-k * r).astype(np.float32)
    for _ in range(n):
        oracle.vv_pre(r, v, F, m, dt, [0])
        F = (-k * r).astype(np.float32)
        oracle.vv_post(v, F, m, dt, [0])
    # velocity Verlet on a harmonic force is a rotation by theta per step, cos(theta) = 1 - (w h)^2/2
    w2 = k / m0
    theta = np.arccos(1.0 - w2 * h * h / 2)
    assert np.allclose(r, r0 * np.cos(n * theta), atol=2e-4)
    v *= -1
    for _ in range(n):
        oracle.vv_pre(r, v, F, m, dt, [0])
        F = (-k * r).astype(np.float32)
        oracle.vv_post(v, F, m, dt, [0])
    assert np.allclose(r, r0, atol=2e-4) and np.abs(v).max() < 2e-4


def _fire_state(M, dt=0.1, **kw):
    f32 = lambda x: np.full(M, x, dtype=np.float32)  # noqa: E731
    st = dict(alpha=f32(0.1), dt=f32(dt), alpha_start=f32(0.1), f_alpha=f32(0.99),
              dt_min=f32(0.02 * dt), dt_max=f32(10 * dt), maxstep=f32(0.2), f_dec=f32(0.5),
              f_inc=f32(1.1), vf=f32(0), vv=f32(0), ff=f32(0),
              n_steps_positive=np.zeros(M, dtype=np.int32), n_min=np.full(M, 5, dtype=np.int32))
    for k_, v_ in kw.items():
        st[k_][:] = v_
    return st


def _one_atom(v0, F0):
    r = np.zeros((1, 3), dtype=np.float32)
    v = np.array([[v0, 0, 0]], dtype=np.float32)
    F = np.array([[F0, 0, 0]], dtype=np.float32)
    return r, v, F, np.ones(1, dtype=np.float32)


def test_fire_integrates_first_then_mixes_with_the_reductions_of_entry():
    """nvalchemi/dynamics/_ops/fire.py:270-272: "an MD integration step followed by FIRE velocity mixing
    and adaptive parameter updates".  One atom, v = 1, F = 2, m = 1, dt = 0.1, alpha = 0.1; the expected
    numbers come from that sentence and from the reductions being those of the arrays passed in
    (nvalchemi/distributed/_dynamics_coordinator.py:296-322), not from the oracle's code:
      kick   v1 = 1 + 0.1*2 = 1.2 ; drift r = 0.1*1.2 = 0.12
      mix    |v|/|F| from entry = 1/2 :  v = 0.9*1.2 + 0.1*0.5*2 = 1.18
    The orders this rules out give other numbers:
      mix first, then integrate (Bitzek/ASE):   v = (0.9*1 + 0.1) + 0.2 = 1.2,  r = 0.12
      reductions after the kick (|v1|/|F| = .6): v = 0.9*1.2 + 0.1*0.6*2 = 1.2
      drift with the mixed velocity:             r = 0.118
    """
    r, v, F, m = _one_atom(1.0, 2.0)
    st = _fire_state(1)
    oracle.fire_step(r, v, F, m, st, [0])
    assert st["vf"][0] == 2 and st["vv"][0] == 1 and st["ff"][0] == 4  # of the entry arrays
    assert r[0, 0] == pytest.approx(0.12, rel=1e-6)
    assert v[0, 0] == pytest.approx(1.18, rel=1e-6)
    assert abs(float(v[0, 0]) - 1.2) > 1e-3
    assert st["n_steps_positive"][0] == 1 and st["dt"][0] == np.float32(0.1) and st["alpha"][0] == np.float32(0.1)


def test_fire_uphill_step_is_integrated_with_the_stored_dt_before_the_reset():
    """F.v < 0 at entry: the integration still happens first, with the time step of before the
    update, and only then are the velocities zeroed and dt halved.  A mix-first order would move the
    atom by dt'^2 F/m = -0.005 with the halved dt' and leave v = dt' F/m = -0.1."""
    r, v, F, m = _one_atom(1.0, -2.0)
    st = _fire_state(1)
    st["n_steps_positive"][:] = 3
    oracle.fire_step(r, v, F, m, st, [0])
    assert r[0, 0] == pytest.approx(0.1 * (1.0 - 0.2), rel=1e-6)  # dt (v + dt F/m) with dt = 0.1
    assert v[0, 0] == 0.0
    assert st["dt"][0] == np.float32(0.05) and st["alpha"][0] == np.float32(0.1) and st["n_steps_positive"][0] == 0


def test_fire_the_time_step_grown_by_a_step_is_first_used_by_the_next():
    """Parameter updates come last: the step that grows dt (n+ passes n_min) still integrates with
    the old one."""
    r, v, F, m = _one_atom(1.0, 2.0)
    st = _fire_state(1)
    st["n_steps_positive"][:] = 5
    oracle.fire_step(r, v, F, m, st, [0])
    assert r[0, 0] == pytest.approx(0.12, rel=1e-6)  # 0.1 * 1.2, not 0.11 * 1.22
    assert st["dt"][0] == pytest.approx(0.11, rel=1e-6) and st["alpha"][0] == pytest.approx(0.099, rel=1e-6)
    v1 = float(v[0, 0])
    oracle.fire_step(r, v, F, m, st, [0])
    assert r[0, 0] == pytest.approx(0.12 + 0.11 * (v1 + 0.11 * 2.0), rel=1e-6)


def test_fire_leaves_rest():
    """A system at rest has F.v = 0 on entry.  With the velocities reset AFTER the integration, that
    zero has to count as downhill, or the velocity gained by the kick would be thrown away on every
    step and the system would creep at dt_min for ever."""
    r, v, F, m = _one_atom(0.0, 2.0)
    st = _fire_state(1)
    oracle.fire_step(r, v, F, m, st, [0])
    assert v[0, 0] == pytest.approx(0.9 * 0.2, rel=1e-6) and r[0, 0] == pytest.approx(0.02, rel=1e-6)
    assert st["dt"][0] == np.float32(0.1) and st["n_steps_positive"][0] == 1
    oracle.fire_step(r, v, F, m, st, [0])
    assert st["vf"][0] > 0 and v[0, 0] > 0.18


def test_fire_dt_growth_after_n_min_and_caps():
    r = np.zeros((1, 3), dtype=np.float32)
    v = np.zeros((1, 3), dtype=np.float32)
    F = np.array([[1e-3, 0, 0]], dtype=np.float32)
    m = np.ones(1, dtype=np.float32)
    st = _fire_state(1, dt=0.1)
    dts, alphas = [], []
    for _ in range(60):
        oracle.fire_step(r, v, F, m, st, [0])
        dts.append(float(st["dt"][0]))
        alphas.append(float(st["alpha"][0]))
    # steps 1..5 are downhill steps 1..5 (no growth); growth starts at the 6th
    assert dts[0] == pytest.approx(0.1) and dts[4] == pytest.approx(0.1)
    assert dts[5] == pytest.approx(0.1 * 1.1, rel=1e-6) and alphas[5] == pytest.approx(0.099, rel=1e-6)
    assert max(dts) == pytest.approx(1.0, rel=1e-6)  # dt_max = 10 dt
    assert all(b >= a for a, b in zip(dts, dts[1:]))


def test_fire_maxstep_clamp_is_per_atom():
    r = np.zeros((2, 3), dtype=np.float32)
    v = np.zeros((2, 3), dtype=np.float32)
    F = np.array([[3e4, 4e4, 0], [1e-3, 0, 0]], dtype=np.float32)
    m = np.ones(2, dtype=np.float32)
    st = _fire_state(1)
    oracle.fire_step(r, v, F, m, st, [0, 0])
    assert np.linalg.norm(r[0]) == pytest.approx(0.2, rel=1e-5)
    assert r[0, 0] / r[0, 1] == pytest.approx(0.75, rel=1e-5)
    assert r[1, 0] == pytest.approx(0.1 * 0.1 * 1e-3, rel=1e-5)


def test_fire_relaxes_a_quadratic_bowl_and_respects_masks():
    rng = np.random.default_rng(0)
    n = 40
    r = rng.normal(0, 1, (n, 3)).astype(np.float32)
    v = np.zeros((n, 3), dtype=np.float32)
    m = rng.uniform(1, 3, n).astype(np.float32)
    bi = np.repeat(np.arange(4), 10).astype(np.int32)
    st = _fire_state(4, dt=0.05)
    frozen = r[bi == 3].copy()
    active = np.array([1, 1, 1, 0], dtype=np.uint8)
    for _ in range(300):
        F = (-1.5 * r).astype(np.float32)
        oracle.fire_step(r, v, F, m, st, bi, active=active)
        assert np.all(st["dt"] >= st["dt_min"]) and np.all(st["dt"] <= st["dt_max"])
    assert np.array_equal(r[bi == 3], frozen)
    assert oracle.fmax(-1.5 * r, bi, 4)[:3].max() < 1e-3


def test_fmax_is_max_atom_force_norm_per_system():
    F = np.array([[3, 4, 0], [0, 0, 1], [0, 0, 0], [1, 2, 2]], dtype=np.float32)
    out = oracle.fmax(F, [0, 0, 2, 2], 3)
    assert out[0] == 5 and out[1] == -np.inf and out[2] == 3


def test_segment_reductions_and_kinetic_energy_literals():
    """The per-system observables of nvalchemi/dynamics/hooks/_utils.py:172-290 on cases small enough
    to check by hand, including an empty system."""
    v = np.array([1.0, -2.0, 3.0, 0.5, 4.0], np.float32)
    idx = np.array([0, 0, 0, 2, 2], np.int32)
    assert oracle.segment_reduce(v, idx, 3, "sum").tolist() == [2.0, 0.0, 4.5]
    assert oracle.segment_reduce(v, idx, 3, "amax").tolist() == [3.0, -np.inf, 4.0]
    assert oracle.segment_reduce(v, idx, 3, "amin").tolist() == [-2.0, np.inf, 0.5]
    assert np.allclose(oracle.segment_reduce(v, idx, 3, "mean"), [2.0 / 3.0, 0.0, 2.25])
    vel = np.array([[1, 2, 2], [0, 3, 4], [1, 0, 0]], np.float32)
    m = np.array([2.0, 1.0, 4.0], np.float32)
    assert oracle.kinetic_energy(vel, m, np.array([0, 0, 1], np.int32), 3).tolist() == [9.0 + 12.5, 2.0, 0.0]
    # T = 2 KE / (3 N kB): one atom of mass m and speed v has T = m v^2 / (3 kB)
    kb = 8.617333262e-5
    ke = oracle.kinetic_energy(np.array([[0.1, 0, 0]], np.float32), np.array([12.0], np.float32), [0], 1)[0]
    assert abs(2 * ke / (3 * 1 * kb) - 12.0 * 0.01 / (3 * kb)) < 1e-3


def test_fire_with_its_default_parameters_stays_finite_on_an_overlapped_start():
    """The order integrate -> mix damps the first kicks less than mix -> integrate would.  A moderately
    overlapped start (a jittered lattice of argon-sized atoms, closest pairs at 0.85 sigma) relaxed with the
    optimizer's defaults (maxstep 0.2 A, alpha 0.1, dt_max 10 dt, dt_min 0.02 dt) must stay finite and end
    lower in energy; a random gas, whose closest pairs sit far up the repulsive wall, is what needs a
    shorter leash (bench.py relaxes with maxstep 0.07 sigma)."""
    rng = np.random.default_rng(4)
    sigma, eps, rc = 3.4, 0.0104, 8.5
    m = 4
    a = 1.12 * sigma
    L = m * a
    grid = np.stack(np.meshgrid(*[np.arange(m)] * 3, indexing="ij"), -1).reshape(-1, 3) * a
    P = (grid + rng.uniform(-0.135, 0.135, grid.shape) * sigma).astype(np.float32)
    n = len(P)
    C = (np.eye(3, dtype=np.float32) * L).reshape(1, 3, 3)
    pb = np.ones((1, 3), dtype=np.uint8)
    ptr = np.array([0, n], dtype=np.int32)
    bi = np.zeros(n, dtype=np.int32)
    M = np.full(n, 39.948, dtype=np.float32)
    V = np.zeros_like(P)
    dt = 1.0
    f32 = lambda v: np.array([v], dtype=np.float32)  # noqa: E731
    state = dict(alpha=f32(0.1), dt=f32(dt), alpha_start=f32(0.1), f_alpha=f32(0.99), dt_min=f32(0.02 * dt),
                 dt_max=f32(10 * dt), maxstep=f32(0.2), f_dec=f32(0.5), f_inc=f32(1.1), vf=f32(0), vv=f32(0), ff=f32(0),
                 n_steps_positive=np.zeros(1, dtype=np.int32), n_min=np.array([5], dtype=np.int32))

    def forces():
        nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, 256)
        assert nn.max() < 256
        out = oracle.lj_matrix(P, C, nm, sh, nn, bi, n, eps, sigma, rc)
        return out["forces"], float(out["energy"][0])

    edges = oracle.nl_brute(P, C, pb, ptr, 0.9 * sigma)
    assert len(edges) > 0  # some pairs do start inside 0.9 sigma
    F, e0 = forces()
    fmax0 = float(np.abs(F).max())
    energies = [e0]
    for _ in range(300):
        oracle.fire_step(P, V, F, M, state, bi)
        assert np.isfinite(P).all() and np.isfinite(V).all()
        F, e = forces()
        energies.append(e)
    assert np.isfinite(energies).all()
    assert energies[-1] < e0 - 0.5 * abs(e0) or energies[-1] < e0 - 1.0
    assert float(np.abs(F).max()) < 0.1 * fmax0
