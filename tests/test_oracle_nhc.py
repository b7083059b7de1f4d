"""The oracle's Nose-Hoover chain propagator (oracle/md_oracle.c: orc_nhc_chain_update) against what
the mathematics fixes.  The reference's kernel is inside an absent library, so nothing the reference
holds pins the numbers; what is pinned here is that the restatement integrates the Nose-Hoover chain
equations of motion (Martyna, Klein, Tuckerman 1992; Martyna, Tuckerman, Tobias, Klein 1996):

    r' = v            v' = F/m - u_1 v            eta_k' = u_k
    u_1' = (sum m v^2 - N_f kT) / Q_1 - u_2 u_1
    u_k' = (Q_{k-1} u_{k-1}^2 - kT) / Q_k - u_{k+1} u_k        (last link: no friction term)

A dropped term, a wrong sign or a wrong sub-step length fails the second-order convergence to an
adaptive integration of these equations, the conservation of the extended energy or the reversal.
"""

import numpy as np
import pytest
from scipy.integrate import solve_ivp

import oracle

N = 5
KT = 0.7
RNG = np.random.default_rng(11)
MASS = (1.0 + RNG.random(N) * 2.0).astype(np.float32)
SPRING = 1.0 + RNG.random((N, 3)) * 3.0
R0 = RNG.normal(0, 0.5, (N, 3)).astype(np.float32)
V0 = RNG.normal(0, 1.0, (N, 3)).astype(np.float32)
BIDX = np.zeros(N, dtype=np.int32)


def force(r):
    """Anisotropic wells with a quartic term and a pair coupling (so that nothing is separable)."""
    r = np.asarray(r, dtype=np.float64)
    f = -SPRING * r - 0.3 * r ** 3
    d = r[:, None, :] - r[None, :, :]
    f -= 0.2 * d.sum(axis=1)
    return f


def potential(r):
    r = np.asarray(r, dtype=np.float64)
    d = r[:, None, :] - r[None, :, :]
    return float((0.5 * SPRING * r ** 2 + 0.075 * r ** 4).sum() + 0.05 * (d ** 2).sum())


def masses_of(chain, tau):
    return oracle.nhc_masses([KT], [tau], [3 * N], chain)


def run(n_steps, dt, chain, tau, order=3, r0=R0, v0=V0, eta0=None, u0=None):
    r, v = r0.copy(), v0.copy()
    eta = np.zeros((1, chain), np.float32) if eta0 is None else eta0.copy()
    u = np.zeros((1, chain), np.float32) if u0 is None else u0.copy()
    Q = masses_of(chain, tau)
    h = np.array([dt], np.float32)
    args = dict(Q=Q, kT=[KT], dt=h, ndof=[3 * N], batch_idx=BIDX, yoshida_order=order)
    f = force(r).astype(np.float32)
    for _ in range(n_steps):
        oracle.nhc_chain_update(v, MASS, eta, u, **args)
        oracle.vv_post(v, f, MASS, h, BIDX)
        oracle.nhc_position_update(r, v, h, BIDX)
        f = force(r).astype(np.float32)
        oracle.vv_post(v, f, MASS, h, BIDX)
        oracle.nhc_chain_update(v, MASS, eta, u, **args)
    return r, v, eta, u


def exact(t_end, chain, tau):
    Q = masses_of(chain, tau)[0].astype(np.float64)
    m = MASS.astype(np.float64)[:, None]
    nf = 3 * N

    def rhs(_, y):
        r, v = y[:3 * N].reshape(N, 3), y[3 * N:6 * N].reshape(N, 3)
        u = y[6 * N + chain:]
        du = np.empty(chain)
        for k in range(chain):
            g = ((m * v * v).sum() - nf * KT) / Q[0] if k == 0 else (Q[k - 1] * u[k - 1] ** 2 - KT) / Q[k]
            du[k] = g - (u[k + 1] * u[k] if k + 1 < chain else 0.0)
        return np.concatenate([v.ravel(), (force(r) / m - u[0] * v).ravel(), u, du])

    y0 = np.concatenate([R0.astype(np.float64).ravel(), V0.astype(np.float64).ravel(), np.zeros(2 * chain)])
    sol = solve_ivp(rhs, (0.0, t_end), y0, rtol=1e-11, atol=1e-12, method="DOP853")
    y = sol.y[:, -1]
    reached = np.abs(sol.y[6 * N + chain:]).max(axis=1)  # the largest value every chain velocity took
    return y[:3 * N].reshape(N, 3), y[3 * N:6 * N].reshape(N, 3), y[6 * N:6 * N + chain], y[6 * N + chain:], reached


def extended_energy(r, v, eta, u, chain, tau):
    Q = masses_of(chain, tau)[0].astype(np.float64)
    ke = 0.5 * float((MASS[:, None].astype(np.float64) * v.astype(np.float64) ** 2).sum())
    e = ke + potential(r) + 0.5 * float((Q * u[0].astype(np.float64) ** 2).sum())
    e += 3 * N * KT * float(eta[0, 0]) + KT * float(eta[0, 1:].astype(np.float64).sum())
    return e


@pytest.mark.parametrize("chain,order", [(1, 3), (3, 3), (3, 5), (4, 1)])
def test_the_step_converges_at_second_order_to_the_chain_equations_of_motion(chain, order):
    tau, t_end = 0.35, 1.2  # a tight thermostat: the chain velocities reach order one within the run
    r_x, v_x, eta_x, u_x, reached = exact(t_end, chain, tau)
    assert reached[0] > 0.3 and (chain == 1 or reached[1] > 0.05), reached
    errs = []
    for n in (48, 96, 192):
        r, v, eta, u = run(n, t_end / n, chain, tau, order)
        errs.append(max(np.abs(r - r_x).max(), np.abs(v - v_x).max(), np.abs(eta[0] - eta_x).max(),
                        np.abs(u[0] - u_x).max()))
    assert errs[0] < 1e-2 and errs[2] < errs[1] < errs[0]
    assert 3.3 < errs[0] / errs[1] < 4.8 and 3.0 < errs[1] / errs[2] < 5.0, errs


def test_the_extended_energy_is_conserved():
    chain, tau, dt = 3, 0.5, 0.01
    r, v, eta, u = R0, V0, None, None
    e0 = extended_energy(R0, V0, np.zeros((1, chain), np.float32), np.zeros((1, chain), np.float32), chain, tau)
    worst = 0.0
    for _ in range(20):
        r, v, eta, u = run(100, dt, chain, tau, r0=r, v0=v, eta0=eta, u0=u)
        worst = max(worst, abs(extended_energy(r, v, eta, u, chain, tau) - e0))
    # the thermostat exchanges several kT with the particles over the run; the sum stays put
    assert abs(3 * N * KT * float(eta[0, 0])) > 1.0
    assert worst < 2e-3, worst


def test_the_step_is_time_reversible():
    chain, tau, dt, n = 3, 0.5, 0.01, 150
    r, v, eta, u = run(n, dt, chain, tau)
    assert np.abs(r - R0).max() > 0.3
    rb, vb, etab, ub = run(n, dt, chain, tau, r0=r, v0=-v, eta0=eta, u0=-u)
    assert np.abs(rb - R0).max() < 2e-4 and np.abs(-vb - V0).max() < 2e-4
    assert np.abs(etab).max() < 2e-4 and np.abs(ub).max() < 2e-4


def test_arguments_outputs_masks_and_the_supplied_kinetic_energy():
    M, chain = 3, 2
    bidx = np.array([0, 0, 1, 1, 1, 2], np.int32)
    rng = np.random.default_rng(3)
    v0 = rng.normal(0, 1, (6, 3)).astype(np.float32)
    m = (1 + rng.random(6)).astype(np.float32)
    ndof = np.array([6, 9, 3], np.float32)
    kT = np.array([0.5, 1.0, 2.0], np.float32)
    Q = oracle.nhc_masses(kT, [0.4, 0.5, 0.6], ndof, chain)
    assert Q.shape == (M, chain) and np.allclose(Q[:, 1], kT * np.array([0.4, 0.5, 0.6]) ** 2)
    assert np.allclose(Q[:, 0], ndof * Q[:, 1])
    dt = np.array([0.02, 0.03, 0.04], np.float32)
    eta0 = rng.normal(0, 0.1, (M, chain)).astype(np.float32)
    u0 = rng.normal(0, 0.5, (M, chain)).astype(np.float32)

    v, eta, u = v0.copy(), eta0.copy(), u0.copy()
    ke2, scale = oracle.nhc_chain_update(v, m, eta, u, Q, kT, dt, ndof, bidx)
    want = np.array([(m[bidx == s, None].astype(np.float64) * v0[bidx == s].astype(np.float64) ** 2).sum()
                     for s in range(M)])
    assert np.allclose(ke2, want, rtol=1e-6)
    assert np.array_equal(v, v0 * scale[bidx][:, None])
    # to first order in dt the friction is the chain velocity: scale = exp(-u_1 dt/2) (1 + O(dt))
    assert np.allclose(scale, np.exp(-0.5 * dt * u0[:, 0]), rtol=0.05 * dt.max() * 10)
    assert np.allclose(eta - eta0, 0.5 * dt[:, None] * u0, atol=2e-3)

    # a masked system keeps everything
    v2, eta2, u2 = v0.copy(), eta0.copy(), u0.copy()
    oracle.nhc_chain_update(v2, m, eta2, u2, Q, kT, dt, ndof, bidx, active=[1, 0, 1])
    keep = bidx == 1
    assert np.array_equal(v2[keep], v0[keep]) and np.array_equal(eta2[1], eta0[1]) and np.array_equal(u2[1], u0[1])
    assert np.array_equal(v2[~keep], v[~keep]) and np.array_equal(u2[[0, 2]], u[[0, 2]])

    # a supplied sum m v^2 takes the place of the velocities' own
    v3, eta3, u3 = v0.copy(), eta0.copy(), u0.copy()
    ke2_in = (want * 3.0).astype(np.float32)
    oracle.nhc_chain_update(v3, m, eta3, u3, Q, kT, dt, ndof, bidx, ke2=ke2_in)
    assert not np.allclose(u3[:, 0], u[:, 0])
    v4 = (v0 * np.sqrt(3.0)).astype(np.float32)
    eta4, u4 = eta0.copy(), u0.copy()
    oracle.nhc_chain_update(v4, m, eta4, u4, Q, kT, dt, ndof, bidx)
    assert np.allclose(u3, u4, rtol=2e-6, atol=1e-7) and np.allclose(eta3, eta4, rtol=2e-6, atol=1e-7)

    # weights of the factorisation: one pass of the plain step, three or five summing to one
    pos = np.zeros((6, 3), np.float32)
    oracle.nhc_position_update(pos, v0, dt, bidx)
    assert np.array_equal(pos, v0 * dt[bidx][:, None])
