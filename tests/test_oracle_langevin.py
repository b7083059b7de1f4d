"""Pins the oracle's Langevin half step (CPU only).  The reference's random stream cannot be
matched (its generator is inside the absent kernel library), so the pins are mathematical: the
published known answers of Philox4x32-10, the moments of the normal deviates, the limits of the
step, and the invariance of the Maxwell-Boltzmann variance under the Ornstein-Uhlenbeck update."""

import numpy as np
import pytest

import oracle

KB_EV = 8.617333262e-5


def test_philox_known_answers():
    """Random123 kat_vectors, philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11)."""
    z = [0, 0, 0, 0]
    assert [hex(x) for x in oracle.philox4x32_10(z, [0, 0])] == ["0x6627e8d5", "0xe169c58d", "0xbc57ac4c", "0x9b00dbd8"]
    f = [0xFFFFFFFF] * 4
    assert [hex(x) for x in oracle.philox4x32_10(f, f[:2])] == ["0x408f276d", "0x41c83b0e", "0xa20bc7c6", "0x6d5451fd"]
    pi = [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344]
    assert [hex(x) for x in oracle.philox4x32_10(pi, [0xA4093822, 0x299F31D0])] == \
        ["0xd16cfe09", "0x94fdcceb", "0x5001e420", "0x24126ea1"]


def test_normal_deviates_have_the_right_moments_and_depend_on_seed_and_atom():
    xi = np.array([oracle.langevin_normals(7, i)[:3] for i in range(40000)]).ravel()
    n = len(xi)
    assert abs(xi.mean()) < 4 / np.sqrt(n) and abs(xi.var() - 1) < 4 * np.sqrt(2 / n)
    assert abs((xi ** 3).mean()) < 4 * np.sqrt(15 / n) and abs((xi ** 4).mean() - 3) < 4 * np.sqrt(96 / n)
    a = np.array([oracle.langevin_normals(7, i)[:3] for i in range(2000)])
    assert abs(np.corrcoef(a[:, 0], a[:, 1])[0, 1]) < 0.1 and abs(np.corrcoef(a[:-1, 0], a[1:, 0])[0, 1]) < 0.1
    assert not np.array_equal(oracle.langevin_normals(7, 3), oracle.langevin_normals(8, 3))
    assert np.array_equal(oracle.langevin_normals(7, 3), oracle.langevin_normals(7, 3))


def _state(n=6, seed=0):
    rng = np.random.default_rng(seed)
    return (rng.normal(0, 2, (n, 3)).astype(np.float32), rng.normal(0, 0.1, (n, 3)).astype(np.float32),
            rng.normal(0, 0.5, (n, 3)).astype(np.float32), rng.uniform(1, 40, n).astype(np.float32))


def test_without_friction_it_is_the_first_half_of_velocity_verlet():
    P, V, F, M = _state()
    bi = np.array([0, 0, 0, 1, 1, 1], np.int32)
    dt = np.array([0.05, 0.11], np.float32)
    p, v = P.copy(), V.copy()
    oracle.langevin_half_step(p, v, F, M, dt, np.array([0.02, 0.03], np.float32), np.zeros(2, np.float32), 5, bi)
    h = dt[bi][:, None].astype(np.float64)
    vh = V + F / M[:, None] * h / 2
    assert np.allclose(v, vh, rtol=1e-6, atol=1e-7) and np.allclose(p, P + vh * h, rtol=1e-6, atol=1e-6)
    # inactive systems are left alone
    p2, v2 = P.copy(), V.copy()
    oracle.langevin_half_step(p2, v2, F, M, dt, np.array([0.02, 0.03], np.float32), np.zeros(2, np.float32), 5, bi,
                              active=np.array([1, 0], np.uint8))
    assert np.array_equal(p2[3:], P[3:]) and np.array_equal(v2[3:], V[3:]) and np.array_equal(p2[:3], p[:3])


def test_infinite_friction_redraws_the_velocities_at_the_temperature():
    n = 30000
    rng = np.random.default_rng(1)
    P = np.zeros((n, 3), np.float32)
    V = rng.normal(0, 5, (n, 3)).astype(np.float32)  # far from equilibrium
    M = np.full(n, 12.0, np.float32)
    kT = np.array([300 * KB_EV], np.float32)
    v = V.copy()
    oracle.langevin_half_step(P.copy(), v, np.zeros_like(P), M, np.array([0.1], np.float32), kT,
                              np.array([1e4], np.float32), 11, np.zeros(n, np.int32))
    var = kT[0] / 12.0
    assert abs(v.mean()) < 4 * np.sqrt(var / (3 * n)) and abs(v.var() / var - 1) < 4 * np.sqrt(2 / (3 * n))
    # the deviates are the generator's: v = c2 xi exactly when c1 = 0
    xi = oracle.langevin_normals(11, 17)[:3]
    assert np.allclose(v[17], np.float32(np.sqrt(var)) * xi.astype(np.float32), rtol=1e-6)


@pytest.mark.parametrize("gamma_dt", [0.05, 0.7, 3.0])
def test_the_thermostat_keeps_the_maxwell_boltzmann_variance(gamma_dt):
    """c1^2 var + c2^2 = kT/m when var = kT/m: velocities drawn at the temperature stay there."""
    n = 40000
    rng = np.random.default_rng(2)
    m, T = 39.95, 150.0
    var = T * KB_EV / m
    V = rng.normal(0, np.sqrt(var), (n, 3)).astype(np.float32)
    v = V.copy()
    oracle.langevin_half_step(np.zeros((n, 3), np.float32), v, np.zeros((n, 3), np.float32), np.full(n, m, np.float32),
                              np.array([0.2], np.float32), np.array([T * KB_EV], np.float32),
                              np.array([gamma_dt / 0.2], np.float32), 3, np.zeros(n, np.int32))
    assert abs(v.var() / var - 1) < 5 * np.sqrt(2 / (3 * n))
    # and the memory of the old velocity decays as exp(-gamma dt)
    c1 = np.sum(v.astype(np.float64) * V) / np.sum(V.astype(np.float64) ** 2)
    assert abs(c1 - np.exp(-gamma_dt)) < 0.02
