"""The oracle's FIRE 2.0 step (oracle/md_oracle.c: orc_fire2_step).  The reference's step is inside an
absent library and its own tests only ask that positions move (test/dynamics/test_ops.py:868-921), so
nothing pins the numbers: what is checked is what the published algorithm fixes -- the semi-implicit
Euler limit, the reset with its half step back, the bounds on the time step and on the displacement,
the counter and its delay -- and that it relaxes systems to their minimum.
"""

import numpy as np

import oracle


def state(M, dt=0.05, alpha=0.09):
    return (np.full(M, alpha, np.float32), np.full(M, dt, np.float32), np.zeros(M, np.int32))


def test_first_step_from_rest_is_a_plain_kick_and_drift_and_the_reference_cases_move():
    # the reference's own cases: zero velocities, random forces, two systems / one system
    rng = np.random.default_rng(7)
    for M, N in ((2, 8), (1, 4), (2, 6)):
        pos = rng.normal(0, 1, (N, 3)).astype(np.float32)
        vel = np.zeros((N, 3), np.float32)
        frc = rng.normal(0, 1, (N, 3)).astype(np.float32)
        sizes = [N // M] * M
        sizes[-1] += N - sum(sizes)
        bidx = np.repeat(np.arange(M), sizes).astype(np.int32)
        alpha, dt, cnt = state(M)
        p0 = pos.copy()
        out = oracle.fire2_step(pos, vel, frc, bidx, alpha, dt, cnt)
        assert not np.allclose(pos, p0)
        # P = 0 counts as not downhill: alpha restarts, the step shrinks, v = dt F, r += dt v
        h = np.float32(0.05) * np.float32(0.75)
        assert np.all(dt == h) and np.all(alpha == np.float32(0.09)) and np.all(cnt == 0)
        assert np.array_equal(vel, h * frc) and np.array_equal(pos, p0 + h * (h * frc))
        assert np.all(out["vf"] == 0) and np.all(out["v_sumsq"] == 0)
        assert np.allclose(out["f_sumsq"], [float((frc[bidx == s].astype(np.float64) ** 2).sum()) for s in range(M)])


def test_downhill_step_mixes_after_the_kick_and_counts_towards_the_delay():
    rng = np.random.default_rng(1)
    N = 6
    bidx = np.zeros(N, np.int32)
    frc = rng.normal(0, 1, (N, 3)).astype(np.float32)
    vel = (0.3 * frc + 0.05 * rng.normal(0, 1, (N, 3))).astype(np.float32)  # mostly along the force
    pos = rng.normal(0, 1, (N, 3)).astype(np.float32)
    # no mixing: the semi-implicit Euler step v += dt F, r += dt v
    alpha, dt, cnt = state(1, dt=0.01, alpha=0.0)
    p, v = pos.copy(), vel.copy()
    oracle.fire2_step(p, v, frc, bidx, alpha, dt, cnt, alpha0=0.0, maxstep=10.0)
    h = np.float32(0.01)
    assert np.array_equal(v, vel + h * frc) and np.array_equal(p, pos + h * (vel + h * frc)) and cnt[0] == 1
    assert dt[0] == h
    # mixing: factors from the entry's alpha, |v| and |F|, applied to the kicked velocity
    alpha, dt, cnt = state(1, dt=0.01, alpha=0.09)
    p, v = pos.copy(), vel.copy()
    out = oracle.fire2_step(p, v, frc, bidx, alpha, dt, cnt, maxstep=10.0)
    b = 0.09 * np.sqrt((vel.astype(np.float64) ** 2).sum() / (frc.astype(np.float64) ** 2).sum())
    want = (1 - 0.09) * (vel + h * frc).astype(np.float64) + b * frc
    assert np.allclose(v, want, rtol=1e-6, atol=1e-8) and np.allclose(p, pos + h * want, rtol=1e-6, atol=1e-7)
    assert out["vf"][0] > 0 and alpha[0] == np.float32(0.09) and dt[0] == h  # within the delay: nothing adapts
    # past the delay the step grows up to tmax and alpha decays
    alpha, dt, cnt = state(1, dt=0.07, alpha=0.09)
    cnt[0] = 60
    oracle.fire2_step(pos.copy(), vel.copy(), frc, bidx, alpha, dt, cnt)
    assert cnt[0] == 61 and dt[0] == np.float32(0.07) * np.float32(1.05) and alpha[0] == np.float32(0.09) * np.float32(0.985)
    for _ in range(2):
        oracle.fire2_step(pos.copy(), vel.copy(), frc, bidx, alpha, dt, cnt)
    assert dt[0] == np.float32(0.08) and cnt[0] == 63


def test_uphill_step_goes_half_a_step_back_and_restarts():
    rng = np.random.default_rng(2)
    N = 5
    bidx = np.zeros(N, np.int32)
    frc = rng.normal(0, 1, (N, 3)).astype(np.float32)
    vel = (-0.4 * frc).astype(np.float32)
    pos = rng.normal(0, 1, (N, 3)).astype(np.float32)
    alpha, dt, cnt = state(1, dt=0.04, alpha=0.02)
    cnt[0] = 17
    p, v = pos.copy(), vel.copy()
    out = oracle.fire2_step(p, v, frc, bidx, alpha, dt, cnt, maxstep=10.0)
    h_old, h = np.float32(0.04), np.float32(0.04) * np.float32(0.75)
    assert out["vf"][0] < 0 and cnt[0] == 0 and alpha[0] == np.float32(0.09) and dt[0] == h
    assert np.array_equal(v, h * frc)
    assert np.array_equal(p, (pos - (np.float32(0.5) * h_old) * vel) + h * (h * frc))
    # the step never shrinks below tmin
    alpha, dt, cnt = state(1, dt=0.006)
    oracle.fire2_step(pos.copy(), vel.copy(), frc, bidx, alpha, dt, cnt)
    assert dt[0] == np.float32(0.006)
    # a masked system keeps everything
    bidx2 = np.array([0, 0, 1, 1, 1], np.int32)
    alpha, dt, cnt = state(2, dt=0.04)
    p, v = pos.copy(), vel.copy()
    oracle.fire2_step(p, v, frc, bidx2, alpha, dt, cnt, active=[0, 1])
    assert np.array_equal(p[:2], pos[:2]) and np.array_equal(v[:2], vel[:2]) and dt[0] == np.float32(0.04)
    assert not np.array_equal(p[2:], pos[2:]) and dt[1] == np.float32(0.03)


def test_the_largest_displacement_of_a_system_is_limited_by_scaling_its_whole_step():
    rng = np.random.default_rng(3)
    bidx = np.array([0, 0, 0, 1, 1], np.int32)
    frc = rng.normal(0, 1, (5, 3)).astype(np.float32)
    frc[1] *= 50.0   # one fast atom in system 0
    vel = (2.0 * frc).astype(np.float32)
    pos = np.zeros((5, 3), np.float32)
    alpha, dt, cnt = state(2, dt=0.05, alpha=0.0)
    p, v = pos.copy(), vel.copy()
    out = oracle.fire2_step(p, v, frc, bidx, alpha, dt, cnt, alpha0=0.0, maxstep=0.1)
    step = np.linalg.norm(p - pos, axis=1)
    free = np.linalg.norm(np.float32(0.05) * v, axis=1)
    assert np.isclose(out["max_norm"][0], free[:3].max(), rtol=1e-6) and out["max_norm"][0] > 0.1
    assert np.isclose(step[:3].max(), 0.1, rtol=1e-5) and np.allclose(step[:3] / free[:3], 0.1 / free[:3].max(), rtol=1e-5)
    # the velocities are not touched by the limit, and system 1 is limited by its own largest step
    assert np.array_equal(v, vel + np.float32(0.05) * frc)
    assert np.isclose(step[3:].max(), min(0.1, free[3:].max()), rtol=1e-5)


def test_relaxes_a_quadratic_bowl_and_a_lennard_jones_cluster_to_the_minimum():
    # anisotropic bowl, two systems of different stiffness in one batch
    rng = np.random.default_rng(4)
    N = 12
    bidx = np.repeat([0, 1], 6).astype(np.int32)
    k = np.where(bidx[:, None] == 0, 1.0, 6.0) * (1.0 + rng.random((N, 3)))
    pos = rng.normal(0, 1, (N, 3)).astype(np.float32)
    vel = np.zeros((N, 3), np.float32)
    alpha, dt, cnt = state(2, dt=0.02)
    energy = lambda p: 0.5 * (k * p.astype(np.float64) ** 2).sum()
    e0 = energy(pos)
    seen_dt = []
    for _ in range(600):
        oracle.fire2_step(pos, vel, (-k * pos).astype(np.float32), bidx, alpha, dt, cnt, delaystep=5)
        seen_dt.append(dt.copy())
    seen_dt = np.array(seen_dt)
    assert energy(pos) < 1e-8 * e0 and np.abs(k * pos).max() < 1e-3
    assert seen_dt.min() >= 0.005 and seen_dt.max() <= np.float32(0.08) and seen_dt.max() > 0.05

    # 13-atom LJ cluster (reduced units): forces below 1e-3 and the icosahedron's energy -44.3268
    def lj(p):
        d = p[:, None, :] - p[None, :, :]
        r2 = (d ** 2).sum(-1) + np.eye(len(p))
        s6 = 1.0 / r2 ** 3
        e = 4.0 * (s6 * s6 - s6)
        np.fill_diagonal(e, 0.0)
        g = 24.0 * (2.0 * s6 * s6 - s6) / r2
        np.fill_diagonal(g, 0.0)
        return 0.5 * e.sum(), (g[:, :, None] * d).sum(1)

    phi = (1 + 5 ** 0.5) / 2
    ico = np.array([[0, s1, s2 * phi] for s1 in (-1, 1) for s2 in (-1, 1)])
    ico = np.concatenate([ico, np.roll(ico, 1, axis=1), np.roll(ico, 2, axis=1), [[0, 0, 0]]])
    ico = ico / np.linalg.norm(ico[0]) * 1.15 + rng.normal(0, 0.05, (13, 3))
    pos = ico.astype(np.float32)
    vel = np.zeros((13, 3), np.float32)
    bidx = np.zeros(13, np.int32)
    alpha, dt, cnt = state(1, dt=0.01)
    for it in range(3000):
        e, f = lj(pos.astype(np.float64))
        if np.abs(f).max() < 1e-3:
            break
        oracle.fire2_step(pos, vel, f.astype(np.float32), bidx, alpha, dt, cnt, delaystep=10, tmax=0.03)
    assert it < 2500 and abs(e - (-44.326801)) < 1e-3, (it, e)
