"""Pins the oracle's Lennard-Jones function (CPU only): closed forms, literal dimer
values, finite differences of the energy (forces, virial), Newton's third law and the
conventions the reference documents (nvalchemi/models/_ops/lj.py:31-45,167-168,270-273;
nvalchemi/models/lj.py:321-324,464-477)."""

import numpy as np
import pytest

import oracle
from _systems import fcc_boxes, periodic_batch

EPS, SIG = 0.01, 2.5


def _dimer(r, eps=EPS, sig=SIG, rc=100.0, half=False, virial=False):
    pos = np.array([[0.0, 0, 0], [r, 0, 0]], dtype=np.float32)
    nm = np.array([[1, 2], [0, 2]], dtype=np.int32)
    nn = np.array([1, 1], dtype=np.int32)
    if half:
        nm = np.array([[1, 2], [2, 2]], dtype=np.int32)
        nn = np.array([1, 0], dtype=np.int32)
    return oracle.lj_matrix(pos, np.eye(3)[None], nm, None, nn, [0, 0], 2, eps, sig, rc,
                            half=half, virial=virial)


def test_zero_crossing_at_sigma():
    out = _dimer(SIG)
    assert abs(out["energy"][0]) < 1e-9
    # u'(sigma) = -24 eps / sigma: repulsive, atom 0 pushed to -x
    assert out["forces"][0, 0] == pytest.approx(-24 * EPS / SIG, rel=1e-6)
    assert out["forces"][1, 0] == pytest.approx(+24 * EPS / SIG, rel=1e-6)


def test_minimum_at_two_to_one_sixth_sigma():
    out = _dimer(2 ** (1 / 6) * SIG)
    assert out["energy"][0] == pytest.approx(-EPS, rel=1e-6)
    assert np.abs(out["forces"]).max() < 1e-7
    assert np.allclose(out["atomic_energies"], -EPS / 2, rtol=1e-6)


def test_literal_value_at_one_and_a_half_sigma():
    # 4[(2/3)^12 - (2/3)^6] = 4 (4096/531441 - 64/729) = -0.32033659427858
    # -u'(r) sigma/eps = 24/1.5 (2 (2/3)^12 - (2/3)^6) = -1.1580288310462 (attractive)
    out = _dimer(1.5, eps=1.0, sig=1.0)
    assert out["energy"][0] == pytest.approx(-0.32033659427858, rel=2e-7)
    assert out["forces"][0, 0] == pytest.approx(+1.1580288310462, rel=2e-7)
    assert out["forces"][1, 0] == pytest.approx(-1.1580288310462, rel=2e-7)
    assert np.all(out["forces"][:, 1:] == 0)


def test_plain_truncation_and_strict_cutoff():
    assert _dimer(3.0, rc=3.0)["energy"][0] == 0.0
    inside = _dimer(2.999, eps=1.0, sig=1.0, rc=3.0)["energy"][0]
    assert inside == pytest.approx(4 * (2.999 ** -12 - 2.999 ** -6), rel=1e-5)  # no shift


def test_half_list_gives_the_same_totals():
    full = _dimer(1.2 * SIG, virial=True)
    half = _dimer(1.2 * SIG, half=True, virial=True)
    for k in ("atomic_energies", "forces", "energy", "virials"):
        assert np.allclose(full[k], half[k], rtol=1e-6, atol=1e-12), k


def _dyadic_cluster(seed, n, box, min_dist=0.8):
    rng = np.random.default_rng(seed)
    pts = []
    while len(pts) < n:
        p = rng.integers(0, int(box * 1024), 3) / 1024.0
        if all(np.linalg.norm(p - q) > min_dist for q in pts):
            pts.append(p)
    return np.array(pts, dtype=np.float32)


def _energy_fixed_list(P, C, ptr, nm, nn, sh, rc_eval):
    bi = oracle.batch_idx_from_ptr(ptr)
    cells = C if C is not None else np.eye(3)[None].repeat(len(ptr) - 1, 0)
    out = oracle.lj_matrix(P, cells, nm, sh, nn, bi, len(P), 1.0, 1.0, rc_eval)
    return out


def test_forces_are_minus_energy_gradient_cluster():
    P = _dyadic_cluster(0, 12, 3.0)
    ptr = np.array([0, 12], dtype=np.int32)
    nm, nn, sh = oracle.nl_cell(P, None, None, ptr, 2.5, 16)
    out = _energy_fixed_list(P, None, ptr, nm, nn, None, 10.0)
    h = 2.0 ** -9
    for i in (0, 5, 11):
        for a in range(3):
            Pp, Pm = P.copy(), P.copy()
            Pp[i, a] += h
            Pm[i, a] -= h
            ep = _energy_fixed_list(Pp, None, ptr, nm, nn, None, 10.0)["atomic_energies"].astype(np.float64).sum()
            em = _energy_fixed_list(Pm, None, ptr, nm, nn, None, 10.0)["atomic_energies"].astype(np.float64).sum()
            fd = -(ep - em) / (2 * h)
            assert out["forces"][i, a] == pytest.approx(fd, rel=5e-3, abs=2e-3)
    assert np.abs(out["forces"].astype(np.float64).sum(0)).max() < 1e-4 * np.abs(out["forces"]).max()


def test_forces_periodic_triclinic_match_gradient_and_sum_to_zero():
    P, C, pb, ptr = periodic_batch(7, 2, 20, 30, 0.6, triclinic=True)
    P = (np.round(P * 1024) / 1024).astype(np.float32)
    ref = oracle.nl_brute(P, C, pb, ptr, 2.0)
    # drop overlapping pairs so finite differences stay well conditioned
    K = int(np.bincount(ref[:, 0], minlength=len(P)).max()) + 1
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, 2.0, K)
    out = _energy_fixed_list(P, C, ptr, nm, nn, sh, 50.0)
    bi = oracle.batch_idx_from_ptr(ptr)
    F = out["forces"].astype(np.float64)
    for s in range(2):
        assert np.abs(F[bi == s].sum(0)).max() < 1e-5 * np.abs(F[bi == s]).max()
    assert np.allclose(out["energy"],
                       [out["atomic_energies"][bi == s].astype(np.float64).sum() for s in range(2)], rtol=1e-6)
    h = 2.0 ** -10
    i = int(np.argmin(np.abs(F).max(1)))  # the gentlest atom: smallest curvature
    for a in range(3):
        Pp, Pm = P.copy(), P.copy()
        Pp[i, a] += h
        Pm[i, a] -= h
        ep = _energy_fixed_list(Pp, C, ptr, nm, nn, sh, 50.0)["atomic_energies"].astype(np.float64).sum()
        em = _energy_fixed_list(Pm, C, ptr, nm, nn, sh, 50.0)["atomic_energies"].astype(np.float64).sum()
        fd = -(ep - em) / (2 * h)
        scale = max(1.0, abs(ep))
        assert F[i, a] == pytest.approx(fd, rel=2e-2, abs=2e-4 * scale / h * 1e-3 + 1e-2)


def test_virial_is_minus_strain_derivative_and_stress_sign():
    # compressed FCC (nearest neighbour 0.95 sigma): repulsive, so W_aa > 0 and stress = -W/V < 0
    P, C, pb, ptr = fcc_boxes(seed=1, n_boxes=1, reps=2, a=0.95 * np.sqrt(2.0), jitter=0.02)
    rc = 1.3
    ref = oracle.nl_brute(P, C, pb, ptr, rc)
    K = int(np.bincount(ref[:, 0]).max()) + 1
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, K)
    bi = oracle.batch_idx_from_ptr(ptr)

    def run(Pq, Cq):
        return oracle.lj_matrix(Pq, Cq, nm, sh, nn, bi, len(P), 1.0, 1.0, 10.0, virial=True)

    out = run(P, C)
    W = out["virials"].reshape(3, 3).astype(np.float64)
    assert np.allclose(W, W.T, rtol=1e-5, atol=1e-4)
    assert np.all(np.diag(W) > 0)
    eta = 2.0 ** -8
    for a, b in ((0, 0), (1, 1), (0, 1), (2, 0)):
        E = []
        for sgn in (+1, -1):
            D = np.eye(3)
            D[a, b] += sgn * eta / 2
            D[b, a] += sgn * eta / 2  # symmetric strain
            Pq = (P.astype(np.float64) @ D).astype(np.float32)
            Cq = (C[0].astype(np.float64) @ D).astype(np.float32)[None]
            E.append(run(Pq, Cq)["atomic_energies"].astype(np.float64).sum())
        dE = (E[0] - E[1]) / (2 * eta)
        # symmetric strain (eps_ab = eps_ba = eta/2 off-diagonal, eta on the diagonal)
        expect = -W[a, b] if a == b else -(W[a, b] + W[b, a]) / 2
        assert dE == pytest.approx(expect, rel=2e-3, abs=2e-2)


def test_per_system_energy_is_fp64_sum_of_rounded_atomic_energies():
    P, C, pb, ptr = periodic_batch(9, 3, 30, 60, 0.7)
    ref = oracle.nl_brute(P, C, pb, ptr, 2.5)
    K = int(np.bincount(ref[:, 0], minlength=len(P)).max()) + 1
    nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, 2.5, K)
    bi = oracle.batch_idx_from_ptr(ptr)
    out = oracle.lj_matrix(P, C, nm, sh, nn, bi, len(P), 1.0, 1.0, 2.5)
    exp = np.array([out["atomic_energies"][bi == s].astype(np.float64).sum() for s in range(3)]).astype(np.float32)
    assert np.array_equal(out["energy"], exp)


def _dimer_switched(r, width, rc=7.5):
    pos = np.array([[0.0, 0, 0], [r, 0, 0]], dtype=np.float32)
    nm = np.array([[1, 2], [0, 2]], dtype=np.int32)
    nn = np.array([1, 1], dtype=np.int32)
    return oracle.lj_matrix(pos, np.eye(3)[None], nm, None, nn, [0, 0], 2, EPS, SIG, rc, switch_width=width)


def test_switch_leaves_the_inner_region_alone_and_halves_the_energy_midway():
    rc, w = 7.5, 1.5
    for r in (2.6, 4.0, 5.99):  # below rc - w = 6.0
        a, b = _dimer_switched(r, w), _dimer_switched(r, 0.0)
        assert np.array_equal(a["forces"], b["forces"]) and np.array_equal(a["energy"], b["energy"])
    mid = rc - w / 2  # 6.75: exactly representable
    assert _dimer_switched(mid, w)["energy"][0] == pytest.approx(0.5 * _dimer_switched(mid, 0.0)["energy"][0], rel=1e-6)
    # S falls monotonically from 1 to 0
    ratios = [_dimer_switched(r, w)["energy"][0] / _dimer_switched(r, 0.0)["energy"][0]
              for r in np.linspace(6.0, 7.49, 12)]
    assert all(x > y for x, y in zip(ratios, ratios[1:])) and ratios[0] == pytest.approx(1.0) and ratios[-1] < 1e-4


def test_switched_force_is_minus_energy_gradient():
    rc, w, h = 7.5, 1.5, 2.0 ** -9
    for r in (6.125, 6.5, 6.75, 7.0, 7.375):
        ep = float(_dimer_switched(r + h, w)["energy"][0])
        em = float(_dimer_switched(r - h, w)["energy"][0])
        f1 = float(_dimer_switched(r, w)["forces"][1, 0])  # force on the atom at +x is -dE/dr
        assert f1 == pytest.approx(-(ep - em) / (2 * h), rel=2e-3, abs=1e-9), r


def test_switch_is_c2_at_both_ends():
    """Energy, force and force derivative meet the unswitched potential at r_on and vanish at the
    cutoff: with S ~ 1 - 10 t^3 near r_on and S ~ 10 (1 - t)^3 near the cutoff, the differences shrink
    with the third, second and first power of the distance to the end."""
    rc, w = 7.5, 1.5
    for d in (2.0 ** -4, 2.0 ** -6):
        t = d / w
        near_on_sw, near_on = _dimer_switched(6.0 + d, w), _dimer_switched(6.0 + d, 0.0)
        u = float(near_on["energy"][0])
        assert abs(float(near_on_sw["energy"][0]) - u) < 11 * t ** 3 * abs(u)
        f_sw, f = float(near_on_sw["forces"][1, 0]), float(near_on["forces"][1, 0])
        # |u S'| <= 30 t^2 |u| / w on top of the unswitched force
        assert abs(f_sw - f) < 31 * t ** 2 * abs(u) / w + 11 * t ** 3 * abs(f)
        near_rc_sw, near_rc = _dimer_switched(7.5 - d, w), _dimer_switched(7.5 - d, 0.0)
        u = float(near_rc["energy"][0])
        assert abs(float(near_rc_sw["energy"][0])) < 11 * t ** 3 * abs(u)
        assert abs(float(near_rc_sw["forces"][1, 0])) < 31 * t ** 2 * abs(u) / w + 11 * t ** 3 * abs(float(near_rc["forces"][1, 0]))
    # the force derivative is continuous: slopes across r_on agree
    h = 2.0 ** -7
    f = lambda r: float(_dimer_switched(r, w)["forces"][1, 0])  # noqa: E731
    slope_in = (f(6.0) - f(6.0 - h)) / h
    slope_out = (f(6.0 + h) - f(6.0)) / h
    g = lambda r: float(_dimer_switched(r, 0.0)["forces"][1, 0])  # noqa: E731
    plain = (g(6.0 + h) - g(6.0)) / h
    # (a switch that is only C1, such as 1 - 3 t^2 + 2 t^3, would add u S'' = 6 u / w^2: twice the slope itself)
    assert slope_out == pytest.approx(plain, rel=0.1)
    assert slope_in == pytest.approx(slope_out, rel=0.1)
