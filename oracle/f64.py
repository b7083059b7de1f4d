"""CPU restatement of the hot path for float64 inputs (numpy; test infrastructure only).

The reference's ops take float32 or float64 arrays (nvalchemi/dynamics/_ops/_bridge.py ``_vec_type`` /
``_scalar_type``; nvalchemi/dynamics/_ops/fire.py:281-287; nvalchemi/models/_ops/lj.py:116-216).  These
functions state the same definitions as ``oracle/md_oracle.c`` does for float32 inputs, on doubles,
one IEEE operation per numpy operation (numpy does not fuse multiply-adds):

* ``nl_brute``        the pair (i, j, S) is a neighbor iff ``d = (r_j - r_i) + (S0 a0 + S1 a1 + S2 a2)``,
                      ``(d0 d0 + d1 d1) + d2 d2 < rc rc`` (nvalchemi/models/_ops/neighbor_filter.py:98-119)
* ``lj_matrix``       nvalchemi/models/_ops/lj.py:116-216, 246-321; nvalchemi/models/lj.py:467-477
* ``vv_pre/vv_post``  nvalchemi/dynamics/_ops/velocity_verlet.py:50-92, 102-138
* ``fire_step``       nvalchemi/dynamics/_ops/fire.py:245-362, order of :270-272
* ``fmax``            nvalchemi/dynamics/base.py:304-349
* ``rebuild_check``   nvalchemi/dynamics/_ops/neighbor_list_rebuild.py:37-139 (flags cleared, then set for
                      systems with an atom displaced by more than the threshold, strictly; nearest image on
                      periodic axes when the cell is given; the whole flagged system's reference refreshed)
* ``wrap_positions``  nvalchemi/hooks/periodic.py:42-114, 159-163 (fractional coordinates mod 1, back to
                      Cartesian, per Cartesian component where that component's pbc flag is set)
* ``langevin_half_step``  nvalchemi/dynamics/_ops/langevin.py:52-117 (B-A-O-A; the same normal deviates as the
                      float32 oracle, which are made in double from the seed and the atom index)
* ``nhc_chain_update / nhc_position_update``  nvalchemi/dynamics/_ops/nose_hoover.py:143-246, 291-325
* ``fire2_step``      nvalchemi/dynamics/_ops/fire.py:467-557

Pinned (tests/test_oracle_f64.py) against the float32 oracle on inputs that float32 holds exactly
(where both must agree: to the bit for the neighbor sets, to float32 rounding elsewhere), against
closed forms in double (the Lennard-Jones dimer, F = -dE/dr by finite differences at 1e-9, the
discrete harmonic oscillator), and by pairs that only double resolves around the cutoff.  What the
float32 oracle leaves unpinned against the reference (FIRE's order beyond the reference's sentences,
the switching polynomial, the energy at the cutoff; for the skin test: strictness, the nearest-image form,
the whole-system refresh) is unpinned here in the same way.  ``rebuild_check`` and ``wrap_positions`` are
pinned against the float32 oracle on inputs float32 holds exactly and by what the definitions fix (a wrapped
position lies in the cell and differs from the old one by whole lattice vectors; a displacement of
``threshold (1 +- 1e-12)``, which float32 cannot tell from the threshold, lands on the right side).
The thermostats and FIRE 2.0 are PARITY UNPINNED against the reference like their float32 forms (their kernels
are in the absent library); here they are pinned against the float32 oracle on inputs float32 holds exactly
(agreement to float32 rounding) and by what their definitions fix in double: without friction the Langevin half
step is the velocity-Verlet drift; without forces and noise the velocity decays by exp(-gamma dt); a chain at rest
with the kinetic energy at its target does not move; a chain of one link follows its closed form; a FIRE 2.0 step
with P <= 0 steps half a step back, stops, and kicks once.
"""

from __future__ import annotations

import itertools

import numpy as np


def _inv_cell(h):
    return np.linalg.inv(h)


def nl_brute(positions, cell, pbc, batch_ptr, cutoff: float, half: bool = False) -> np.ndarray:
    """All ``(i, j, sx, sy, sz)`` inside the cutoff, canonical (lexicographic) order, int64."""
    pos = np.asarray(positions, dtype=np.float64)
    ptr = np.asarray(batch_ptr, dtype=np.int64)
    B = len(ptr) - 1
    out = []
    rc2 = float(cutoff) * float(cutoff)
    for s in range(B):
        lo, hi = int(ptr[s]), int(ptr[s + 1])
        n = hi - lo
        if n == 0:
            continue
        p = pos[lo:hi]
        if cell is None or pbc is None:
            h = np.eye(3)
            per = np.zeros(3, bool)
        else:
            h = np.asarray(cell, dtype=np.float64).reshape(B, 3, 3)[s]
            per = np.asarray(pbc).reshape(B, 3)[s].astype(bool)
        hinv = _inv_cell(h) if per.any() else np.eye(3)
        width = 1.0 / np.linalg.norm(hinv, axis=0) if per.any() else np.ones(3)
        R = [int(np.ceil(cutoff / width[d])) if per[d] else 0 for d in range(3)]
        frac = p @ hinv
        df = frac[None, :, :] - frac[:, None, :]  # [i, j] = frac_j - frac_i
        base = np.where(per[None, None, :], -np.rint(df), 0.0)
        dr = p[None, :, :] - p[:, None, :]
        ii, jj = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
        for o in itertools.product(*[range(-r, r + 1) for r in R]):
            S = base + np.asarray(o, dtype=np.float64)[None, None, :]
            t = [(S[..., 0] * h[0, k] + S[..., 1] * h[1, k]) + S[..., 2] * h[2, k] for k in range(3)]
            d = [dr[..., k] + t[k] for k in range(3)]
            r2 = (d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]
            hit = r2 < rc2
            hit &= ~((ii == jj) & (S[..., 0] == 0) & (S[..., 1] == 0) & (S[..., 2] == 0))
            if half:
                Si = S.astype(np.int64)
                pos_shift = (Si[..., 0] > 0) | ((Si[..., 0] == 0) & ((Si[..., 1] > 0) | ((Si[..., 1] == 0) & (Si[..., 2] > 0))))
                hit &= (ii < jj) | ((ii == jj) & pos_shift)
            a, b = np.nonzero(hit)
            if len(a):
                rec = np.empty((len(a), 5), dtype=np.int64)
                rec[:, 0] = a + lo
                rec[:, 1] = b + lo
                rec[:, 2:] = S[a, b].astype(np.int64)
                out.append(rec)
    if not out:
        return np.zeros((0, 5), dtype=np.int64)
    e = np.concatenate(out)
    return e[np.lexsort((e[:, 4], e[:, 3], e[:, 2], e[:, 1], e[:, 0]))]


def lj_matrix(positions, cells, neighbor_matrix, shifts, num_neighbors, batch_idx, fill_value, epsilon, sigma,
              cutoff, half=False, virial=False, switch_width=0.0):
    """dict(atomic_energies (N), forces (N,3), energy (B)[, virials (B,9)]), all float64."""
    pos = np.asarray(positions, dtype=np.float64)
    N = pos.shape[0]
    nm = np.asarray(neighbor_matrix)
    nn = np.asarray(num_neighbors)
    bi = np.asarray(batch_idx).astype(np.int64)
    h = np.asarray(cells, dtype=np.float64).reshape(-1, 3, 3)
    B = h.shape[0]
    K = nm.shape[1] if nm.ndim == 2 else 0
    valid = np.arange(K)[None, :] < np.minimum(nn, K)[:, None] if K else np.zeros((N, 0), bool)
    i, k = np.nonzero(valid)
    j = nm[i, k].astype(np.int64)
    ok = (j >= 0) & (j < min(int(fill_value), N))
    i, k, j = i[ok], k[ok], j[ok]
    S = np.zeros((len(i), 3)) if shifts is None else np.asarray(shifts)[i, k].astype(np.float64)
    hs = h[bi[i]]
    t = [(S[:, 0] * hs[:, 0, c] + S[:, 1] * hs[:, 1, c]) + S[:, 2] * hs[:, 2, c] for c in range(3)]
    d = np.stack([(pos[j, c] - pos[i, c]) + t[c] for c in range(3)], axis=1)
    r2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
    inside = r2 < float(cutoff) * float(cutoff)
    i, j, d, r2 = i[inside], j[inside], d[inside], r2[inside]
    ir2 = 1.0 / r2
    q2 = (sigma * sigma) * ir2
    q6 = q2 * q2 * q2
    q12 = q6 * q6
    u = (4.0 * epsilon) * (q12 - q6)
    g = -((24.0 * epsilon) * (2.0 * q12 - q6)) * ir2  # u'(r)/r
    if switch_width > 0.0:
        r = np.sqrt(r2)
        r_on = cutoff - switch_width
        tt = np.where(r > r_on, (r - r_on) / switch_width, 0.0)
        Sw = 1.0 - tt ** 3 * (10.0 - 15.0 * tt + 6.0 * tt * tt)
        dS = -30.0 * tt * tt * (1.0 - tt) ** 2 / switch_width
        g = g * Sw + u * dS / r
        u = u * Sw
    e = np.zeros(N)
    f = np.zeros((N, 3))
    np.add.at(e, i, 0.5 * u)
    np.add.at(f, i, g[:, None] * d)
    if half:
        np.add.at(e, j, 0.5 * u)
        np.add.at(f, j, -g[:, None] * d)
    es = np.zeros(B)
    np.add.at(es, bi, e)
    out = {"atomic_energies": e, "forces": f, "energy": es}
    if virial:
        w = np.zeros((B, 3, 3))
        hg = (-g if half else -0.5 * g)
        np.add.at(w, bi[i], hg[:, None, None] * d[:, :, None] * d[:, None, :])
        out["virials"] = w.reshape(B, 9)
    return out


def vv_pre(positions, velocities, forces, masses, dt, batch_idx, active=None):
    """In place: a = F/m; v += a (dt/2); r += v dt (each operation rounded once)."""
    bi = np.asarray(batch_idx).astype(np.int64)
    h = np.asarray(dt, dtype=np.float64)[bi][:, None]
    on = np.ones(len(bi), bool) if active is None else np.asarray(active).astype(bool)[bi]
    a = forces / np.asarray(masses, dtype=np.float64)[:, None]
    vh = velocities + a * (0.5 * h)
    dr = vh * h
    velocities[on] = vh[on]
    positions[on] = (positions + dr)[on]


def vv_post(velocities, forces, masses, dt, batch_idx, active=None):
    bi = np.asarray(batch_idx).astype(np.int64)
    h = np.asarray(dt, dtype=np.float64)[bi][:, None]
    on = np.ones(len(bi), bool) if active is None else np.asarray(active).astype(bool)[bi]
    a = forces / np.asarray(masses, dtype=np.float64)[:, None]
    velocities[on] = (velocities + a * (0.5 * h))[on]


def fire_step(positions, velocities, forces, masses, state: dict, batch_idx, active=None):
    """In place, the order of ``orc_fire_step``: sums over the arrays as passed in; MD integration with
    the stored dt (kick, drift limited to maxstep per atom); mixing with the stored alpha or reset;
    update of dt, alpha, n_steps_positive."""
    bi = np.asarray(batch_idx).astype(np.int64)
    M = len(state["alpha"])
    on_s = np.ones(M, bool) if active is None else np.asarray(active).astype(bool)
    P = np.zeros(M)
    VV = np.zeros(M)
    FF = np.zeros(M)
    np.add.at(P, bi, (forces * velocities).sum(1))
    np.add.at(VV, bi, (velocities * velocities).sum(1))
    np.add.at(FF, bi, (forces * forces).sum(1))
    state["vf"][:], state["vv"][:], state["ff"][:] = P, VV, FF
    h_use = state["dt"].copy()
    ma = np.ones(M)
    mb = np.zeros(M)
    for s in range(M):
        if not on_s[s]:
            continue
        h = state["dt"][s]
        if P[s] >= 0.0:
            al = state["alpha"][s]
            ma[s] = 1.0 - al
            mb[s] = al * np.sqrt(VV[s] / FF[s]) if FF[s] > 0.0 else 0.0
            state["n_steps_positive"][s] += 1
            if state["n_steps_positive"][s] > state["n_min"][s]:
                h = min(h * state["f_inc"][s], state["dt_max"][s])
                state["alpha"][s] = al * state["f_alpha"][s]
        else:
            ma[s] = mb[s] = 0.0
            state["n_steps_positive"][s] = 0
            h = max(h * state["f_dec"][s], state["dt_min"][s])
            state["alpha"][s] = state["alpha_start"][s]
        state["dt"][s] = h
    on = on_s[bi]
    h = h_use[bi][:, None]
    v = velocities + h * (forces / np.asarray(masses, dtype=np.float64)[:, None])
    v = np.clip(v, -1.0e300, 1.0e300)
    dr = h * v
    big = np.abs(dr).max(1)
    safe = np.where(big > 0.0, big, 1.0)
    a = dr / safe[:, None]
    nrm = np.where(big > 0.0, big * np.sqrt((a[:, 0] * a[:, 0] + a[:, 1] * a[:, 1]) + a[:, 2] * a[:, 2]), 0.0)
    ms = np.asarray(state["maxstep"], dtype=np.float64)[bi]
    over = nrm > ms
    sc = np.where(over, ms / np.where(over, nrm, 1.0), 1.0)
    dr = np.where(over[:, None], dr * sc[:, None], dr)
    velocities[on] = ((ma[bi][:, None] * v) + (mb[bi][:, None] * forces))[on]
    positions[on] = (positions + dr)[on]


def fmax(forces, batch_idx, n_systems: int) -> np.ndarray:
    f = np.asarray(forces, dtype=np.float64)
    n = np.sqrt((f[:, 0] * f[:, 0] + f[:, 1] * f[:, 1]) + f[:, 2] * f[:, 2])
    out = np.full(n_systems, -np.inf)
    np.maximum.at(out, np.asarray(batch_idx).astype(np.int64), n)
    return out


def _inv3(h):
    """The adjugate-over-determinant inverse in the operation order of oracle/md_oracle.c (orc_inv3)."""
    m = np.asarray(h, dtype=np.float64).reshape(9)
    c00 = m[4] * m[8] - m[5] * m[7]
    c01 = m[5] * m[6] - m[3] * m[8]
    c02 = m[3] * m[7] - m[4] * m[6]
    det = m[0] * c00 + m[1] * c01 + m[2] * c02
    i = 1.0 / det
    return np.array([c00 * i, (m[2] * m[7] - m[1] * m[8]) * i, (m[1] * m[5] - m[2] * m[4]) * i,
                     c01 * i, (m[0] * m[8] - m[2] * m[6]) * i, (m[2] * m[3] - m[0] * m[5]) * i,
                     c02 * i, (m[1] * m[6] - m[0] * m[7]) * i, (m[0] * m[4] - m[1] * m[3]) * i])


def rebuild_check(reference_positions, current_positions, batch_idx, n_systems: int, threshold: float,
                  update_reference: bool = False, cell=None, pbc=None) -> np.ndarray:
    """Flags ``(M,) uint8``; ``reference_positions`` (float64, C-contiguous) is refreshed in place for the atoms
    of flagged systems when ``update_reference``."""
    ref = reference_positions
    assert ref.dtype == np.float64
    cur = np.asarray(current_positions, dtype=np.float64)
    bi = np.asarray(batch_idx, dtype=np.int64)
    flags = np.zeros(int(n_systems), dtype=np.uint8)
    thr2 = float(threshold) * float(threshold)
    for i in range(len(cur)):
        s = bi[i]
        d = cur[i] - ref[i]
        if cell is not None and pbc is not None and np.any(pbc[s]):
            h = np.asarray(cell[s], dtype=np.float64).reshape(9)
            hv = _inv3(h)
            f = np.array([(d[0] * hv[0] + d[1] * hv[3]) + d[2] * hv[6],
                          (d[0] * hv[1] + d[1] * hv[4]) + d[2] * hv[7],
                          (d[0] * hv[2] + d[1] * hv[5]) + d[2] * hv[8]])
            for k in range(3):
                if pbc[s][k]:
                    f[k] -= np.rint(f[k])
            d = np.array([(f[0] * h[0] + f[1] * h[3]) + f[2] * h[6],
                          (f[0] * h[1] + f[1] * h[4]) + f[2] * h[7],
                          (f[0] * h[2] + f[1] * h[5]) + f[2] * h[8]])
        if (d[0] * d[0] + d[1] * d[1]) + d[2] * d[2] > thr2:
            flags[s] = 1
    if update_reference:
        hit = flags[bi] != 0
        ref[hit] = cur[hit]
    return flags


def wrap_positions(positions, cell, pbc, batch_idx) -> np.ndarray:
    """Wrapped copy of ``positions`` (float64)."""
    pos = np.array(positions, dtype=np.float64)
    bi = np.asarray(batch_idx, dtype=np.int64)
    for i in range(len(pos)):
        s = bi[i]
        if not np.any(pbc[s]):
            continue
        h = np.asarray(cell[s], dtype=np.float64).reshape(9)
        hv = _inv3(h)
        x, y, z = pos[i]
        f = np.array([(x * hv[0] + y * hv[3]) + z * hv[6], (x * hv[1] + y * hv[4]) + z * hv[7],
                      (x * hv[2] + y * hv[5]) + z * hv[8]])
        f -= np.floor(f)
        w = np.array([(f[0] * h[0] + f[1] * h[3]) + f[2] * h[6], (f[0] * h[1] + f[1] * h[4]) + f[2] * h[7],
                      (f[0] * h[2] + f[1] * h[5]) + f[2] * h[8]])
        for k in range(3):
            if pbc[s][k]:
                pos[i, k] = w[k]
    return pos


# ---------------------------------------------------------------------------------------------
# Langevin, Nose-Hoover chain, FIRE 2.0: the definitions of md_oracle.c's orc_langevin_half_step,
# orc_nhc_chain_update, orc_nhc_position_update and orc_fire2_step on doubles
# ---------------------------------------------------------------------------------------------
def langevin_half_step(positions, velocities, forces, masses, dt, kT, friction, seed, batch_idx, active=None):
    """In place on float64 ``positions`` / ``velocities``:
    v += (F/m)(dt/2); r += v (dt/2); v = c1 v + c2 xi; r += v (dt/2), c1 = exp(-gamma dt),
    c2 = sqrt((kT/m)(1 - c1^2)); xi(seed, atom) as in the float32 oracle."""
    from . import langevin_normals

    assert positions.dtype == np.float64 and velocities.dtype == np.float64
    bi = np.asarray(batch_idx).astype(np.int64)
    N = len(bi)
    on = np.ones(N, bool) if active is None else np.asarray(active).astype(bool)[bi]
    m = np.asarray(masses, dtype=np.float64)
    h = np.asarray(dt, dtype=np.float64)[bi]
    hh = 0.5 * h
    c1 = np.exp(-np.asarray(friction, dtype=np.float64)[bi] * h)
    c2 = np.sqrt((np.asarray(kT, dtype=np.float64)[bi] / m) * (1.0 - c1 * c1))
    xi = np.array([langevin_normals(seed, i)[:3] for i in range(N)], dtype=np.float64).reshape(N, 3)
    acc = np.asarray(forces, dtype=np.float64) / m[:, None]
    v = velocities + acc * hh[:, None]
    r = positions + v * hh[:, None]
    v = c1[:, None] * v + c2[:, None] * xi
    r = r + v * hh[:, None]
    velocities[on] = v[on]
    positions[on] = r[on]


def _ys_weights(order: int):
    if order == 3:
        a = 1.0 / (2.0 - np.cbrt(2.0))
        return [a, 1.0 - 2.0 * a, a]
    if order == 5:
        a = 1.0 / (4.0 - np.cbrt(4.0))
        return [a, a, 1.0 - 4.0 * a, a, a]
    return [1.0]


def nhc_chain_update(velocities, masses, eta, eta_dot, Q, kT, dt, ndof, batch_idx, ke2=None, active=None,
                     yoshida_order=3):
    """In place on float64 ``velocities (N,3)``, ``eta`` and ``eta_dot (M,C)``; returns ``(ke2, total_scale)``.
    The propagator of ``orc_nhc_chain_update`` (Martyna, Tuckerman, Tobias, Klein 1996), every value a double."""
    import math

    assert velocities.dtype == np.float64 and eta.dtype == np.float64 and eta_dot.dtype == np.float64
    bi = np.asarray(batch_idx).astype(np.int64)
    M, C = eta.shape
    m = np.asarray(masses, dtype=np.float64)
    if ke2 is None:
        v = velocities
        k2_all = np.bincount(bi, weights=m * ((v[:, 0] * v[:, 0] + v[:, 1] * v[:, 1]) + v[:, 2] * v[:, 2]), minlength=M)
    else:
        k2_all = np.asarray(ke2, dtype=np.float64).copy()
    scale_all = np.ones(M)
    on_s = np.ones(M, bool) if active is None else np.asarray(active).astype(bool)
    out_k2 = k2_all.copy() if ke2 is not None else np.where(on_s, k2_all, 0.0)  # (computed sums: live systems only)
    for s in range(M):
        if not on_s[s]:
            continue
        u = [float(x) for x in eta_dot[s]]
        x = [float(t) for t in eta[s]]
        q = [float(t) for t in np.asarray(Q, dtype=np.float64)[s]]
        kt, nf, h = float(kT[s]), float(ndof[s]), float(dt[s])
        k2, scale = float(k2_all[s]), 1.0

        def g_of(k):
            return (k2 - nf * kt) / q[0] if k == 0 else (q[k - 1] * u[k - 1] * u[k - 1] - kt) / q[k]

        for w in _ys_weights(yoshida_order):
            d = w * h
            d2, d4, d8 = 0.5 * d, 0.25 * d, 0.125 * d
            u[C - 1] += g_of(C - 1) * d4
            for k in range(C - 2, -1, -1):
                aa = math.exp(-d8 * u[k + 1])
                u[k] = (u[k] * aa + g_of(k) * d4) * aa
            sc = math.exp(-d2 * u[0])
            scale *= sc
            k2 *= sc * sc
            for k in range(C):
                x[k] += d2 * u[k]
            for k in range(C - 1):
                aa = math.exp(-d8 * u[k + 1])
                u[k] = (u[k] * aa + g_of(k) * d4) * aa
            u[C - 1] += g_of(C - 1) * d4
        eta_dot[s] = u
        eta[s] = x
        scale_all[s] = scale
    on = on_s[bi]
    velocities[on] = (velocities * scale_all[bi][:, None])[on]
    return out_k2, scale_all


def nhc_position_update(positions, velocities, dt, batch_idx, active=None):
    """In place: r += v dt."""
    assert positions.dtype == np.float64
    bi = np.asarray(batch_idx).astype(np.int64)
    on = np.ones(len(bi), bool) if active is None else np.asarray(active).astype(bool)[bi]
    h = np.asarray(dt, dtype=np.float64)[bi][:, None]
    positions[on] = (positions + np.asarray(velocities, dtype=np.float64) * h)[on]


def fire2_step(positions, velocities, forces, batch_idx, alpha, dt, nsteps_inc, active=None, **params):
    """In place on float64 ``positions``, ``velocities`` (N,3), ``alpha``, ``dt`` (M) and int32 ``nsteps_inc`` (M);
    returns ``dict(vf, v_sumsq, f_sumsq, max_norm)``.  The step of ``orc_fire2_step``, every value a double."""
    from . import FIRE2_DEFAULTS

    for a in (positions, velocities, alpha, dt):
        assert a.dtype == np.float64
    p = dict(FIRE2_DEFAULTS)
    p.update(params)
    bi = np.asarray(batch_idx).astype(np.int64)
    f = np.asarray(forces, dtype=np.float64)
    M = alpha.shape[0]
    on_s = np.ones(M, bool) if active is None else np.asarray(active).astype(bool)
    P = np.bincount(bi, weights=(f * velocities).sum(1), minlength=M)
    VV = np.bincount(bi, weights=(velocities * velocities).sum(1), minlength=M)
    FF = np.bincount(bi, weights=(f * f).sum(1), minlength=M)
    ma, mb, back, up = np.ones(M), np.zeros(M), np.zeros(M), np.zeros(M, bool)
    for s in range(M):
        if not on_s[s]:
            continue
        if P[s] > 0.0:
            al = alpha[s]
            up[s] = True
            ma[s] = 1.0 - al
            mb[s] = al * np.sqrt(VV[s] / FF[s]) if FF[s] > 1e-20 else 0.0
            nsteps_inc[s] += 1
            if nsteps_inc[s] > p["delaystep"]:
                dt[s] = min(dt[s] * p["dtgrow"], p["tmax"])
                alpha[s] = al * p["alphashrink"]
        else:
            nsteps_inc[s] = 0
            alpha[s] = p["alpha0"]
            back[s] = 0.5 * dt[s]
            nd = dt[s] * p["dtshrink"]
            if nd >= p["tmin"]:
                dt[s] = nd
    on = on_s[bi]
    up_a = up[bi][:, None]
    h = dt[bi][:, None]
    r = np.where(up_a, positions, positions - back[bi][:, None] * velocities)
    v = np.where(up_a, velocities, 0.0)
    v = v + h * f
    v = np.where(up_a, ma[bi][:, None] * v + mb[bi][:, None] * f, v)
    v = np.clip(v, -1.0e300, 1.0e300)
    dr = h * v
    top = np.abs(dr).max(1) if len(bi) else np.zeros(0)
    safe = np.where(top > 0.0, top, 1.0)
    a = dr / safe[:, None]
    nrm = np.where(top > 0.0, top * np.sqrt((a[:, 0] * a[:, 0] + a[:, 1] * a[:, 1]) + a[:, 2] * a[:, 2]), 0.0)
    big = np.zeros(M)
    np.maximum.at(big, bi[on], nrm[on])
    sc = np.where(big > p["maxstep"], p["maxstep"] / np.where(big > 0.0, big, 1.0), 1.0)
    dr = (h * v) * sc[bi][:, None]
    velocities[on] = v[on]
    positions[on] = (r + dr)[on]
    max_norm = np.where(on_s, big, 0.0)
    return {"vf": P, "v_sumsq": VV, "f_sumsq": FF, "max_norm": max_norm}
