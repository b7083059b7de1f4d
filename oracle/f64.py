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
