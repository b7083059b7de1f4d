"""Seeded synthetic inputs shared by the oracle tests and the GPU parity tests."""

from __future__ import annotations

import numpy as np


def ptr_from_counts(counts):
    return np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)


def random_triclinic_cell(rng, length, angle_lo=60.0, angle_hi=120.0):
    """Lattice with |a|=|b|=|c|=length-ish and angles uniform in [lo, hi] degrees."""
    while True:
        al, be, ga = np.deg2rad(rng.uniform(angle_lo, angle_hi, 3))
        a, b, c = length * rng.uniform(0.8, 1.2, 3)
        ax = np.array([a, 0, 0])
        bx = np.array([b * np.cos(ga), b * np.sin(ga), 0])
        cx = c * np.cos(be)
        cy = c * (np.cos(al) - np.cos(be) * np.cos(ga)) / np.sin(ga)
        cz2 = c * c - cx * cx - cy * cy
        if cz2 <= (0.3 * c) ** 2:
            continue
        H = np.stack([ax, bx, np.array([cx, cy, np.sqrt(cz2)])])
        if np.linalg.det(H) > 0:
            return H.astype(np.float32)


def periodic_batch(seed, n_systems, n_lo, n_hi, density, triclinic=False, pbc=None, spread=0.0):
    """Random periodic systems; positions uniform in the cell, optionally spilled out by
    ``spread`` cell lengths (unwrapped coordinates)."""
    rng = np.random.default_rng(seed)
    counts = rng.integers(n_lo, n_hi + 1, n_systems)
    cells, pos = [], []
    for n in counts:
        L = (n / density) ** (1.0 / 3.0)
        H = random_triclinic_cell(rng, L) if triclinic else (np.eye(3) * L).astype(np.float32)
        f = rng.uniform(-spread, 1.0 + spread, (n, 3))
        pos.append((f @ H.astype(np.float64)).astype(np.float32))
        cells.append(H)
    P = np.concatenate(pos).astype(np.float32)
    C = np.stack(cells).astype(np.float32)
    if pbc is None:
        pb = np.ones((n_systems, 3), dtype=bool)
    else:
        pb = np.broadcast_to(np.asarray(pbc, dtype=bool), (n_systems, 3)).copy()
    return P, C, pb, ptr_from_counts(counts)


def molecules_batch(seed=0, n_systems=8, n_lo=4, n_hi=32, sigma_pos=1.5):
    """Non-periodic molecules: uniform atom count, positions N(0, sigma_pos), Z in {1,6,7,8}."""
    rng = np.random.default_rng(seed)
    counts = rng.integers(n_lo, n_hi + 1, n_systems)
    N = int(counts.sum())
    P = rng.normal(0.0, sigma_pos, (N, 3)).astype(np.float32)
    Z = rng.choice(np.array([1, 6, 7, 8]), N)
    mass_of = {1: 1.008, 6: 12.011, 7: 14.007, 8: 15.999}
    M = np.array([mass_of[int(z)] for z in Z], dtype=np.float32)
    return P, Z.astype(np.int64), M, ptr_from_counts(counts)


def fcc_boxes(seed=0, n_boxes=4, reps=5, a=3.6, jitter=0.05):
    """Cubic FCC boxes (reps^3 conventional cells, 4 atoms each) with Gaussian jitter."""
    rng = np.random.default_rng(seed)
    base = np.array([[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]])
    g = np.stack(np.meshgrid(*[np.arange(reps)] * 3, indexing="ij"), -1).reshape(-1, 1, 3)
    lat = ((g + base[None]) * a).reshape(-1, 3)
    n = lat.shape[0]
    P = np.concatenate([lat + rng.normal(0, jitter, lat.shape) for _ in range(n_boxes)])
    C = np.broadcast_to(np.eye(3) * reps * a, (n_boxes, 3, 3))
    pb = np.ones((n_boxes, 3), dtype=bool)
    return P.astype(np.float32), C.astype(np.float32).copy(), pb, ptr_from_counts([n] * n_boxes)


def sheared_fcc_boxes(seed=0, n_boxes=3, reps=3, a=1.5496, jitter=0.03, shear=0.25):
    """FCC boxes deformed by a random shear per box: triclinic cells without overlapping atoms."""
    rng = np.random.default_rng(seed)
    P, C, pb, ptr = fcc_boxes(seed=seed, n_boxes=n_boxes, reps=reps, a=a, jitter=jitter)
    P = P.astype(np.float64)
    C = C.astype(np.float64)
    for s in range(n_boxes):
        D = np.eye(3) + np.tril(rng.uniform(-shear, shear, (3, 3)), -1)
        P[ptr[s]:ptr[s + 1]] = P[ptr[s]:ptr[s + 1]] @ D
        C[s] = C[s] @ D
    return P.astype(np.float32), C.astype(np.float32), pb, ptr
