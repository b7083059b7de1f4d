"""Step loops driven by the CPU oracle, in the reference's order of operations
(nvalchemi/dynamics/base.py:1875-1883: pre_update -> neighbor hook -> model -> post_update;
the first step integrates with the forces already in the batch, zeros here)."""

from __future__ import annotations

import numpy as np

import oracle

FS_PER_INTERNAL_TIME = 10.180505710759414


def build_and_eval(P, C, pb, ptr, bi, rc, eps, sig, K):
    while True:
        nm, nn, sh = oracle.nl_cell(P, C, pb, ptr, rc, K)
        if nn.max(initial=0) < K:
            break
        K = int(nn.max() * 1.5) + 1
    cells = C if C is not None else np.eye(3, dtype=np.float32)[None].repeat(len(ptr) - 1, 0)
    out = oracle.lj_matrix(P, cells, nm, sh if C is not None else None, nn, bi, len(P), eps, sig, rc)
    return out, K


def nve(P, V, M, C, pb, ptr, rc, eps, sig, dt_fs, n_steps, K=64, record=None):
    """Velocity-Verlet trajectory; returns positions, velocities, forces, per-system energies."""
    P, V = P.copy(), V.copy()
    bi = oracle.batch_idx_from_ptr(ptr)
    B = len(ptr) - 1
    dt = np.full(B, np.float32(dt_fs / FS_PER_INTERNAL_TIME), dtype=np.float32)
    F = np.zeros_like(P)
    E = np.zeros(B, dtype=np.float32)
    for step in range(n_steps):
        oracle.vv_pre(P, V, F, M, dt, bi)
        out, K = build_and_eval(P, C, pb, ptr, bi, rc, eps, sig, K)
        F, E = out["forces"], out["energy"]
        oracle.vv_post(V, F, M, dt, bi)
        if record is not None:
            record(step, P, V, F, E)
    return P, V, F, E


def fire(P, V, M, C, pb, ptr, rc, eps, sig, dt, n_steps, K=64, active_fn=None, fmax_tol=None):
    """FIRE relaxation with the reference's defaults; optional per-system freezing once
    fmax <= fmax_tol (status migration of the convergence hook)."""
    P, V = P.copy(), V.copy()
    bi = oracle.batch_idx_from_ptr(ptr)
    B = len(ptr) - 1
    f32 = lambda x: np.full(B, x, dtype=np.float32)  # noqa: E731
    dt0 = f32(dt)
    st = dict(alpha=f32(0.1), dt=dt0.copy(), alpha_start=f32(0.1), f_alpha=f32(0.99),
              dt_min=(dt0 * np.float32(0.02)).astype(np.float32), dt_max=(dt0 * np.float32(10.0)).astype(np.float32),
              maxstep=f32(0.2), f_dec=f32(0.5), f_inc=f32(1.1), vf=f32(0), vv=f32(0), ff=f32(0),
              n_steps_positive=np.zeros(B, dtype=np.int32), n_min=np.full(B, 5, dtype=np.int32))
    F = np.zeros_like(P)
    E = np.zeros(B, dtype=np.float32)
    status = np.zeros(B, dtype=np.int64)
    for step in range(n_steps):
        active = (status < 1).astype(np.uint8) if fmax_tol is not None else None
        oracle.fire_step(P, V, F, M, st, bi, active=active)
        out, K = build_and_eval(P, C, pb, ptr, bi, rc, eps, sig, K)
        F, E = out["forces"], out["energy"]
        if fmax_tol is not None:
            conv = oracle.fmax(F, bi, B) <= fmax_tol
            status[conv & (status == 0)] = 1
    return P, V, F, E, st, status
