"""numpy/ctypes front end of the CPU oracle (``md_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports it.

Every function takes and returns numpy arrays with the reference's layouts
(positions ``(N,3) f32``, cell ``(B,3,3) f32`` rows = lattice vectors, pbc ``(B,3) bool``,
``batch_ptr (B+1) i32``, ``batch_idx (N) i32``; see nvalchemi/neighbors.py:239-266).
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libmd_oracle.so"
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u8p = ctypes.POINTER(ctypes.c_uint8)


def build(force: bool = False) -> Path:
    """Compile ``md_oracle.c`` with gcc (``make -C oracle``)."""
    if force and _LIB_PATH.exists():
        _LIB_PATH.unlink()
    subprocess.run(["make", "-C", str(_HERE), "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        L = ctypes.CDLL(str(_LIB_PATH))
        L.orc_nl_brute.restype = ctypes.c_int64
        L.orc_nl_brute.argtypes = [_f32p, _f32p, _u8p, _i32p, ctypes.c_int32, ctypes.c_double,
                                   ctypes.c_int32, ctypes.c_int64, _i32p]
        L.orc_nl_cell.restype = ctypes.c_int32
        L.orc_nl_cell.argtypes = [_f32p, _f32p, _u8p, _i32p, ctypes.c_int32, ctypes.c_double,
                                  ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _i32p, _i32p, _i32p]
        L.orc_lj_matrix.restype = ctypes.c_int32
        L.orc_lj_matrix.argtypes = [_f32p, _f32p, _i32p, _i32p, _i32p, _i32p, ctypes.c_int32,
                                    ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                    ctypes.c_double, ctypes.c_double, ctypes.c_double,
                                    ctypes.c_int32, _f32p, _f32p, _f32p, _f32p]
        L.orc_lj_matrix_switched.restype = ctypes.c_int32
        L.orc_lj_matrix_switched.argtypes = [_f32p, _f32p, _i32p, _i32p, _i32p, _i32p, ctypes.c_int32,
                                             ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                             ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double,
                                             ctypes.c_int32, _f32p, _f32p, _f32p, _f32p]
        _u32p = ctypes.POINTER(ctypes.c_uint32)
        _f64p = ctypes.POINTER(ctypes.c_double)
        L.orc_philox4x32_10.restype = None
        L.orc_philox4x32_10.argtypes = [_u32p, _u32p, _u32p]
        L.orc_langevin_normals.restype = None
        L.orc_langevin_normals.argtypes = [ctypes.c_uint64, ctypes.c_int32, _f64p]
        L.orc_langevin_half_step.restype = None
        L.orc_langevin_half_step.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, ctypes.c_uint64,
                                             _i32p, _u8p, ctypes.c_int32]
        L.orc_fire2_step.restype = None
        L.orc_fire2_step.argtypes = [_f32p, _f32p, _f32p, _i32p, _f32p, _f32p, _i32p, _f32p, _f32p, _f32p, _f32p,
                                     ctypes.c_int32] + [ctypes.c_double] * 7 + [_u8p, ctypes.c_int32, ctypes.c_int32]
        L.orc_nhc_chain_update.restype = None
        L.orc_nhc_chain_update.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                           _i32p, _u8p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                           ctypes.c_int32, ctypes.c_int32]
        L.orc_nhc_position_update.restype = None
        L.orc_nhc_position_update.argtypes = [_f32p, _f32p, _f32p, _i32p, _u8p, ctypes.c_int32]
        L.orc_vv_pre.restype = None
        L.orc_vv_pre.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _i32p, _u8p, ctypes.c_int32]
        L.orc_vv_post.restype = None
        L.orc_vv_post.argtypes = [_f32p, _f32p, _f32p, _f32p, _i32p, _u8p, ctypes.c_int32]
        L.orc_fire_step.restype = None
        L.orc_fire_step.argtypes = [_f32p, _f32p, _f32p, _f32p] + [_f32p] * 7 + [_i32p, _i32p] + \
            [_f32p] * 5 + [_i32p, _u8p, ctypes.c_int32, ctypes.c_int32]
        L.orc_fmax.restype = None
        L.orc_fmax.argtypes = [_f32p, _i32p, ctypes.c_int32, ctypes.c_int32, _f32p]
        L.orc_rebuild_check.restype = None
        L.orc_rebuild_check.argtypes = [_f32p, _f32p, _i32p, _f32p, _u8p, ctypes.c_int32, ctypes.c_int32,
                                        ctypes.c_double, ctypes.c_int32, _u8p]
        L.orc_wrap_positions.restype = None
        L.orc_wrap_positions.argtypes = [_f32p, _f32p, _u8p, _i32p, ctypes.c_int32]
        L.orc_num_threads.restype = ctypes.c_int32
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


def set_threads(n: int) -> None:
    """Thread count of the OpenMP loops (read by libgomp at the next parallel region)."""
    os.environ["OMP_NUM_THREADS"] = str(n)
    try:
        ctypes.CDLL("libgomp.so.1").omp_set_num_threads(int(n))
    except OSError:
        pass


def num_threads() -> int:
    return int(lib().orc_num_threads())


def batch_idx_from_ptr(batch_ptr) -> np.ndarray:
    ptr = np.asarray(batch_ptr, dtype=np.int64)
    return np.repeat(np.arange(len(ptr) - 1, dtype=np.int32), np.diff(ptr)).astype(np.int32)


def canonical_edges(edges: np.ndarray) -> np.ndarray:
    """Sort ``(E,5)`` records ``(i, j, sx, sy, sz)`` lexicographically."""
    e = np.asarray(edges, dtype=np.int64).reshape(-1, 5)
    if len(e) == 0:
        return e
    order = np.lexsort((e[:, 4], e[:, 3], e[:, 2], e[:, 1], e[:, 0]))
    return e[order]


def matrix_to_edges(nm, nn, shifts=None) -> np.ndarray:
    """Dense ``(N,K)`` matrix + counts (+ ``(N,K,3)`` shifts) -> canonical ``(E,5)`` records.

    Rows are read in ``[0, min(count, K))`` as the reference does
    (nvalchemi/models/_ops/neighbor_filter.py:255-283).
    """
    nm = np.asarray(nm)
    nn = np.asarray(nn)
    N, K = nm.shape
    cols = np.arange(K)[None, :]
    valid = cols < np.minimum(nn, K)[:, None]
    ii, kk = np.nonzero(valid)
    out = np.zeros((len(ii), 5), dtype=np.int64)
    out[:, 0] = ii
    out[:, 1] = nm[ii, kk]
    if shifts is not None:
        out[:, 2:] = np.asarray(shifts)[ii, kk]
    return canonical_edges(out)


def nl_brute(positions, cell, pbc, batch_ptr, cutoff: float, half: bool = False) -> np.ndarray:
    """All ``(i, j, S)`` with ``|r_j - r_i + S.cell| < cutoff`` by brute force; canonical order."""
    pos = _f32(positions)
    ptr = _i32(batch_ptr)
    B = len(ptr) - 1
    c = None if cell is None else _f32(cell).reshape(B, 9)
    p = None if (pbc is None or cell is None) else _u8(pbc).reshape(B, 3)
    L = lib()
    args = (_p(pos, _f32p), _p(c, _f32p), _p(p, _u8p), _p(ptr, _i32p), B, float(cutoff), int(half))
    total = L.orc_nl_brute(*args, 0, None)
    out = np.zeros((max(total, 1), 5), dtype=np.int32)
    total2 = L.orc_nl_brute(*args, total, _p(out, _i32p))
    assert total2 == total
    return canonical_edges(out[:total])


def nl_cell(positions, cell, pbc, batch_ptr, cutoff: float, max_neighbors: int, half: bool = False):
    """Cell-list build into ``(neighbor_matrix, num_neighbors, shifts)`` (reference layout)."""
    pos = _f32(positions)
    ptr = _i32(batch_ptr)
    B = len(ptr) - 1
    N = pos.shape[0]
    K = int(max_neighbors)
    c = None if cell is None else _f32(cell).reshape(B, 9)
    p = None if (pbc is None or cell is None) else _u8(pbc).reshape(B, 3)
    nm = np.empty((N, K), dtype=np.int32)
    nn = np.empty(N, dtype=np.int32)
    sh = np.empty((N, K, 3), dtype=np.int32)
    lib().orc_nl_cell(_p(pos, _f32p), _p(c, _f32p), _p(p, _u8p), _p(ptr, _i32p), B, float(cutoff),
                      int(half), K, N, _p(nm, _i32p), _p(nn, _i32p), _p(sh, _i32p))
    return nm, nn, sh


def lj_matrix(positions, cells, neighbor_matrix, shifts, num_neighbors, batch_idx, fill_value,
              epsilon, sigma, cutoff, half=False, virial=False, switch_width=0.0):
    """LJ over the dense matrix -> dict(atomic_energies, forces, energy[, virials])."""
    pos = _f32(positions)
    N = pos.shape[0]
    nm = _i32(neighbor_matrix)
    K = nm.shape[1] if nm.ndim == 2 else 0
    cells = _f32(cells).reshape(-1, 9)
    B = cells.shape[0]
    sh = None if shifts is None else _i32(shifts)
    nn = _i32(num_neighbors)
    bi = _i32(batch_idx)
    e = np.zeros(N, dtype=np.float32)
    f = np.zeros((N, 3), dtype=np.float32)
    w = np.zeros((B, 9), dtype=np.float32) if virial else None
    es = np.zeros(B, dtype=np.float32)
    lib().orc_lj_matrix_switched(_p(pos, _f32p), _p(cells, _f32p), _p(nm, _i32p), _p(sh, _i32p), _p(nn, _i32p),
                                 _p(bi, _i32p), N, K, B, int(fill_value), float(epsilon), float(sigma),
                                 float(cutoff), float(switch_width), int(half), _p(e, _f32p), _p(f, _f32p),
                                 _p(w, _f32p), _p(es, _f32p))
    out = {"atomic_energies": e, "forces": f, "energy": es}
    if virial:
        out["virials"] = w
    return out


def vv_pre(positions, velocities, forces, masses, dt, batch_idx, active=None):
    """In-place first half of velocity Verlet on float32 arrays."""
    for a in (positions, velocities):
        assert a.dtype == np.float32 and a.flags.c_contiguous
    act = None if active is None else _u8(active)
    lib().orc_vv_pre(_p(positions, _f32p), _p(velocities, _f32p), _p(_f32(forces), _f32p),
                     _p(_f32(masses), _f32p), _p(_f32(dt), _f32p), _p(_i32(batch_idx), _i32p),
                     _p(act, _u8p), positions.shape[0])


def vv_post(velocities, forces, masses, dt, batch_idx, active=None):
    """In-place second half of velocity Verlet on float32 arrays."""
    assert velocities.dtype == np.float32 and velocities.flags.c_contiguous
    act = None if active is None else _u8(active)
    lib().orc_vv_post(_p(velocities, _f32p), _p(_f32(forces), _f32p), _p(_f32(masses), _f32p),
                      _p(_f32(dt), _f32p), _p(_i32(batch_idx), _i32p), _p(act, _u8p),
                      velocities.shape[0])


def fire_step(positions, velocities, forces, masses, state: dict, batch_idx, active=None):
    """In-place FIRE step.  ``state`` holds float32 ``alpha, dt, alpha_start, f_alpha, dt_min,
    dt_max, maxstep, f_dec, f_inc, vf, vv, ff`` and int32 ``n_steps_positive, n_min`` arrays
    of length M; ``alpha, dt, n_steps_positive, vf, vv, ff`` are updated."""
    for a in (positions, velocities):
        assert a.dtype == np.float32 and a.flags.c_contiguous
    for k in ("alpha", "dt", "vf", "vv", "ff"):
        assert state[k].dtype == np.float32
    assert state["n_steps_positive"].dtype == np.int32
    M = state["alpha"].shape[0]
    act = None if active is None else _u8(active)
    g = lambda k: _p(_f32(state[k]), _f32p)  # noqa: E731
    lib().orc_fire_step(_p(positions, _f32p), _p(velocities, _f32p), _p(_f32(forces), _f32p),
                        _p(_f32(masses), _f32p), _p(state["alpha"], _f32p), _p(state["dt"], _f32p),
                        g("alpha_start"), g("f_alpha"), g("dt_min"), g("dt_max"), g("maxstep"),
                        _p(state["n_steps_positive"], _i32p), _p(_i32(state["n_min"]), _i32p),
                        g("f_dec"), g("f_inc"), _p(state["vf"], _f32p), _p(state["vv"], _f32p),
                        _p(state["ff"], _f32p), _p(_i32(batch_idx), _i32p), _p(act, _u8p),
                        positions.shape[0], M)


def fmax(forces, batch_idx, n_systems: int) -> np.ndarray:
    f = _f32(forces)
    out = np.empty(n_systems, dtype=np.float32)
    lib().orc_fmax(_p(f, _f32p), _p(_i32(batch_idx), _i32p), f.shape[0], int(n_systems),
                   _p(out, _f32p))
    return out


def rebuild_check(reference_positions, current_positions, batch_idx, n_systems: int, threshold: float,
                  update_reference: bool = False, cell=None, pbc=None):
    """Verlet-skin displacement test -> ``(flags (M) bool, reference positions after the call)``."""
    ref = _f32(reference_positions).copy()
    cur = _f32(current_positions)
    c = None if cell is None else _f32(cell).reshape(-1, 9)
    p = None if (pbc is None or cell is None) else _u8(pbc).reshape(-1, 3)
    flags = np.zeros(int(n_systems), dtype=np.uint8)
    lib().orc_rebuild_check(_p(ref, _f32p), _p(cur, _f32p), _p(_i32(batch_idx), _i32p), _p(c, _f32p),
                            _p(p, _u8p), ref.shape[0], int(n_systems), float(threshold),
                            int(update_reference), _p(flags, _u8p))
    return flags.astype(bool), ref


def wrap_positions(positions, cell, pbc, batch_idx) -> np.ndarray:
    """Positions wrapped into their cells (a copy), per-axis flags as the reference applies them."""
    pos = _f32(positions).copy()
    lib().orc_wrap_positions(_p(pos, _f32p), _p(_f32(cell).reshape(-1, 9), _f32p),
                             _p(_u8(pbc).reshape(-1, 3), _u8p), _p(_i32(batch_idx), _i32p), pos.shape[0])
    return pos


def segment_reduce(values, batch_idx, n_segments: int, op: str) -> np.ndarray:
    """Per-segment ``sum`` / ``amax`` / ``amin`` / ``mean`` of a float32 vector (numpy restatement of
    nvalchemi/dynamics/hooks/_utils.py:58-136: sums in float64, rounded once; empty segments give
    0, -inf, +inf, 0)."""
    v = _f32(values)
    idx = _i32(batch_idx)
    m = int(n_segments)
    if op == "amax":
        out = np.full(m, -np.inf, dtype=np.float32)
        np.maximum.at(out, idx, v)
        return out
    if op == "amin":
        out = np.full(m, np.inf, dtype=np.float32)
        np.minimum.at(out, idx, v)
        return out
    acc = np.zeros(m, dtype=np.float64)
    np.add.at(acc, idx, v.astype(np.float64))
    if op == "sum":
        return acc.astype(np.float32)
    cnt = np.bincount(idx, minlength=m).astype(np.float64)
    return np.where(cnt > 0, acc / np.maximum(cnt, 1), 0.0).astype(np.float32)


def kinetic_energy(velocities, masses, batch_idx, n_systems: int) -> np.ndarray:
    """``0.5 sum m |v|^2`` per system (nvalchemi/dynamics/hooks/_utils.py:215-243), float64 sum, rounded once."""
    v = _f32(velocities).astype(np.float64)
    per_atom = 0.5 * _f32(masses).astype(np.float64) * ((v[:, 0] * v[:, 0] + v[:, 1] * v[:, 1]) + v[:, 2] * v[:, 2])
    acc = np.zeros(int(n_systems), dtype=np.float64)
    np.add.at(acc, _i32(batch_idx), per_atom)
    return acc.astype(np.float32)


# ---------------------------------------------------------------------------------------------
# masked copy / compaction of rows and segments (numpy, in place like the reference's functions)
# nvalchemi/data/buffer_kernels.py; pinned by the reference's own cases
# (test/data/test_buffer_kernels.py:49-535), restated in tests/test_oracle_buffers.py
# ---------------------------------------------------------------------------------------------
def _rows2d(a):
    return a.reshape(a.shape[0], int(np.prod(a.shape[1:])))


def _put_plan_per_system(source_mask, dest_mask):
    """exclusive scan of the mask, number of rows that may move, first empty slot
    (buffer_kernels.py:58-140)"""
    m = np.asarray(source_mask, dtype=bool)
    scan = np.cumsum(m) - m
    count_empty = int((~np.asarray(dest_mask, dtype=bool)).sum())
    max_copy = min(int(m.sum()), count_empty)
    empty = np.flatnonzero(~np.asarray(dest_mask, dtype=bool))
    first_empty = int(empty[0]) if len(empty) else len(dest_mask)
    return m, scan, max_copy, first_empty


def put_masked_per_system(source, source_mask, dest, dest_mask, source_data_copied):
    """buffer_kernels.py:143-186, 970-1079"""
    if source.shape[0] == 0:
        return
    src, dst = _rows2d(source), _rows2d(dest)
    m, scan, max_copy, first_empty = _put_plan_per_system(source_mask, dest_mask)
    for i in range(len(m)):
        if not m[i] or scan[i] >= max_copy:
            continue
        k = first_empty + scan[i]
        dst[k] = src[i]
        dest_mask[k] = True
        source_data_copied[i] = True


def put_fit_mask_per_system(source_mask, dest_mask, fit_mask):
    """buffer_kernels.py:612-622, 1081-1169"""
    if len(source_mask) == 0:
        return
    m, scan, max_copy, _ = _put_plan_per_system(source_mask, dest_mask)
    fit_mask[:] = m & (scan < max_copy)


def defrag_per_system(source, source_data_copied):
    """buffer_kernels.py:189-253, 1222-1333"""
    if source.shape[0] == 0:
        return
    src = _rows2d(source)
    keep = ~np.asarray(source_data_copied, dtype=bool)
    kept = src[keep].copy()
    src[:] = 0
    src[: len(kept)] = kept
    source_data_copied[:] = np.arange(len(keep)) >= len(kept)


def _put_plan_segmented(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments, dest_capacity):
    """buffer_kernels.py:372-399, 454-497"""
    ptr = np.asarray(source_batch_ptr, dtype=np.int64)
    m = np.asarray(source_mask, dtype=bool)
    lengths = np.where(m, ptr[1:] - ptr[:-1], 0)
    offset = np.cumsum(lengths) - lengths
    base = int(dest_batch_ptr[num_dest_segments])
    fits = m & (base + offset + lengths <= dest_capacity)
    return ptr, lengths, offset, base, fits


def put_fit_mask_segmented(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments, dest_capacity,
                           fit_mask):
    """buffer_kernels.py:500-610"""
    n = len(source_batch_ptr) - 1
    if n == 0:
        return
    if len(dest_batch_ptr) < num_dest_segments + n + 2:
        fit_mask[:] = False
        return
    fit_mask[:] = _put_plan_segmented(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments,
                                      dest_capacity)[4]


def put_masked_segmented(source, source_batch_ptr, source_mask, dest, dest_batch_ptr, num_dest_segments,
                         source_data_copied):
    """buffer_kernels.py:624-659, 1335-1527; returns the new number of destination segments"""
    n = len(source_batch_ptr) - 1
    if n == 0:
        return None
    need = num_dest_segments + n + 2
    if len(dest_batch_ptr) < need:
        raise ValueError(f"dest_batch_ptr must have size >= num_dest_segments + num_systems + 2 ({need}); "
                         f"got {len(dest_batch_ptr)}")
    src, dst = _rows2d(source), _rows2d(dest)
    ptr, lengths, offset, base, fits = _put_plan_segmented(source_batch_ptr, source_mask, dest_batch_ptr,
                                                           num_dest_segments, dst.shape[0])
    fit_scan = np.cumsum(fits) - fits
    n_fit = int(fits.sum())
    for i in range(n):
        if not fits[i]:
            continue
        a = base + offset[i]
        dst[a: a + lengths[i]] = src[ptr[i]: ptr[i + 1]]
        source_data_copied[i] = True
        end = base + offset[i] + lengths[i]
        dest_batch_ptr[num_dest_segments + 1 + fit_scan[i]] = end
        if fit_scan[i] == n_fit - 1:
            dest_batch_ptr[num_dest_segments + 1 + n_fit] = end
    return num_dest_segments + n_fit


def defrag_segmented(source, source_batch_ptr, source_data_copied):
    """buffer_kernels.py:661-967, 1529-1741; returns the number of kept segments"""
    n = len(source_batch_ptr) - 1
    if n == 0:
        source_batch_ptr[0] = 0
        return 0
    src = _rows2d(source)
    ptr = np.asarray(source_batch_ptr, dtype=np.int64).copy()
    keep = ~np.asarray(source_data_copied, dtype=bool)
    pieces = [src[ptr[i]: ptr[i + 1]].copy() for i in range(n) if keep[i]]
    lengths = [len(p) for p in pieces]
    total = int(sum(lengths))
    src[:] = 0
    if total:
        src[:total] = np.concatenate(pieces)
    num_kept = len(pieces)
    source_batch_ptr[: num_kept + 1] = np.concatenate([[0], np.cumsum(lengths)]) if num_kept else [0]
    source_batch_ptr[num_kept + 1:] = total
    return num_kept


# ---------------------------------------------------------------------------------------------
# filtering a list to a tighter cutoff (numpy restatement of the in-tree Torch code,
# nvalchemi/models/_ops/neighbor_filter.py:43-283, with the distance in double on the float32
# inputs as everywhere in this library; pinned by the reference's own cases,
# test/models/test_neighbor_filter.py:49-760, restated in tests/test_oracle_filter.py)
# ---------------------------------------------------------------------------------------------
def _filter_d2(pos_i, pos_j, shifts, cells):
    d = pos_j.astype(np.float64) - pos_i.astype(np.float64)
    if shifts is not None and cells is not None:
        s = shifts.astype(np.float64)
        h = cells.astype(np.float64)
        # (S0 a0 + S1 a1) + S2 a2 per component, as orc_pair_d2 does
        t = (s[..., 0:1] * h[..., 0, :] + s[..., 1:2] * h[..., 1, :]) + s[..., 2:3] * h[..., 2, :]
        d = d + t
    return (d[..., 0] * d[..., 0] + d[..., 1] * d[..., 1]) + d[..., 2] * d[..., 2]


def filter_neighbor_matrix(positions, cutoff, neighbor_matrix, num_neighbors, fill_value, cell=None,
                           neighbor_matrix_shifts=None, batch_idx=None):
    """neighbor_filter.py:43-144 -> (matrix, counts, shifts | None)"""
    pos = _f32(positions)
    nm = _i32(neighbor_matrix)
    N, K = nm.shape
    valid = nm < fill_value
    j = np.clip(nm, 0, max(N - 1, 0))
    cells = None
    if cell is not None and neighbor_matrix_shifts is not None:
        c = _f32(cell)
        if c.ndim == 2:
            cells = np.broadcast_to(c, (N, 1, 3, 3))
        else:
            if batch_idx is None:
                raise ValueError("batch_idx is required when cell has shape (B, 3, 3).")
            cells = c[_i32(batch_idx)][:, None]
    d2 = _filter_d2(pos[:, None, :], pos[j], None if cells is None else _i32(neighbor_matrix_shifts), cells)
    keep = valid & (d2 < float(cutoff) * float(cutoff))
    order = np.argsort(~keep, axis=1, kind="stable")
    keep_sorted = np.take_along_axis(keep, order, 1)
    out_nm = np.where(keep_sorted, np.take_along_axis(nm, order, 1), fill_value).astype(np.int32)
    out_nn = keep.sum(1).astype(np.asarray(num_neighbors).dtype)
    out_sh = None
    if neighbor_matrix_shifts is not None:
        sh = np.take_along_axis(_i32(neighbor_matrix_shifts), order[..., None], 1)
        out_sh = np.where(keep_sorted[..., None], sh, 0).astype(np.int32)
    return out_nm, out_nn, out_sh


def filter_neighbor_list(positions, cutoff, neighbor_list, neighbor_ptr, cell=None, neighbor_list_shifts=None,
                         batch_idx=None):
    """neighbor_filter.py:147-224 -> (edges, ptr, shifts | None)"""
    pos = _f32(positions)
    nl = _i32(neighbor_list)
    N = pos.shape[0]
    i, j = nl[:, 0], nl[:, 1]
    cells = None
    if cell is not None and neighbor_list_shifts is not None:
        c = _f32(cell)
        if c.ndim == 2:
            cells = np.broadcast_to(c, (len(i), 3, 3))
        else:
            if batch_idx is None:
                raise ValueError("batch_idx is required when cell has shape (B, 3, 3).")
            cells = c[_i32(batch_idx)[i]]
    d2 = _filter_d2(pos[i], pos[j], None if cells is None else _i32(neighbor_list_shifts), cells)
    keep = d2 < float(cutoff) * float(cutoff)
    ptr = np.zeros(N + 1, dtype=np.asarray(neighbor_ptr).dtype)
    ptr[1:] = np.cumsum(np.bincount(i[keep], minlength=N))
    return nl[keep], ptr, None if neighbor_list_shifts is None else _i32(neighbor_list_shifts)[keep]


def neighbor_matrix_to_list(neighbor_matrix, num_neighbors, fill_value, neighbor_matrix_shifts=None):
    """neighbor_filter.py:227-283 -> (edges (M,2), ptr (N+1), shifts | None)"""
    nm = _i32(neighbor_matrix)
    N, K = nm.shape
    ii, kk = np.nonzero(nm < fill_value)
    nl = np.stack([ii.astype(np.int32), nm[ii, kk]], axis=1)
    ptr = np.zeros(N + 1, dtype=np.int32)
    ptr[1:] = np.cumsum(_i32(num_neighbors))
    return nl, ptr, None if neighbor_matrix_shifts is None else _i32(neighbor_matrix_shifts)[ii, kk]


# ---------------------------------------------------------------------------------------------
# Langevin (BAOAB half step) and its generator
# ---------------------------------------------------------------------------------------------
def philox4x32_10(counter, key):
    c = np.asarray(counter, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    out = np.zeros(4, dtype=np.uint32)
    u32p = ctypes.POINTER(ctypes.c_uint32)
    lib().orc_philox4x32_10(c.ctypes.data_as(u32p), k.ctypes.data_as(u32p), out.ctypes.data_as(u32p))
    return out


def langevin_normals(seed, atom):
    xi = np.zeros(4, dtype=np.float64)
    lib().orc_langevin_normals(int(seed), int(atom), xi.ctypes.data_as(ctypes.POINTER(ctypes.c_double)))
    return xi


def langevin_half_step(positions, velocities, forces, masses, dt, kT, friction, seed, batch_idx, active=None):
    """In place on float32 ``positions`` / ``velocities``."""
    assert positions.dtype == np.float32 and velocities.dtype == np.float32
    act = None if active is None else np.ascontiguousarray(active, dtype=np.uint8)
    lib().orc_langevin_half_step(_p(positions, _f32p), _p(velocities, _f32p), _p(_f32(forces), _f32p),
                                 _p(_f32(masses), _f32p), _p(_f32(dt), _f32p), _p(_f32(kT), _f32p),
                                 _p(_f32(friction), _f32p), int(seed), _p(_i32(batch_idx), _i32p),
                                 None if act is None else _p(act, _u8p), positions.shape[0])


# ---------------------------------------------------------------------------------------------
# Nose-Hoover chain (md_oracle.c: orc_nhc_chain_update)
# ---------------------------------------------------------------------------------------------
def nhc_masses(kT, tau, ndof, chain_length):
    """Q (M, C): Q_1 = N_f kT tau^2, Q_k = kT tau^2 (nvalchemi/dynamics/_ops/nose_hoover.py:67-70)."""
    kT, tau, ndof = (np.asarray(a, dtype=np.float64) for a in (kT, tau, ndof))
    q = np.repeat((kT * tau * tau)[:, None], chain_length, axis=1)
    q[:, 0] *= ndof
    return q.astype(np.float32)


def nhc_chain_update(velocities, masses, eta, eta_dot, Q, kT, dt, ndof, batch_idx, ke2=None, active=None,
                     yoshida_order=3):
    """In place on float32 ``velocities (N,3)``, ``eta`` and ``eta_dot (M,C)``.  With ``ke2`` given it is
    used as sum m v^2 per system instead of the velocities.  Returns ``(ke2, total_scale)``."""
    assert velocities.dtype == np.float32 and eta.dtype == np.float32 and eta_dot.dtype == np.float32
    assert eta.flags.c_contiguous and eta_dot.flags.c_contiguous and velocities.flags.c_contiguous
    M, C = eta.shape
    assert C <= 16
    compute = ke2 is None
    k2 = np.zeros(M, dtype=np.float32) if compute else np.ascontiguousarray(ke2, dtype=np.float32).copy()
    scale = np.ones(M, dtype=np.float32)
    act = None if active is None else np.ascontiguousarray(active, dtype=np.uint8)
    lib().orc_nhc_chain_update(_p(velocities, _f32p), _p(_f32(masses), _f32p), _p(eta, _f32p), _p(eta_dot, _f32p),
                               _p(_f32(Q), _f32p), _p(_f32(kT), _f32p), _p(_f32(dt), _f32p), _p(_f32(ndof), _f32p),
                               _p(k2, _f32p), _p(scale, _f32p), _p(_i32(batch_idx), _i32p),
                               None if act is None else _p(act, _u8p), int(compute), C, int(yoshida_order),
                               velocities.shape[0], M)
    return k2, scale


def nhc_position_update(positions, velocities, dt, batch_idx, active=None):
    assert positions.dtype == np.float32
    act = None if active is None else np.ascontiguousarray(active, dtype=np.uint8)
    lib().orc_nhc_position_update(_p(positions, _f32p), _p(_f32(velocities), _f32p), _p(_f32(dt), _f32p),
                                  _p(_i32(batch_idx), _i32p), None if act is None else _p(act, _u8p),
                                  positions.shape[0])


# ---------------------------------------------------------------------------------------------
# FIRE 2.0 (md_oracle.c: orc_fire2_step)
# ---------------------------------------------------------------------------------------------
FIRE2_DEFAULTS = dict(delaystep=60, dtgrow=1.05, dtshrink=0.75, alphashrink=0.985, alpha0=0.09, tmax=0.08,
                      tmin=0.005, maxstep=0.1)  # nvalchemi/dynamics/optimizers/fire2.py:54-63


def fire2_step(positions, velocities, forces, batch_idx, alpha, dt, nsteps_inc, active=None, **params):
    """In place on float32 ``positions``, ``velocities`` (N,3), ``alpha``, ``dt`` (M) and int32
    ``nsteps_inc`` (M).  Returns ``dict(vf, v_sumsq, f_sumsq, max_norm)`` (M each)."""
    for a in (positions, velocities, alpha, dt):
        assert a.dtype == np.float32 and a.flags.c_contiguous
    assert nsteps_inc.dtype == np.int32
    p = dict(FIRE2_DEFAULTS)
    p.update(params)
    M = alpha.shape[0]
    out = {k: np.zeros(M, dtype=np.float32) for k in ("vf", "v_sumsq", "f_sumsq", "max_norm")}
    act = None if active is None else np.ascontiguousarray(active, dtype=np.uint8)
    lib().orc_fire2_step(_p(positions, _f32p), _p(velocities, _f32p), _p(_f32(forces), _f32p),
                         _p(_i32(batch_idx), _i32p), _p(alpha, _f32p), _p(dt, _f32p), _p(nsteps_inc, _i32p),
                         _p(out["vf"], _f32p), _p(out["v_sumsq"], _f32p), _p(out["f_sumsq"], _f32p),
                         _p(out["max_norm"], _f32p), int(p["delaystep"]), float(p["dtgrow"]), float(p["dtshrink"]),
                         float(p["alphashrink"]), float(p["alpha0"]), float(p["tmax"]), float(p["tmin"]),
                         float(p["maxstep"]), None if act is None else _p(act, _u8p), positions.shape[0], M)
    return out
