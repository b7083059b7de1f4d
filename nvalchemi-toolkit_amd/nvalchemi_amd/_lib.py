"""ctypes binding of ``libnvalchemi_amd.so`` (declared in ``include/nvalchemi_amd.h``).

This module is the only place that touches the C ABI.  It hands raw device pointers,
sizes and the current HIP stream to the library; tensors are checked here (device, dtype,
contiguity, shape) because the kernels trust their arguments.  There is no CPU
implementation behind these functions: a tensor that is not on a ROCm device, or a missing
library, raises.
"""

from __future__ import annotations

import ctypes
import math
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
LIB_PATH = _HERE / "lib" / "libnvalchemi_amd.so"

OK = 0
_c = ctypes
_vp = _c.c_void_p
_i32 = _c.c_int32
_f64 = _c.c_double

_SIGNATURES = {
    "nvamd_abi_version": (_i32, []),
    "nvamd_last_error": (_c.c_char_p, []),
    "nvamd_nl_workspace_bytes": (_i32, [_i32, _i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_nl_status": (_i32, [_vp, _c.c_size_t, _i32, _i32, _vp, _i32, _vp]),
    "nvamd_nl_build_f64": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _f64, _i32, _i32, _i32, _i32,
                                  _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_f64_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_lj_energy_forces_f64": (_i32, [_vp] * 6 + [_i32, _i32, _i32, _i32, _f64, _f64, _f64, _f64, _i32,
                                          _vp, _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_vv_position_update_f64": (_i32, [_vp] * 7 + [_i32, _i32, _vp]),
    "nvamd_vv_velocity_finalize_f64": (_i32, [_vp] * 6 + [_i32, _i32, _vp]),
    "nvamd_fire_step_f64": (_i32, [_vp] * 20 + [_i32, _vp, _i32, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_segment_fmax_f64": (_i32, [_vp, _vp, _i32, _i32, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_nl_build": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _f64, _i32, _i32, _i32,
                              _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_nl_build_path": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _f64, _i32, _i32, _i32, _i32,
                                   _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_coo_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_nl_coo_from_matrix": (_i32, [_vp, _vp, _vp, _i32, _i32, _c.c_int64, _vp, _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_nl_edge_ptr": (_i32, [_vp, _i32, _i32, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_nl_matrix_to_coo": (_i32, [_vp, _vp, _vp, _i32, _i32, _c.c_int64, _vp, _vp, _vp]),
    "nvamd_lj_workspace_bytes": (_i32, [_i32, _i32, _i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_lj_energy_forces": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _f64, _f64,
                                      _f64, _f64, _i32, _vp, _vp, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_vv_position_update": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_vv_finalize_then_update": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_vv_velocity_finalize": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_fire_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_fire_step": (_i32, [_vp] * 20 + [_i32, _vp, _i32, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_segment_fmax": (_i32, [_vp, _vp, _i32, _i32, _vp, _vp]),
    "nvamd_status_migrate": (_i32, [_vp, _f64, _vp, _c.c_int64, _c.c_int64, _i32, _vp]),
    "nvamd_status_migrate_f64": (_i32, [_vp, _f64, _vp, _c.c_int64, _c.c_int64, _i32, _vp]),
    "nvamd_lj_energy_forces_hinted": (_i32, [_vp] * 7 + [_c.c_double] + [_i32] * 4 + [_c.c_double] * 4 + [_i32] + [_vp] * 5 + [_c.c_size_t, _vp]),
    "nvamd_lj_energy_forces_repeat": (_i32, [_vp] * 7 + [_c.c_double] + [_i32] * 4 + [_c.c_double] * 4 + [_i32] + [_vp] * 5 + [_c.c_size_t, _vp]),
    "nvamd_lj_energy_forces_tiles": (_i32, [_vp] * 11 + [_c.c_double] + [_i32] * 4 + [_c.c_double] * 3 + [_i32] + [_vp] * 5 + [_c.c_size_t, _vp]),
    "nvamd_nl_build_extras": (_i32, [_vp] * 6 + [_i32, _i32, _c.c_double, _i32, _i32, _i32, _i32] + [_vp] * 9 + [_c.c_size_t, _vp]),
    "nvamd_nl_tile_records": (_i32, [_i32, _i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_lj_energy_forces_static": (_i32, [_vp] * 7 + [_c.c_double] + [_i32] * 4 + [_c.c_double] * 4 + [_vp] * 5),
    "nvamd_nl_atom_order": (_i32, [_vp, _c.c_size_t, _vp, _vp, _i32, _i32, _vp, _vp]),
    "nvamd_segment_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_segment_reduce": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_kinetic_energy": (_i32, [_vp, _vp, _vp, _i32, _i32, _vp, _vp, _c.c_size_t, _vp]),
    "nvamd_nl_rebuild_check": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _c.c_double, _i32, _vp, _vp]),
    "nvamd_wrap_positions": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_nl_rebuild_check_f64": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _c.c_double, _i32, _vp, _vp]),
    "nvamd_wrap_positions_f64": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_langevin_half_step": (_i32, [_vp] * 7 + [_c.c_uint64, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_langevin_half_step_f64": (_i32, [_vp] * 7 + [_c.c_uint64, _vp, _vp, _i32, _i32, _vp]),
    "nvamd_fire2_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_fire2_step": (_i32, [_vp] * 11 + [_i32] + [_c.c_double] * 7 + [_vp, _i32, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_fire2_step_f64": (_i32, [_vp] * 11 + [_i32] + [_c.c_double] * 7 + [_vp, _i32, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_nhc_workspace_bytes": (_i32, [_i32, _c.POINTER(_c.c_size_t)]),
    "nvamd_nhc_chain_update": (_i32, [_vp] * 12 + [_i32] * 5 + [_vp, _c.c_size_t, _vp]),
    "nvamd_nhc_position_update": (_i32, [_vp] * 5 + [_i32, _i32, _vp]),
    "nvamd_nhc_chain_update_f64": (_i32, [_vp] * 12 + [_i32] * 5 + [_vp, _c.c_size_t, _vp]),
    "nvamd_nhc_position_update_f64": (_i32, [_vp] * 5 + [_i32, _i32, _vp]),
    "nvamd_nl_filter_matrix": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _f64, _vp, _vp, _vp, _vp]),
    "nvamd_nl_filter_coo_flags": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _c.c_int64, _f64, _vp, _vp]),
    "nvamd_buffer_workspace_bytes": (_i32, [_c.c_int64, _c.c_int64, _c.POINTER(_c.c_size_t)]),
    "nvamd_put_masked_per_system": (_i32, [_vp] * 5 + [_i32, _i32, _c.c_int64, _vp, _c.c_size_t, _vp]),
    "nvamd_put_fit_mask_per_system": (_i32, [_vp] * 3 + [_i32, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_defrag_per_system": (_i32, [_vp, _vp, _i32, _c.c_int64, _vp, _c.c_size_t, _vp]),
    "nvamd_put_masked_segmented": (_i32, [_vp] * 5 + [_i32, _i32, _vp, _vp, _i32, _i32, _c.c_int64, _vp,
                                          _c.c_size_t, _vp]),
    "nvamd_put_fit_mask_segmented": (_i32, [_vp] * 3 + [_i32, _i32, _vp, _i32, _vp, _c.c_size_t, _vp]),
    "nvamd_defrag_segmented": (_i32, [_vp] * 4 + [_i32, _i32, _c.c_int64, _vp, _c.c_size_t, _vp]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


class KernelLibraryError(RuntimeError):
    """The HIP library is missing, or one of its entry points reported an error."""


def library() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise KernelLibraryError(
                f"{LIB_PATH} not found: build it with `python nvalchemi-toolkit_amd/build.py` "
                "(there is no fallback implementation)"
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != OK:
        msg = library().nvamd_last_error().decode(errors="replace")
        raise KernelLibraryError(f"{what} failed with code {rc}: {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device) -> int:
    """The current stream of ``device`` as a raw handle (without building a ``torch.cuda.Stream`` object
    where Torch offers the direct call: six of these per MD step)."""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


def _dev(t: torch.Tensor, name: str, dtype: torch.dtype, shape: tuple | None = None) -> int:
    """Validate a tensor the kernels will index blindly and return its device pointer."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor, got {type(t).__name__}")
    if t.device.type != "cuda":
        raise KernelLibraryError(
            f"{name}: tensor is on {t.device}; the nvalchemi_amd kernels run on a ROCm device only"
        )
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: tensor must be contiguous")
    if shape is not None:
        got = t.shape
        ok = len(got) == len(shape)
        if ok:
            for s, e in zip(got, shape):
                if e is not None and s != e:
                    ok = False
                    break
        if not ok:
            raise ValueError(f"{name}: expected shape {shape}, got {tuple(t.shape)}")
    return t.data_ptr()


def _real_dtype(t: torch.Tensor, name: str) -> torch.dtype:
    """float32 (the tuned kernels) or float64 (the plain ones); anything else is refused."""
    if t.dtype not in (torch.float32, torch.float64):
        raise TypeError(f"{name}: expected float32 or float64, got {t.dtype}")
    return t.dtype


def _opt(t, name, dtype, shape=None) -> int | None:
    return None if t is None else _dev(t, name, dtype, shape)


def _as_u8(t: torch.Tensor | None) -> torch.Tensor | None:
    """bool tensors are passed as bytes (same storage)."""
    if t is None:
        return None
    if t.dtype == torch.bool:
        return t.view(torch.uint8)
    return t


class _Workspaces:
    """One growing scratch buffer per (device, stream, purpose): kernels of one purpose on one
    stream run in order and can share it; another stream gets its own."""

    def __init__(self) -> None:
        self._bufs: dict[tuple, torch.Tensor] = {}

    def get(self, device: torch.device, purpose: str, nbytes: int) -> torch.Tensor:
        if torch.device(device).type != "cuda":
            raise KernelLibraryError(f"tensors are on {device}; the nvalchemi_amd kernels run on a ROCm device only")
        key = (device.index, _stream(device), purpose)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            old = buf
            # Some kernels keep state in their workspace from call to call (the neighbor build its unit counter and
            # status bits, FIRE the slot its sums are in): a buffer starts as zeros, and a regrown one takes over the
            # first 256 bytes of the buffer it replaces, where that state lives (so that, e.g., an overflow recorded
            # through the smaller buffer is still reported by nvamd_nl_status).
            buf = torch.zeros(max(int(nbytes), 256), dtype=torch.uint8, device=device)
            if old is not None:
                buf[:256].copy_(old[:256])
            self._bufs[key] = buf
        return buf

    def share(self, device: torch.device, from_stream: int, to_stream: int) -> None:
        """Let ``to_stream`` use the buffers of ``from_stream`` (raw stream handles).  For a capture stream whose
        graph will be replayed into ``from_stream``: the two never run side by side."""
        for (dev, stream, purpose), buf in list(self._bufs.items()):
            if dev == device.index and stream == from_stream:
                self._bufs[(dev, to_stream, purpose)] = buf
        # (what is known about the contents of a shared buffer goes with it)
        if (device.index, from_stream) in _lj_tables:
            _lj_tables[(device.index, to_stream)] = _lj_tables[(device.index, from_stream)]

    def unshare(self, device: torch.device, stream: int) -> None:
        """Forget every entry of ``stream`` (the buffers stay with whoever else holds them)."""
        for key in [k for k in self._bufs if k[0] == device.index and k[1] == stream]:
            del self._bufs[key]
        _lj_tables.pop((device.index, stream), None)


workspaces = _Workspaces()


def _size(fn, *args) -> int:
    out = ctypes.c_size_t(0)
    _check(fn(*args, ctypes.byref(out)), fn.__name__)
    return int(out.value)


# --------------------------------------------------------------------------------------------
# neighbor list
# --------------------------------------------------------------------------------------------
def nl_workspace_bytes(n_atoms: int, n_systems: int) -> int:
    return _size(library().nvamd_nl_workspace_bytes, int(n_atoms), int(n_systems))


NL_SORT_AUTO, NL_SORT_PER_SYSTEM, NL_SORT_GLOBAL = 0, 1, 2
# how nl_build brings the atoms into cell order when its caller does not say (sort_path=None): the
# library's own choice.  The GPU tests set this to run every case on both paths.
nl_sort_path = NL_SORT_AUTO


def nl_build(positions, cell, pbc, batch_ptr, batch_idx, rebuild_flags, cutoff, max_neighbors,
             half_fill, tail_mode, neighbor_matrix, num_neighbors, neighbor_matrix_shifts,
             workspace: torch.Tensor | None = None, sort_path: int | None = None, pair_tiles=None,
             shift_groups=None) -> None:
    """``pair_tiles``: ``(tile_index (N,K) i16, ordered_positions (N,4) f32, tile_records (R, NL_TILE_RECORD_INTS) i32,
    tile_count (1) i32)``, R = ``nl_tile_records(N, B)``: also leave behind what the pair kernel of large systems
    walks (float32 positions, full list, every system built, K a multiple of 8).  ``shift_groups`` (N) i32: per
    row, which groups of slots of ``neighbor_matrix_shifts`` may hold a shift that is not zero; with it the build
    does not write zeros over zeros (float32 positions, ``tail_mode`` 0, buffers that only this function writes and
    that were zeroed together with it)."""
    lib = library()
    if sort_path is None:
        sort_path = nl_sort_path
    N = positions.shape[0]
    B = batch_ptr.shape[0] - 1
    K = int(max_neighbors)
    # float32 or float64 positions, the cell in the same type (the reference's ops take both)
    real = _real_dtype(positions, "positions")
    p_pos = _dev(positions, "positions", real, (N, 3))
    p_cell = _opt(cell, "cell", real, (B, 3, 3))
    p_pbc = _opt(_as_u8(pbc), "pbc", torch.uint8, (B, 3))
    p_ptr = _dev(batch_ptr, "batch_ptr", torch.int32, (B + 1,))
    p_idx = _dev(batch_idx, "batch_idx", torch.int32, (N,))
    p_flags = _opt(_as_u8(rebuild_flags), "rebuild_flags", torch.uint8, (B,))
    p_nm = _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K))
    p_nn = _dev(num_neighbors, "num_neighbors", torch.int32, (N,))
    p_sh = _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3))
    need = nl_workspace_bytes(N, B)
    ws = workspace if workspace is not None else workspaces.get(positions.device, "nl", need)
    if ws.device != positions.device or ws.numel() * ws.element_size() < need:
        raise ValueError("neighbor-list workspace too small or on another device")
    if pair_tiles is not None or shift_groups is not None:
        if real != torch.float32:
            raise ValueError("pair tiles and shift groups need float32 positions")
        if pair_tiles is not None and (half_fill or rebuild_flags is not None):
            raise ValueError("pair tiles need a full list and a build of every system")
        if shift_groups is not None and tail_mode:
            raise ValueError("shift groups go with tail_mode 0")
        index, ordered, records, count = pair_tiles if pair_tiles is not None else (None,) * 4
        _check(lib.nvamd_nl_build_extras(
            p_pos, p_cell, p_pbc, p_ptr, p_idx, p_flags, N, B, float(cutoff), K, int(bool(half_fill)), int(tail_mode),
            int(sort_path), p_nm, p_nn, p_sh,
            _opt(index, "tile_index", torch.int16, (N, K)), _opt(ordered, "ordered_positions", torch.float32, (N, 4)),
            _opt(records, "tile_records", torch.int32, (nl_tile_records(N, B), NL_TILE_RECORD_INTS)),
            _opt(count, "tile_count", torch.int32, (1,)), _opt(shift_groups, "shift_groups", torch.int32, (N,)),
            ws.data_ptr(), ws.numel() * ws.element_size(), _stream(positions.device)), "nvamd_nl_build_extras")
        return
    entry = lib.nvamd_nl_build_f64 if real == torch.float64 else lib.nvamd_nl_build_path
    _check(entry(p_pos, p_cell, p_pbc, p_ptr, p_idx, p_flags, N, B, float(cutoff), K,
                 int(bool(half_fill)), int(tail_mode), int(sort_path), p_nm, p_nn, p_sh,
                 ws.data_ptr(), ws.numel() * ws.element_size(), _stream(positions.device)),
           "nvamd_nl_build")


NL_TILE_RECORD_INTS = 132


def nl_tile_records(n_atoms: int, n_systems: int) -> int:
    """Rows of the ``tile_records`` table that a build of this size may write."""
    return _size(library().nvamd_nl_tile_records, int(n_atoms), int(n_systems))


NL_STATUS_CELL_TOO_THIN = 1
NL_STATUS_ROW_OVERFLOW = 2


def nl_status(n_atoms: int, n_systems: int, device, clear: bool = False,
              workspace: torch.Tensor | None = None) -> torch.Tensor:
    """``(2,)`` int32 on the device: status bits of the last neighbor build through the workspace of
    this device and stream, and the bits of all builds since they were last cleared.  No host
    synchronisation here; reading the tensor on the host is one."""
    lib = library()
    need = nl_workspace_bytes(n_atoms, n_systems)
    ws = workspace if workspace is not None else workspaces.get(torch.device(device), "nl", need)
    out = torch.empty(2, dtype=torch.int32, device=device)
    _check(lib.nvamd_nl_status(ws.data_ptr(), ws.numel() * ws.element_size(), int(n_atoms), int(n_systems),
                               out.data_ptr(), int(bool(clear)), _stream(torch.device(device))), "nvamd_nl_status")
    return out


def nl_edge_ptr(num_neighbors, max_neighbors, edge_ptr) -> None:
    lib = library()
    N = num_neighbors.shape[0]
    need = _size(lib.nvamd_coo_workspace_bytes, N)
    ws = workspaces.get(num_neighbors.device, "coo", need)
    _check(lib.nvamd_nl_edge_ptr(_dev(num_neighbors, "num_neighbors", torch.int32, (N,)), N,
                                 int(max_neighbors), _dev(edge_ptr, "edge_ptr", torch.int32, (N + 1,)),
                                 ws.data_ptr(), ws.numel(), _stream(num_neighbors.device)),
           "nvamd_nl_edge_ptr")


def nl_coo_from_matrix(neighbor_matrix, neighbor_matrix_shifts, num_neighbors, edge_ptr, neighbor_list,
                       neighbor_list_shifts, counts) -> None:
    """Edge pointer and edges in one call; ``neighbor_list (E_cap, 2)`` sets the capacity, ``counts (2)``
    receives the edge count and an overflow flag on the device.  No host synchronisation."""
    lib = library()
    N, K = neighbor_matrix.shape
    cap = neighbor_list.shape[0]
    ws = workspaces.get(neighbor_matrix.device, "coo", _size(lib.nvamd_coo_workspace_bytes, N))
    _check(lib.nvamd_nl_coo_from_matrix(
        _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
        _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
        _dev(num_neighbors, "num_neighbors", torch.int32, (N,)), N, K, cap,
        _dev(edge_ptr, "edge_ptr", torch.int32, (N + 1,)),
        _dev(neighbor_list, "neighbor_list", torch.int32, (cap, 2)),
        _opt(neighbor_list_shifts, "neighbor_list_shifts", torch.int32, (cap, 3)),
        _dev(counts, "counts", torch.int32, (2,)), ws.data_ptr(), ws.numel(),
        _stream(neighbor_matrix.device)), "nvamd_nl_coo_from_matrix")


def nl_matrix_to_coo(neighbor_matrix, neighbor_matrix_shifts, edge_ptr, neighbor_list,
                     neighbor_list_shifts) -> None:
    lib = library()
    N, K = neighbor_matrix.shape
    E = neighbor_list.shape[0]
    _check(lib.nvamd_nl_matrix_to_coo(
        _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
        _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
        _dev(edge_ptr, "edge_ptr", torch.int32, (N + 1,)), N, K, E,
        _dev(neighbor_list, "neighbor_list", torch.int32, (E, 2)),
        _opt(neighbor_list_shifts, "neighbor_list_shifts", torch.int32, (E, 3)),
        _stream(neighbor_matrix.device)), "nvamd_nl_matrix_to_coo")


# --------------------------------------------------------------------------------------------
# Lennard-Jones
# --------------------------------------------------------------------------------------------
def lj_energy_forces(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors,
                     batch_idx, fill_value, epsilon, sigma, cutoff, switch_width, half_list,
                     atomic_energies, forces, virials=None, system_energies=None, row_order=None,
                     neighbor_list_cutoff: float = 0.0, pair_tiles=None) -> None:
    """``pair_tiles``: the four ``pair_tiles`` tensors of the ``nl_build`` that made this matrix from the positions in
    hand, with the ``row_order`` of that build (full list, no switching, shifts given; ignored otherwise)."""
    lib = library()
    N = positions.shape[0]
    K = neighbor_matrix.shape[1]
    B = cells.shape[0]
    if _real_dtype(positions, "positions") == torch.float64:
        f64 = torch.float64
        ws = workspaces.get(positions.device, "f64", _size(lib.nvamd_f64_workspace_bytes, B))
        _check(lib.nvamd_lj_energy_forces_f64(
            _dev(positions, "positions", f64, (N, 3)), _dev(cells, "cells", f64, (B, 3, 3)),
            _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
            _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
            _dev(num_neighbors, "num_neighbors", torch.int32, (N,)),
            _dev(batch_idx, "batch_idx", torch.int32, (N,)),
            N, K, B, int(fill_value), float(epsilon), float(sigma), float(cutoff), float(switch_width),
            int(bool(half_list)), _dev(atomic_energies, "atomic_energies", f64, (N,)),
            _dev(forces, "forces", f64, (N, 3)), _opt(virials, "virials", f64, (B, 9)),
            _opt(system_energies, "system_energies", f64, (B,)),
            ws.data_ptr(), ws.numel(), _stream(positions.device)), "nvamd_lj_energy_forces_f64")
        return
    need = _size(lib.nvamd_lj_workspace_bytes, N, B, int(bool(half_list)))
    ws = workspaces.get(positions.device, "lj", need)
    if not half_list:
        # The per-system tables that the pair kernel keeps in this workspace depend on batch_idx, cells and the
        # list's cutoff only: while those stand as they were at the previous call through the same buffer (same
        # storage, no in-place write since: Torch's version counters), that call's tables are used again.
        tables = (ws.data_ptr(), batch_idx.data_ptr(), batch_idx._version, cells.data_ptr(), cells._version, N, K, B,
                  float(neighbor_list_cutoff), neighbor_matrix_shifts is None, virials is None, system_energies is None)
        state = (positions.device.index, _stream(positions.device))
        reuse = _lj_tables.get(state) == tables
        _lj_tables[state] = tables
        if (pair_tiles is not None and row_order is not None and neighbor_matrix_shifts is not None
                and float(switch_width) == 0.0 and float(neighbor_list_cutoff) > 0.0 and K % 8 == 0):
            index, ordered, records, count = pair_tiles
            _check(lib.nvamd_lj_energy_forces_tiles(
                _dev(positions, "positions", torch.float32, (N, 3)),
                _dev(cells, "cells", torch.float32, (B, 3, 3)),
                _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
                _dev(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
                _dev(num_neighbors, "num_neighbors", torch.int32, (N,)),
                _dev(batch_idx, "batch_idx", torch.int32, (N,)),
                _dev(row_order, "row_order", torch.int32, (N,)),
                _dev(index, "tile_index", torch.int16, (N, K)),
                _dev(ordered, "ordered_positions", torch.float32, (N, 4)),
                _dev(records, "tile_records", torch.int32, (nl_tile_records(N, B), NL_TILE_RECORD_INTS)),
                _dev(count, "tile_count", torch.int32, (1,)), float(neighbor_list_cutoff),
                N, K, B, int(fill_value), float(epsilon), float(sigma), float(cutoff), int(reuse),
                _dev(atomic_energies, "atomic_energies", torch.float32, (N,)),
                _dev(forces, "forces", torch.float32, (N, 3)),
                _opt(virials, "virials", torch.float32, (B, 9)),
                _opt(system_energies, "system_energies", torch.float32, (B,)),
                ws.data_ptr(), ws.numel(), _stream(positions.device)), "nvamd_lj_energy_forces_tiles")
            return
        _check(lib.nvamd_lj_energy_forces_repeat(
            _dev(positions, "positions", torch.float32, (N, 3)),
            _dev(cells, "cells", torch.float32, (B, 3, 3)),
            _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
            _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
            _dev(num_neighbors, "num_neighbors", torch.int32, (N,)),
            _dev(batch_idx, "batch_idx", torch.int32, (N,)),
            _opt(row_order, "row_order", torch.int32, (N,)), float(neighbor_list_cutoff),
            N, K, B, int(fill_value), float(epsilon), float(sigma), float(cutoff), float(switch_width),
            int(reuse),
            _dev(atomic_energies, "atomic_energies", torch.float32, (N,)),
            _dev(forces, "forces", torch.float32, (N, 3)),
            _opt(virials, "virials", torch.float32, (B, 9)),
            _opt(system_energies, "system_energies", torch.float32, (B,)),
            ws.data_ptr(), ws.numel(), _stream(positions.device)), "nvamd_lj_energy_forces_repeat")
        return
    _lj_tables.pop((positions.device.index, _stream(positions.device)), None)  # (a half-list call writes the workspace its own way)
    _check(lib.nvamd_lj_energy_forces_hinted(
        _dev(positions, "positions", torch.float32, (N, 3)),
        _dev(cells, "cells", torch.float32, (B, 3, 3)),
        _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
        _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
        _dev(num_neighbors, "num_neighbors", torch.int32, (N,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(row_order, "row_order", torch.int32, (N,)), float(neighbor_list_cutoff),
        N, K, B, int(fill_value), float(epsilon), float(sigma), float(cutoff), float(switch_width),
        int(bool(half_list)),
        _dev(atomic_energies, "atomic_energies", torch.float32, (N,)),
        _dev(forces, "forces", torch.float32, (N, 3)),
        _opt(virials, "virials", torch.float32, (B, 9)),
        _opt(system_energies, "system_energies", torch.float32, (B,)),
        ws.data_ptr(), ws.numel(), _stream(positions.device)), "nvamd_lj_energy_forces_hinted")


#: per (device, stream): what the pair kernel's tables in the "lj" workspace were last computed for
_lj_tables: dict[tuple, tuple] = {}

LJ_STATIC_MAX_SYSTEMS = 16384


def lj_energy_forces_static(positions, cells, neighbor_matrix, neighbor_matrix_shifts, num_neighbors,
                            batch_idx, fill_value, epsilon, sigma, cutoff, switch_width,
                            atomic_energies, forces, virials=None, system_energies=None, row_order=None,
                            neighbor_list_cutoff: float = 0.0) -> None:
    """``lj_energy_forces`` (full list) through the entry point that allocates nothing: the kernel's
    scratch is a device array built into the library (at most ``LJ_STATIC_MAX_SYSTEMS`` systems;
    calls that overlap on one GPU race)."""
    lib = library()
    N = positions.shape[0]
    K = neighbor_matrix.shape[1]
    B = cells.shape[0]
    _check(lib.nvamd_lj_energy_forces_static(
        _dev(positions, "positions", torch.float32, (N, 3)),
        _dev(cells, "cells", torch.float32, (B, 3, 3)),
        _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
        _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
        _dev(num_neighbors, "num_neighbors", torch.int32, (N,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(row_order, "row_order", torch.int32, (N,)), float(neighbor_list_cutoff),
        N, K, B, int(fill_value), float(epsilon), float(sigma), float(cutoff), float(switch_width),
        _dev(atomic_energies, "atomic_energies", torch.float32, (N,)),
        _dev(forces, "forces", torch.float32, (N, 3)),
        _opt(virials, "virials", torch.float32, (B, 9)),
        _opt(system_energies, "system_energies", torch.float32, (B,)),
        _stream(positions.device)), "nvamd_lj_energy_forces_static")


def nl_atom_order(batch_idx, n_systems: int, atom_order, rebuild_flags=None) -> None:
    """Atom indices in the cell order of the last neighbor build on this device (same sizes)."""
    lib = library()
    N = batch_idx.shape[0]
    need = _size(lib.nvamd_nl_workspace_bytes, N, int(n_systems))
    ws = workspaces.get(batch_idx.device, "nl", need)
    _check(lib.nvamd_nl_atom_order(
        ws.data_ptr(), ws.numel(), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(_as_u8(rebuild_flags), "rebuild_flags", torch.uint8, (int(n_systems),)), N, int(n_systems),
        _dev(atom_order, "atom_order", torch.int32, (N,)), _stream(batch_idx.device)), "nvamd_nl_atom_order")


# --------------------------------------------------------------------------------------------
# integrators
# --------------------------------------------------------------------------------------------
def vv_position_update(positions, velocities, forces, masses, dt, batch_idx, active=None) -> None:
    N = positions.shape[0]
    M = dt.shape[0]
    real = _real_dtype(positions, "positions")
    entry = library().nvamd_vv_position_update_f64 if real == torch.float64 else library().nvamd_vv_position_update
    _check(entry(
        _dev(positions, "positions", real, (N, 3)),
        _dev(velocities, "velocities", real, (N, 3)),
        _dev(forces, "forces", real, (N, 3)),
        _dev(masses, "masses", real, (N,)),
        _dev(dt, "dt", real, (M,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(_as_u8(active), "active", torch.uint8, (M,)),
        N, M, _stream(positions.device)), "nvamd_vv_position_update")


def vv_velocity_finalize(velocities, forces_new, masses, dt, batch_idx, active=None) -> None:
    N = velocities.shape[0]
    M = dt.shape[0]
    real = _real_dtype(velocities, "velocities")
    entry = library().nvamd_vv_velocity_finalize_f64 if real == torch.float64 else library().nvamd_vv_velocity_finalize
    _check(entry(
        _dev(velocities, "velocities", real, (N, 3)),
        _dev(forces_new, "forces_new", real, (N, 3)),
        _dev(masses, "masses", real, (N,)),
        _dev(dt, "dt", real, (M,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(_as_u8(active), "active", torch.uint8, (M,)),
        N, M, _stream(velocities.device)), "nvamd_vv_velocity_finalize")


def vv_finalize_then_update(positions, velocities, forces, masses, dt, batch_idx, active=None) -> None:
    """``vv_velocity_finalize`` then ``vv_position_update`` with the same forces, in one launch (float32)."""
    N = positions.shape[0]
    M = dt.shape[0]
    f32 = torch.float32
    _check(library().nvamd_vv_finalize_then_update(
        _dev(positions, "positions", f32, (N, 3)), _dev(velocities, "velocities", f32, (N, 3)),
        _dev(forces, "forces", f32, (N, 3)), _dev(masses, "masses", f32, (N,)), _dev(dt, "dt", f32, (M,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)), _opt(_as_u8(active), "active", torch.uint8, (M,)),
        N, M, _stream(positions.device)), "nvamd_vv_finalize_then_update")


def fire_step(positions, velocities, forces, masses, alpha, dt, alpha_start, f_alpha, dt_min, dt_max,
              maxstep, n_steps_positive, n_min, f_dec, f_inc, uphill_flag, vf, vv, ff, batch_idx,
              compute_reductions=True, active=None) -> None:
    lib = library()
    N = positions.shape[0]
    M = alpha.shape[0]
    f32, i32 = _real_dtype(positions, "positions"), torch.int32
    if f32 == torch.float64:
        entry = lib.nvamd_fire_step_f64
        ws = workspaces.get(positions.device, "f64", _size(lib.nvamd_f64_workspace_bytes, M))
    else:
        entry = lib.nvamd_fire_step
        # (the kernels keep the slot of their sums in this workspace from call to call, per system: one buffer per
        # number of systems, so that no call meets what a call over more systems left behind)
        ws = workspaces.get(positions.device, f"fire:{M}", _size(lib.nvamd_fire_workspace_bytes, M))
    _check(entry(
        _dev(positions, "positions", f32, (N, 3)), _dev(velocities, "velocities", f32, (N, 3)),
        _dev(forces, "forces", f32, (N, 3)), _dev(masses, "masses", f32, (N,)),
        _dev(alpha, "alpha", f32, (M,)), _dev(dt, "dt", f32, (M,)),
        _dev(alpha_start, "alpha_start", f32, (M,)), _dev(f_alpha, "f_alpha", f32, (M,)),
        _dev(dt_min, "dt_min", f32, (M,)), _dev(dt_max, "dt_max", f32, (M,)),
        _dev(maxstep, "maxstep", f32, (M,)), _dev(n_steps_positive, "n_steps_positive", i32, (M,)),
        _dev(n_min, "n_min", i32, (M,)), _dev(f_dec, "f_dec", f32, (M,)), _dev(f_inc, "f_inc", f32, (M,)),
        _dev(uphill_flag, "uphill_flag", i32, (M,)), _dev(vf, "vf", f32, (M,)), _dev(vv, "vv", f32, (M,)),
        _dev(ff, "ff", f32, (M,)), _dev(batch_idx, "batch_idx", i32, (N,)),
        int(bool(compute_reductions)), _opt(_as_u8(active), "active", torch.uint8, (M,)),
        N, M, ws.data_ptr(), ws.numel(), _stream(positions.device)), "nvamd_fire_step")


def status_migrate(values, threshold: float, status, source_status: int, target_status: int) -> None:
    """``status[s] = target_status`` where ``values[s] <= threshold`` and ``status[s] == source_status``; ``values (M)``
    float32 or float64, ``status`` int64 with at least M contiguous entries (the first M are looked at)."""
    M = values.shape[0]
    real = _real_dtype(values, "values")
    if status.dtype != torch.int64 or not status.is_contiguous() or status.numel() < M or status.device != values.device:
        raise ValueError("status: expected a contiguous int64 tensor of at least as many entries as values, on their device")
    entry = library().nvamd_status_migrate_f64 if real == torch.float64 else library().nvamd_status_migrate
    _check(entry(_dev(values, "values", real, (M,)), float(threshold), status.data_ptr(), int(source_status),
                 int(target_status), M, _stream(values.device)), "nvamd_status_migrate")


def segment_fmax(forces, batch_idx, fmax) -> None:
    N = forces.shape[0]
    M = fmax.shape[0]
    if _real_dtype(forces, "forces") == torch.float64:
        lib = library()
        ws = workspaces.get(forces.device, "f64", _size(lib.nvamd_f64_workspace_bytes, M))
        _check(lib.nvamd_segment_fmax_f64(
            _dev(forces, "forces", torch.float64, (N, 3)), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
            N, M, _dev(fmax, "fmax", torch.float64, (M,)), ws.data_ptr(), ws.numel(), _stream(forces.device)),
            "nvamd_segment_fmax_f64")
        return
    _check(library().nvamd_segment_fmax(
        _dev(forces, "forces", torch.float32, (N, 3)), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        N, M, _dev(fmax, "fmax", torch.float32, (M,)), _stream(forces.device)), "nvamd_segment_fmax")


def nl_rebuild_check(reference_positions, current_positions, batch_idx, rebuild_flags, threshold: float,
                     update_reference: bool = False, cell=None, pbc=None) -> None:
    N = current_positions.shape[0]
    M = rebuild_flags.shape[0]
    if (cell is None) != (pbc is None):
        cell = pbc = None  # the displacement is plain unless both are given
    real = _real_dtype(current_positions, "current_positions")
    entry = library().nvamd_nl_rebuild_check_f64 if real == torch.float64 else library().nvamd_nl_rebuild_check
    _check(entry(
        _dev(reference_positions, "reference_positions", real, (N, 3)),
        _dev(current_positions, "current_positions", real, (N, 3)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(cell, "cell", real, (M, 3, 3)), _opt(_as_u8(pbc), "pbc", torch.uint8, (M, 3)),
        N, M, float(threshold), int(bool(update_reference)),
        _dev(_as_u8(rebuild_flags), "rebuild_flags", torch.uint8, (M,)),
        _stream(current_positions.device)), "nvamd_nl_rebuild_check")


def wrap_positions(positions, cell, pbc, batch_idx) -> None:
    N = positions.shape[0]
    M = cell.shape[0]
    real = _real_dtype(positions, "positions")
    entry = library().nvamd_wrap_positions_f64 if real == torch.float64 else library().nvamd_wrap_positions
    _check(entry(
        _dev(positions, "positions", real, (N, 3)), _dev(cell, "cell", real, (M, 3, 3)),
        _dev(_as_u8(pbc), "pbc", torch.uint8, (M, 3)), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        N, M, _stream(positions.device)), "nvamd_wrap_positions")


SEGMENT_OPS = {"sum": 0, "amax": 1, "amin": 2, "mean": 3}


def segment_reduce(values, batch_idx, out, op: str) -> None:
    lib = library()
    n = values.shape[0]
    m = out.shape[0]
    ws = workspaces.get(values.device, "segment", _size(lib.nvamd_segment_workspace_bytes, m))
    _check(lib.nvamd_segment_reduce(
        _dev(values, "values", torch.float32, (n,)), _dev(batch_idx, "batch_idx", torch.int32, (n,)),
        n, m, SEGMENT_OPS[op], _dev(out, "out", torch.float32, (m,)), ws.data_ptr(), ws.numel(),
        _stream(values.device)), "nvamd_segment_reduce")


def kinetic_energy(velocities, masses, batch_idx, out) -> None:
    lib = library()
    n = velocities.shape[0]
    m = out.shape[0]
    ws = workspaces.get(velocities.device, "segment", _size(lib.nvamd_segment_workspace_bytes, m))
    _check(lib.nvamd_kinetic_energy(
        _dev(velocities, "velocities", torch.float32, (n, 3)), _dev(masses, "masses", torch.float32, (n,)),
        _dev(batch_idx, "batch_idx", torch.int32, (n,)), n, m, _dev(out, "kinetic_energy", torch.float32, (m,)),
        ws.data_ptr(), ws.numel(), _stream(velocities.device)), "nvamd_kinetic_energy")


# --------------------------------------------------------------------------------------------
# masked copy / compaction of rows and segments
# --------------------------------------------------------------------------------------------
BUFFER_DTYPES = (torch.bool, torch.float32, torch.float64, torch.int32, torch.int64)


def _rows(t: torch.Tensor, name: str) -> tuple[int, int]:
    """Device pointer and bytes per row of a contiguous (rows, ...) tensor of a supported dtype."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor, got {type(t).__name__}")
    if t.device.type != "cuda":
        raise KernelLibraryError(f"{name}: tensor is on {t.device}; the nvalchemi_amd kernels run on a ROCm device only")
    if t.dtype not in BUFFER_DTYPES:
        raise KeyError(t.dtype)
    if not t.is_contiguous():
        raise ValueError(f"{name}: tensor must be contiguous")
    return t.data_ptr(), math.prod(t.shape[1:]) * t.element_size()


def _mask(t: torch.Tensor, name: str, n: int) -> int:
    return _dev(_as_u8(t), name, torch.uint8, (n,))


def _buffer_ws(device, n_systems: int, data_bytes: int = 0) -> torch.Tensor:
    if torch.device(device).type != "cuda":
        raise KernelLibraryError(f"tensors are on {device}; the nvalchemi_amd kernels run on a ROCm device only")
    need = _size(library().nvamd_buffer_workspace_bytes, int(n_systems), int(data_bytes))
    return workspaces.get(device, "buffers", need)


def put_masked_per_system(source, source_mask, dest, dest_mask, source_data_copied) -> None:
    n_src, n_dest = source.shape[0], dest.shape[0]
    if source.dtype != dest.dtype:
        raise TypeError(f"source {source.dtype} and dest {dest.dtype} differ")
    sp, rb = _rows(source, "source")
    dp, rb_d = _rows(dest, "dest")
    if n_src and n_dest and rb != rb_d:
        raise ValueError(f"source rows have {rb} bytes, dest rows {rb_d}")
    ws = _buffer_ws(source.device, n_src)
    _check(library().nvamd_put_masked_per_system(
        sp, _mask(source_mask, "source_mask", n_src), dp, _mask(dest_mask, "dest_mask", n_dest),
        _mask(source_data_copied, "source_data_copied", n_src), n_src, n_dest, rb, ws.data_ptr(), ws.numel(),
        _stream(source.device)), "nvamd_put_masked_per_system")


def put_fit_mask_per_system(source_mask, dest_mask, fit_mask) -> None:
    n_src, n_dest = source_mask.shape[0], dest_mask.shape[0]
    ws = _buffer_ws(source_mask.device, n_src)
    _check(library().nvamd_put_fit_mask_per_system(
        _mask(source_mask, "source_mask", n_src), _mask(dest_mask, "dest_mask", n_dest),
        _mask(fit_mask, "fit_mask", n_src), n_src, n_dest, ws.data_ptr(), ws.numel(),
        _stream(source_mask.device)), "nvamd_put_fit_mask_per_system")


def defrag_per_system(source, source_data_copied) -> None:
    n = source.shape[0]
    sp, rb = _rows(source, "source")
    ws = _buffer_ws(source.device, n, n * rb)
    _check(library().nvamd_defrag_per_system(
        sp, _mask(source_data_copied, "source_data_copied", n), n, rb, ws.data_ptr(), ws.numel(),
        _stream(source.device)), "nvamd_defrag_per_system")


def put_masked_segmented(source, source_batch_ptr, source_mask, dest, dest_batch_ptr, num_dest_segments: int,
                         source_data_copied, new_num_dest) -> None:
    n = source_batch_ptr.shape[0] - 1
    if source.dtype != dest.dtype:
        raise TypeError(f"source {source.dtype} and dest {dest.dtype} differ")
    sp, rb = _rows(source, "source")
    dp, rb_d = _rows(dest, "dest")
    if source.shape[0] and dest.shape[0] and rb != rb_d:
        raise ValueError(f"source rows have {rb} bytes, dest rows {rb_d}")
    ws = _buffer_ws(source.device, n)
    _check(library().nvamd_put_masked_segmented(
        sp, _dev(source_batch_ptr, "source_batch_ptr", torch.int32, (n + 1,)), _mask(source_mask, "source_mask", n),
        dp, _dev(dest_batch_ptr, "dest_batch_ptr", torch.int32), int(num_dest_segments), dest.shape[0],
        _mask(source_data_copied, "source_data_copied", n), _dev(new_num_dest, "new_num_dest", torch.int32, (1,)),
        n, source.shape[0], rb if source.shape[0] else rb_d, ws.data_ptr(), ws.numel(), _stream(source.device)),
        "nvamd_put_masked_segmented")


def put_fit_mask_segmented(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments: int,
                           dest_capacity: int, fit_mask) -> None:
    n = source_batch_ptr.shape[0] - 1
    ws = _buffer_ws(source_batch_ptr.device, n)
    _check(library().nvamd_put_fit_mask_segmented(
        _dev(source_batch_ptr, "source_batch_ptr", torch.int32, (n + 1,)), _mask(source_mask, "source_mask", n),
        _dev(dest_batch_ptr, "dest_batch_ptr", torch.int32), int(num_dest_segments), int(dest_capacity),
        _mask(fit_mask, "fit_mask", n), n, ws.data_ptr(), ws.numel(), _stream(source_batch_ptr.device)),
        "nvamd_put_fit_mask_segmented")


def defrag_segmented(source, source_batch_ptr, source_data_copied, num_kept) -> None:
    n = source_batch_ptr.shape[0] - 1
    sp, rb = _rows(source, "source")
    rows = source.shape[0]
    ws = _buffer_ws(source.device, n, rows * rb)
    _check(library().nvamd_defrag_segmented(
        sp, _dev(source_batch_ptr, "source_batch_ptr", torch.int32, (n + 1,)),
        _mask(source_data_copied, "source_data_copied", n), _dev(num_kept, "num_kept", torch.int32, (1,)),
        n, rows, rb, ws.data_ptr(), ws.numel(), _stream(source.device)), "nvamd_defrag_segmented")


# --------------------------------------------------------------------------------------------
# filtering a list to a tighter cutoff
# --------------------------------------------------------------------------------------------
def _cells_arg(cell, n_systems_hint=None):
    if cell is None:
        return None, 0
    if cell.dim() == 2:
        return _dev(cell, "cell", torch.float32, (3, 3)), 0
    return _dev(cell, "cell", torch.float32, (None, 3, 3)), 1


def nl_filter_matrix(positions, cell, neighbor_matrix, neighbor_matrix_shifts, batch_idx, fill_value: int,
                     cutoff: float, out_matrix, out_counts, out_shifts) -> None:
    N, K = neighbor_matrix.shape
    cp, per_system = _cells_arg(cell)
    _check(library().nvamd_nl_filter_matrix(
        _dev(positions, "positions", torch.float32, (N, 3)), cp, per_system,
        _dev(neighbor_matrix, "neighbor_matrix", torch.int32, (N, K)),
        _opt(neighbor_matrix_shifts, "neighbor_matrix_shifts", torch.int32, (N, K, 3)),
        _opt(batch_idx, "batch_idx", torch.int32, (N,)), N, K, int(fill_value), float(cutoff),
        _dev(out_matrix, "out_matrix", torch.int32, (N, K)), _dev(out_counts, "out_counts", torch.int32, (N,)),
        _opt(out_shifts, "out_shifts", torch.int32, (N, K, 3)), _stream(positions.device)), "nvamd_nl_filter_matrix")


def nl_filter_coo_flags(positions, cell, neighbor_list, neighbor_list_shifts, batch_idx, cutoff: float, keep) -> None:
    N = positions.shape[0]
    E = neighbor_list.shape[0]
    cp, per_system = _cells_arg(cell)
    _check(library().nvamd_nl_filter_coo_flags(
        _dev(positions, "positions", torch.float32, (N, 3)), cp, per_system,
        _dev(neighbor_list, "neighbor_list", torch.int32, (E, 2)),
        _opt(neighbor_list_shifts, "neighbor_list_shifts", torch.int32, (E, 3)),
        _opt(batch_idx, "batch_idx", torch.int32, (N,)), E, float(cutoff),
        _dev(_as_u8(keep), "keep", torch.uint8, (E,)), _stream(positions.device)), "nvamd_nl_filter_coo_flags")


# --------------------------------------------------------------------------------------------
# Langevin
# --------------------------------------------------------------------------------------------
def langevin_half_step(positions, velocities, forces, masses, dt, kT, friction, random_seed: int, batch_idx,
                       active=None) -> None:
    N = positions.shape[0]
    M = dt.shape[0]
    real = _real_dtype(positions, "positions")  # float32 or float64: every float array in that one type
    entry = library().nvamd_langevin_half_step_f64 if real == torch.float64 else library().nvamd_langevin_half_step
    _check(entry(
        _dev(positions, "positions", real, (N, 3)), _dev(velocities, "velocities", real, (N, 3)),
        _dev(forces, "forces", real, (N, 3)), _dev(masses, "masses", real, (N,)),
        _dev(dt, "dt", real, (M,)), _dev(kT, "temperature", real, (M,)),
        _dev(friction, "friction", real, (M,)), int(random_seed) & 0xFFFFFFFFFFFFFFFF,
        _dev(batch_idx, "batch_idx", torch.int32, (N,)), _opt(_as_u8(active), "active", torch.uint8, (M,)),
        N, M, _stream(positions.device)), "nvamd_langevin_half_step")


# --------------------------------------------------------------------------------------------
# Nose-Hoover chain
# --------------------------------------------------------------------------------------------
def nhc_chain_update(velocities, masses, eta, eta_dot, chain_masses, kT, dt, ndof, ke2, total_scale, batch_idx,
                     compute_ke: bool = True, yoshida_order: int = 3, active=None) -> None:
    lib = library()
    N = velocities.shape[0]
    M, C = eta.shape
    ws = workspaces.get(velocities.device, "nhc", _size(lib.nvamd_nhc_workspace_bytes, M))
    real = _real_dtype(velocities, "velocities")  # float32 or float64: every float array in that one type
    entry = lib.nvamd_nhc_chain_update_f64 if real == torch.float64 else lib.nvamd_nhc_chain_update
    _check(entry(
        _dev(velocities, "velocities", real, (N, 3)), _dev(masses, "masses", real, (N,)),
        _dev(eta, "eta", real, (M, C)), _dev(eta_dot, "eta_dot", real, (M, C)),
        _dev(chain_masses, "Q", real, (M, C)), _dev(kT, "temperature", real, (M,)),
        _dev(dt, "dt", real, (M,)), _dev(ndof, "ndof", real, (M,)),
        _dev(ke2, "ke2", real, (M,)), _dev(total_scale, "total_scale", real, (M,)),
        _dev(batch_idx, "batch_idx", torch.int32, (N,)), _opt(_as_u8(active), "active", torch.uint8, (M,)),
        1 if compute_ke else 0, C, int(yoshida_order), N, M, ws.data_ptr(), ws.numel(),
        _stream(velocities.device)), "nvamd_nhc_chain_update")


def nhc_position_update(positions, velocities, dt, batch_idx, active=None) -> None:
    N = positions.shape[0]
    M = dt.shape[0]
    real = _real_dtype(positions, "positions")
    entry = library().nvamd_nhc_position_update_f64 if real == torch.float64 else library().nvamd_nhc_position_update
    _check(entry(
        _dev(positions, "positions", real, (N, 3)), _dev(velocities, "velocities", real, (N, 3)),
        _dev(dt, "dt", real, (M,)), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _opt(_as_u8(active), "active", torch.uint8, (M,)), N, M, _stream(positions.device)),
        "nvamd_nhc_position_update")


# --------------------------------------------------------------------------------------------
# FIRE 2.0
# --------------------------------------------------------------------------------------------
def fire2_step(positions, velocities, forces, batch_idx, alpha, dt, nsteps_inc, vf=None, v_sumsq=None,
               f_sumsq=None, max_norm=None, *, delaystep: int, dtgrow: float, dtshrink: float, alphashrink: float,
               alpha0: float, tmax: float, tmin: float, maxstep: float, active=None) -> None:
    lib = library()
    N = positions.shape[0]
    M = dt.shape[0]
    real = _real_dtype(positions, "positions")  # float32 or float64: every float array in that one type
    if real == torch.float64:
        entry = lib.nvamd_fire2_step_f64
        ws = workspaces.get(positions.device, "f64", _size(lib.nvamd_f64_workspace_bytes, M))
    else:
        entry = lib.nvamd_fire2_step
        ws = workspaces.get(positions.device, "fire2", _size(lib.nvamd_fire2_workspace_bytes, M))
    _check(entry(
        _dev(positions, "positions", real, (N, 3)), _dev(velocities, "velocities", real, (N, 3)),
        _dev(forces, "forces", real, (N, 3)), _dev(batch_idx, "batch_idx", torch.int32, (N,)),
        _dev(alpha, "alpha", real, (M,)), _dev(dt, "dt", real, (M,)),
        _dev(nsteps_inc, "nsteps_inc", torch.int32, (M,)), _opt(vf, "vf", real, (M,)),
        _opt(v_sumsq, "v_sumsq", real, (M,)), _opt(f_sumsq, "f_sumsq", real, (M,)),
        _opt(max_norm, "max_norm", real, (M,)), int(delaystep), float(dtgrow), float(dtshrink),
        float(alphashrink), float(alpha0), float(tmax), float(tmin), float(maxstep),
        _opt(_as_u8(active), "active", torch.uint8, (M,)), N, M, ws.data_ptr(), ws.numel(),
        _stream(positions.device)), "nvamd_fire2_step")
