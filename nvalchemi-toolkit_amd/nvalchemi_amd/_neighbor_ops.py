"""The neighbor functions the reference imports from its ops wheel, backed by the HIP
library: ``neighbor_list`` (nvalchemi/neighbors.py:253-266,
nvalchemi/hooks/neighbor_list.py:328-343), ``estimate_max_neighbors``
(nvalchemi/neighbors.py:228) and ``get_neighbor_list_from_neighbor_matrix``
(nvalchemi/neighbors.py:92-103).
"""

from __future__ import annotations

import math

import torch

from . import _lib

_METHODS = {None, "naive", "cell_list", "batch_naive", "batch_cell_list", "batch_cell_list_pair_centric",
            "batch_cluster_tile", "cluster_tile", "naive_tile"}


def ceil16(n: int) -> int:
    return ((int(n) + 15) // 16) * 16


def estimate_max_neighbors(cutoff: float, atomic_density: float = 0.2, safety_factor: float = 1.5) -> int:
    """Row width guess: atoms in the cutoff sphere at ``atomic_density``, times a safety
    factor, rounded up to 16.  Only the buffer width depends on it, never the list: callers
    grow on overflow and trim on over-estimate."""
    expected = atomic_density * (4.0 / 3.0) * math.pi * float(cutoff) ** 3
    return max(16, ceil16(math.ceil(safety_factor * expected)))


def suggest_neighbor_list_method(batch_ptr: torch.Tensor, cell: torch.Tensor, pbc: torch.Tensor, cutoff: float,
                                 half_fill: bool = False, return_neighbor_list: bool = False,
                                 positions_dtype: torch.dtype = torch.float32) -> str:
    """Strategy name for the caller's bookkeeping (call site: nvalchemi/hooks/neighbor_list.py:737-747).
    One cell-list kernel serves every input here, so the answer only says "batched cell list"; the
    reference's cost model lives in its kernel library and picks among strategies this build does
    not have.  Host-only, no synchronisation."""
    if positions_dtype not in (torch.float32, torch.float64):
        raise TypeError(f"neighbor list positions must be float32 or float64, got {positions_dtype}")
    return "batch_cell_list"


def neighbor_list_strategy_run_args(method: str) -> tuple[str, dict]:
    """``(base method, extra keyword arguments)`` of a strategy name (call site:
    nvalchemi/hooks/neighbor_list.py:757-760, which only uses element 0 to choose the scratch it
    allocates).  No strategy of this build takes caller-side scratch: the base name is returned
    with no arguments, and the scratch allocators the reference imports optionally
    (``estimate_batch_cell_list_sizes``, ``allocate_cell_list``, ``compute_naive_num_shifts``,
    ``allocate_batch_cluster_tile_list``, ``estimate_batch_max_tiles_per_group``) have no
    counterpart -- the caller's ``except ImportError`` branches leave them ``None``."""
    if method not in _METHODS or method is None:
        raise ValueError(f"unknown neighbor list method {method!r}")
    base = {"batch_cell_list_pair_centric": "batch_cell_list"}.get(method, method)
    return base, {}


def neighbor_list(positions: torch.Tensor, cutoff: float, cell: torch.Tensor | None = None,
                  pbc: torch.Tensor | None = None, max_neighbors: int | None = None,
                  half_fill: bool = False, batch_ptr: torch.Tensor | None = None,
                  batch_idx: torch.Tensor | None = None, neighbor_matrix: torch.Tensor | None = None,
                  num_neighbors: torch.Tensor | None = None,
                  neighbor_matrix_shifts: torch.Tensor | None = None,
                  rebuild_flags: torch.Tensor | None = None, method: str | None = None,
                  tail_mode: int = 1, pair_tiles: tuple | None = None, shift_groups: torch.Tensor | None = None,
                  **scratch) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """Build the dense neighbor list in place and return ``(neighbor_matrix, num_neighbors,
    neighbor_matrix_shifts)``.

    ``neighbor_matrix (N,K)`` int32 must arrive padded with ``N`` (or hold a previous
    result), ``num_neighbors (N)`` int32 zeroed (or the previous counts); they are allocated
    when ``None``.  ``num_neighbors`` keeps counting past ``K``: ``max >= K`` means overflow.
    ``cell``/``pbc`` ``None`` means non-periodic.  ``rebuild_flags (B) bool``: systems with
    ``False`` keep their rows.  ``method`` is accepted for compatibility (one cell-list
    kernel serves every case); scratch keyword tensors of the reference's strategies are
    ignored.  ``tail_mode=1`` rewrites the padding of every rebuilt row; ``0`` only clears
    what the previous build left (persistent buffers that only this function writes).
    ``pair_tiles`` (not in the reference): four preallocated tensors in which the build also leaves what the
    pair kernel of large systems walks, see ``_lib.nl_build``.  ``shift_groups`` (not in the reference): the
    record that lets a build on persistent buffers skip the stores of zero shifts over zeros, see ``_lib.nl_build``.
    """
    if method not in _METHODS:
        raise ValueError(f"unknown neighbor list method {method!r}")
    if positions.dtype not in (torch.float32, torch.float64):
        raise TypeError(f"neighbor list positions must be float32 or float64, got {positions.dtype}")
    N = positions.shape[0]
    dev = positions.device
    if batch_ptr is None:
        batch_ptr = torch.tensor([0, N], dtype=torch.int32, device=dev)
    if batch_idx is None:
        B = batch_ptr.shape[0] - 1
        batch_idx = torch.repeat_interleave(torch.arange(B, dtype=torch.int32, device=dev),
                                            (batch_ptr[1:] - batch_ptr[:-1]).to(torch.long), output_size=N)
    B = batch_ptr.shape[0] - 1
    if (cell is None) != (pbc is None):
        if cell is None:
            pbc = None
        else:
            pbc = torch.zeros(B, 3, dtype=torch.bool, device=dev)
    if cell is not None:
        cell = cell.to(positions.dtype).reshape(B, 3, 3).contiguous()
        pbc = pbc.reshape(B, 3).contiguous()
    K = int(max_neighbors if max_neighbors is not None else
            (neighbor_matrix.shape[1] if neighbor_matrix is not None else estimate_max_neighbors(cutoff)))
    if neighbor_matrix is None:
        neighbor_matrix = torch.full((N, K), N, dtype=torch.int32, device=dev)
    if num_neighbors is None:
        num_neighbors = torch.zeros(N, dtype=torch.int32, device=dev)
    if neighbor_matrix_shifts is None and cell is not None:
        neighbor_matrix_shifts = torch.zeros((N, K, 3), dtype=torch.int32, device=dev)
    _lib.nl_build(positions.contiguous(), cell, pbc, batch_ptr.to(torch.int32).contiguous(),
                  batch_idx.to(torch.int32).contiguous(), rebuild_flags, cutoff, K, half_fill, tail_mode,
                  neighbor_matrix, num_neighbors, neighbor_matrix_shifts if cell is not None else None,
                  pair_tiles=pair_tiles, shift_groups=shift_groups if cell is not None else None)
    return neighbor_matrix, num_neighbors, neighbor_matrix_shifts


#: edge count of the last conversion of a matrix of the same shape: the capacity the next one starts with
_last_edge_count: dict[tuple, int] = {}


def get_neighbor_list_from_neighbor_matrix(neighbor_matrix: torch.Tensor, num_neighbors: torch.Tensor,
                                           neighbor_shift_matrix: torch.Tensor | None = None,
                                           fill_value: int | None = None):
    """Dense -> COO in row-major order.  Returns ``(edges (2,E) int32, edge_ptr (N+1) int32[,
    shifts (E,3) int32])`` like the reference's helper (the caller transposes ``[0]``).

    The edge pointer is scanned and the edges are written on the device in one call, into buffers
    sized by the edge count of the previous conversion of a matrix of this shape (plus headroom);
    the host then reads the count once, to cut the views to size (tensor shapes live on the host:
    the reference's helper waits for the same number), and repeats the call with larger buffers
    only if they were too small."""
    N, K = neighbor_matrix.shape
    dev = neighbor_matrix.device
    key = (dev.index, N, K)
    guess = _last_edge_count.get(key)
    cap = N * K if guess is None else min(N * K, int(guess * 1.05) + 1024)
    if guess is None and N * K > (1 << 22):
        cap = 0  # a first conversion of a large matrix: count first, rather than allocate N x K edges
    edge_ptr = torch.empty(N + 1, dtype=torch.int32, device=dev)
    counts = torch.empty(2, dtype=torch.int32, device=dev)
    want_shifts = neighbor_shift_matrix is not None
    while True:
        edges = torch.empty((cap, 2), dtype=torch.int32, device=dev)
        shifts = torch.empty((cap, 3), dtype=torch.int32, device=dev) if want_shifts else None
        _lib.nl_coo_from_matrix(neighbor_matrix, neighbor_shift_matrix, num_neighbors, edge_ptr, edges, shifts, counts)
        E, over = (int(v) for v in counts.tolist())
        if not over:
            break
        cap = E
    _last_edge_count[key] = E
    edges = edges[:E]
    if not want_shifts:
        return edges.T, edge_ptr
    return edges.T, edge_ptr, shifts[:E]
