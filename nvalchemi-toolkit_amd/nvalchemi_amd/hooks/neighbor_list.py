"""``NeighborListHook``: rebuild the neighbor list before each model evaluation.

Mirror of nvalchemi/hooks/neighbor_list.py:112-760 for what callers see: constructor
``(config, skin, max_neighbors, stage, method)``, the persistent result buffers
``_neighbor_matrix`` / ``_num_neighbors`` / ``_neighbor_matrix_shifts`` (read by other
wrappers, nvalchemi/models/pipeline.py:185-196), the K policy (start from the estimate or
the override; without PBC cap at ceil16(max atoms per system); after the first build grow
to ceil16(1.5*actual) on overflow and re-run, or trim to ceil16(2*actual) when
over-estimated, never below the override; :401-486), and the published batch keys.

Differences in mechanism, not in results: there are no staging copies (the kernels read the
batch tensors directly), and the padding of rows is maintained by the build kernel itself
instead of a masked fill over the whole ``(N,K)`` buffers after every build (:377-380).
With ``skin > 0`` the list is searched out to ``cutoff + skin`` and, from the second call on, only
the systems in which some atom moved more than ``skin / 2`` since their last build are rebuilt
(:295-311; the displacement is the plain one, so that an atom wrapped back into the cell by another
hook counts as moved and the shifts of its system are made afresh): the displacement test writes the per-system ``_rebuild_flags`` and refreshes
``_ref_positions`` for the flagged systems, and the build kernel leaves the rows of the others as
they are.  The potential applies the bare cutoff to the wider list.
"""

from __future__ import annotations

from enum import Enum

import torch

from .. import _lib
from .._neighbor_ops import ceil16, estimate_max_neighbors, neighbor_list
from ..dynamics._ops.neighbor_list_rebuild import batch_neighbor_list_rebuild_inplace
from ..models.base import NeighborConfig, NeighborListFormat
from ..neighbors import _raise_on_truncated_search, _write_neighbor_data_to_batch
from ._context import HookContext


class NeighborListHook:
    """Compute and cache neighbor lists at ``DynamicsStage.BEFORE_COMPUTE``.

    Parameters
    ----------
    config : NeighborConfig
        Cutoff, format (MATRIX or COO) and half-list flag of the model.
    skin : float
        Extra search radius; see the module note.
    max_neighbors : int | None
        Row width K for the matrix; estimated from the cutoff when ``None``.  Acts as a
        floor when the hook trims an over-estimate.
    stage : Enum | None
        Stage the hook fires at (assigned at registration when ``None``).
    method : str | None
        Accepted for compatibility with the reference's strategy names.
    min_image_skin : bool
        How far an atom has moved since its system's last build.  ``False`` (default): the plain
        displacement, so an atom that a wrap hook has moved by a lattice vector counts as moved and its
        system is rebuilt (the rows that are kept hold integer shifts that belong to the coordinates they
        were built from).  ``True``: the displacement reduced to the nearest image, as the reference does
        (nvalchemi/hooks/neighbor_list.py:295-311): a wrap then triggers nothing, and the stored shifts of a
        wrapped atom's pairs are stale until its system's next build.  Only for a consumer that does not
        read the stored shifts of such systems (the pair kernel of this package derives them from the
        positions where every width of the cell exceeds twice the search radius).
    """

    def __init__(self, config: NeighborConfig, skin: float = 0.0, max_neighbors: int | None = None,
                 stage: Enum | None = None, method: str | None = None, min_image_skin: bool = False) -> None:
        self.config = config
        self.skin = skin
        self.min_image_skin = bool(min_image_skin)
        self.stage = stage
        self.method = method
        self._max_neighbors_override = max_neighbors
        self.frequency = 1
        self._neighbor_list_flag = config.format == NeighborListFormat.COO

        self._neighbor_matrix: torch.Tensor | None = None
        self._num_neighbors: torch.Tensor | None = None
        self._neighbor_matrix_shifts: torch.Tensor | None = None
        self._max_neighbors: int = 0
        self._alloc_N: int | None = None
        self._alloc_B: int | None = None
        self._alloc_periodic: bool | None = None
        self._neighbor_list_method: str | None = None
        self._actual_max_k: torch.Tensor | None = None
        self._first_build: bool = True
        # Verlet-skin state: positions at the last build of each system, per-system flags
        self._ref_positions: torch.Tensor | None = None
        self._rebuild_flags: torch.Tensor | None = None
        # what a full build leaves for the pair kernel of large systems, and whether the last build wrote it
        self._tiles: tuple | None = None
        self._tiles_fresh: bool = False
        # per row, which groups of slots of the shifts may hold a shift that is not zero (the build leaves zeros over
        # zeros unwritten); lives and dies with the shifts buffer
        self._shift_groups: torch.Tensor | None = None
        self._shift_groups_stale: bool = False

    def __call__(self, ctx: HookContext, stage: Enum) -> None:
        self._rebuild(ctx.batch)
        # first build: initialise the skin reference (one-time clone)
        if self.skin > 0.0 and self._ref_positions is None:
            self._ref_positions = ctx.batch.positions.detach().clone()

    # ------------------------------------------------------------------
    def _rebuild(self, batch) -> None:
        positions = batch.positions
        N = batch.num_nodes
        B = batch.num_graphs
        pbc = getattr(batch, "pbc", None)
        cell = getattr(batch, "cell", None)
        if cell is None:
            pbc = None
        periodic = pbc is not None

        if (self._neighbor_matrix is None or self._neighbor_matrix.shape[0] != N
                or self._alloc_periodic != periodic or self._neighbor_matrix.device != positions.device):
            self._alloc_output_tensors(N, batch, pbc)
            self._alloc_periodic = periodic
        if self._alloc_N != N or self._alloc_B != B:
            self._neighbor_list_method = self._select_neighbor_list_method(N, B)
            self._alloc_N = N
            self._alloc_B = B

        if self._rebuild_flags is None or self._rebuild_flags.shape[0] != B \
                or self._rebuild_flags.device != positions.device:
            # all true, so that a first build (before the reference exists) is a full one
            self._rebuild_flags = torch.ones(B, dtype=torch.bool, device=positions.device)
            self._ref_positions = None
        if self.skin > 0.0 and self._ref_positions is not None:
            # The displacement is the plain one, not the one reduced to the nearest image (the
            # reference passes its cell here, nvalchemi/hooks/neighbor_list.py:295-311): rows that are
            # kept hold integer shifts that belong to the coordinates they were built from, so an
            # atom that a wrap has moved by a lattice vector must count as moved, and its system is
            # rebuilt.  (Only a lattice vector shorter than skin / 2 would escape this.)
            batch_neighbor_list_rebuild_inplace(
                reference_positions=self._ref_positions, current_positions=positions,
                batch_idx=batch.batch_idx, rebuild_flags=self._rebuild_flags,
                skin_distance_threshold=self.skin / 2, update_reference_positions=True,
                cell=cell if self.min_image_skin else None, pbc=pbc if self.min_image_skin else None)

        cutoff = self.config.cutoff + self.skin
        self._build(batch, cutoff, cell, pbc,
                    rebuild_flags=self._rebuild_flags if (self.skin > 0.0 and self._ref_positions is not None) else None)

        first = self._first_build
        if self._first_build:
            # the one host synchronisation: validate K against the actual maximum
            self._first_build = False
            _raise_on_truncated_search(N, B, positions.device, cutoff)
            self._actual_max_k = self._num_neighbors.max() if N > 0 else None
            if self._check_and_resize_k(N, positions.device, pbc):
                self._build(batch, cutoff, cell, pbc, rebuild_flags=None)
                # the grown K must be accepted: one spare slot per row
                while N > 0 and int(self._num_neighbors.max()) >= self._max_neighbors:
                    self._max_neighbors = ceil16(int(int(self._num_neighbors.max()) * 1.5))
                    self._realloc_k(N, positions.device, pbc)
                    self._build(batch, cutoff, cell, pbc, rebuild_flags=None)

        if first and N > 0:
            # whatever earlier builds left in the workspace's status bits (the first build's own overflow
            # has been dealt with above) is not this hook's: overflowed() starts from here
            _lib.nl_status(N, B, positions.device, clear=True)
        self._publish_row_order(batch, N, B)
        _write_neighbor_data_to_batch(
            batch=batch, neighbor_matrix=self._neighbor_matrix, num_neighbors=self._num_neighbors,
            neighbor_matrix_shifts=self._neighbor_matrix_shifts,
            format=NeighborListFormat.COO if self._neighbor_list_flag else NeighborListFormat.MATRIX,
            cutoff=self.config.cutoff, search_cutoff=None if self.config.half_list else cutoff)

    # ---- for a dynamics that replays captured steps ---------------------------------------------------
    @property
    def graph_safe(self) -> bool:
        """After the first build (which sizes the rows with the host's help) a call of this hook is kernels
        on persistent buffers only: it can be captured in a HIP graph and replayed."""
        return self._neighbor_matrix is not None and not self._first_build and \
            (self.skin <= 0.0 or self._ref_positions is not None)

    def graph_key(self) -> tuple:
        """The buffers a captured call is tied to."""
        def ptr(t):
            return None if t is None else (t.data_ptr(), tuple(t.shape))

        return (ptr(self._neighbor_matrix), ptr(self._num_neighbors), ptr(self._neighbor_matrix_shifts),
                ptr(self._ref_positions), ptr(self._rebuild_flags), ptr(getattr(self, "_atom_order", None)),
                None if self._tiles is None else tuple(ptr(t) for t in self._tiles), ptr(self._shift_groups))

    def overflowed(self, clear: bool = True) -> bool:
        """Whether any build since the last call left an atom with more neighbors than the rows hold
        (the reference never notices this after its first build, nvalchemi/hooks/neighbor_list.py:351-355;
        the kernels here count past K on the device and keep a flag).  One host synchronisation.  The flag
        lives in the build's workspace, which all builds of a device and stream share: another hook's
        overflow on the same stream shows up here too."""
        if self._neighbor_matrix is None or self._alloc_N in (None, 0):
            return False
        st = _lib.nl_status(self._alloc_N, self._alloc_B, self._neighbor_matrix.device, clear=clear)
        return bool(int(st[1]) & _lib.NL_STATUS_ROW_OVERFLOW)

    #: systems larger than this do not fit the pair kernel's LDS stage (csrc/lj_pair.hip kLdsAtoms)
    _ROW_ORDER_MIN_ATOMS = 4096

    def _publish_row_order(self, batch, N: int, B: int) -> None:
        """For batches with systems too large for the pair kernel to stage in LDS, leave the
        atoms' cell order of this build on the batch (``_neighbor_row_order``): a pair kernel that
        walks its rows in that order gathers neighbor positions from the caches instead of HBM.
        Not part of the reference; purely a hint (any model may ignore it)."""
        tiles = self._tiles if self._tiles_fresh else None
        self._tiles_fresh = False
        if N == 0 or batch.max_num_nodes <= self._ROW_ORDER_MIN_ATOMS:
            if getattr(batch, "_neighbor_row_order", None) is not None:
                object.__setattr__(batch, "_neighbor_row_order", None)
            if getattr(batch, "_neighbor_pair_tiles", None) is not None:
                object.__setattr__(batch, "_neighbor_pair_tiles", None)
            self._atom_order = None
            return
        fresh = (getattr(self, "_atom_order", None) is None or self._atom_order.shape[0] != N
                 or self._atom_order.device != batch.positions.device)
        if fresh:
            self._atom_order = torch.empty(N, dtype=torch.int32, device=batch.positions.device)
        flags = None
        if not fresh and self.skin > 0.0 and self._ref_positions is not None:
            flags = self._rebuild_flags  # systems that were not rebuilt keep the order of their last build
        _lib.nl_atom_order(batch.batch_idx, B, self._atom_order, flags)
        object.__setattr__(batch, "_neighbor_row_order", self._atom_order)
        # what the last build left for the pair kernel, tied to the positions and the matrix of that build
        # (storage and version)
        object.__setattr__(batch, "_neighbor_pair_tiles",
                           None if tiles is None else
                           tiles + (batch.positions.data_ptr(), batch.positions._version,
                                    self._neighbor_matrix.data_ptr()))

    def _pair_tiles_for(self, batch, cell, rebuild_flags):
        """Buffers for what a full build leaves to the pair kernel of systems too large to stage whole (the atoms in
        cell order, the search's tiles, each pair's place in its tile), or None where that does not apply: lists kept
        over several steps, half lists, float64, open systems, small systems."""
        N, B = batch.num_nodes, batch.num_graphs
        K = self._max_neighbors
        if (self.skin > 0.0 or rebuild_flags is not None or self.config.half_list or cell is None or N == 0
                or batch.positions.dtype != torch.float32 or N // max(B, 1) <= self._ROW_ORDER_MIN_ATOMS or K % 8 != 0):
            return None
        dev = batch.positions.device
        t = self._tiles
        if t is None or tuple(t[0].shape) != (N, K) or t[0].device != dev or t[2].shape[0] != _lib.nl_tile_records(N, B):
            t = (torch.empty(N, K, dtype=torch.int16, device=dev), torch.empty(N, 4, dtype=torch.float32, device=dev),
                 torch.empty(_lib.nl_tile_records(N, B), _lib.NL_TILE_RECORD_INTS, dtype=torch.int32, device=dev),
                 torch.zeros(1, dtype=torch.int32, device=dev))
            self._tiles = t
        return t

    def _build(self, batch, cutoff, cell, pbc, rebuild_flags) -> None:
        tiles = self._pair_tiles_for(batch, cell, rebuild_flags)
        # Leaving zero shifts over zeros unwritten pays where most atoms are further than the cutoff from every face of
        # their cell (measured: a tenth off the build of one box of 4 M atoms; a tenth on for boxes of 3900 atoms,
        # where three rows in four hold a shifted pair and the bookkeeping costs more than the stores it saves).
        groups = None
        if self._shift_groups is not None:
            if (batch.positions.dtype == torch.float32
                    and batch.num_nodes // max(batch.num_graphs, 1) > self._ROW_ORDER_MIN_ATOMS):
                groups = self._shift_groups
            elif not self._shift_groups_stale:
                self._shift_groups.fill_(-1)  # (a build that writes every shift keeps no record of where the zeros are)
                self._shift_groups_stale = True
        if groups is not None:
            self._shift_groups_stale = False
        neighbor_list(positions=batch.positions, cutoff=cutoff, cell=cell, pbc=pbc,
                      max_neighbors=self._max_neighbors, half_fill=self.config.half_list,
                      batch_ptr=batch.batch_ptr, batch_idx=batch.batch_idx,
                      neighbor_matrix=self._neighbor_matrix, num_neighbors=self._num_neighbors,
                      neighbor_matrix_shifts=self._neighbor_matrix_shifts, rebuild_flags=rebuild_flags,
                      method=self._neighbor_list_method, tail_mode=0, pair_tiles=tiles, shift_groups=groups)
        self._tiles_fresh = tiles is not None

    # ------------------------------------------------------------------
    def _alloc_output_tensors(self, N: int, batch, pbc: torch.Tensor | None) -> None:
        """(Re)allocate the result buffers for atom count *N* and reset the K check."""
        max_nbrs = self._max_neighbors_override
        if max_nbrs is None:
            max_nbrs = estimate_max_neighbors(cutoff=self.config.cutoff + self.skin)
        if pbc is None and batch.max_num_nodes > 0:
            max_nbrs = min(max_nbrs, ceil16(batch.max_num_nodes))
        self._max_neighbors = int(max_nbrs)
        self._realloc_k(N, batch.device, pbc)
        self._first_build = True
        self._actual_max_k = None
        # new buffers hold no list: the next build is a full one and re-initialises the reference
        self._ref_positions = None
        self._rebuild_flags = None

    def _realloc_k(self, N: int, device: torch.device, pbc: torch.Tensor | None) -> None:
        K = self._max_neighbors
        self._neighbor_matrix = torch.full((N, K), N, dtype=torch.int32, device=device)
        self._num_neighbors = torch.zeros(N, dtype=torch.int32, device=device)
        self._neighbor_matrix_shifts = (
            torch.zeros(N, K, 3, dtype=torch.int32, device=device) if pbc is not None else None)
        self._shift_groups = torch.zeros(N, dtype=torch.int32, device=device) if pbc is not None else None
        self._shift_groups_stale = False

    def _check_and_resize_k(self, N: int, device: torch.device, pbc: torch.Tensor | None) -> bool:
        """Compare K with the actual maximum (host sync).  Returns ``True`` if K grew and the
        build must be re-run; an over-estimate is trimmed in place."""
        if self._actual_max_k is None:
            return False
        actual = int(self._actual_max_k.item())
        if actual >= self._max_neighbors:
            self._max_neighbors = ceil16(int(actual * 1.5))
            self._realloc_k(N, device, pbc)
            return True
        if 0 < actual < 0.5 * self._max_neighbors:
            new_k = ceil16(int(actual * 2))
            if self._max_neighbors_override is not None:
                new_k = max(new_k, self._max_neighbors_override)
            if new_k < self._max_neighbors:
                self._max_neighbors = new_k
                self._neighbor_matrix = self._neighbor_matrix[:, :new_k].contiguous()
                if self._neighbor_matrix_shifts is not None:
                    self._neighbor_matrix_shifts = self._neighbor_matrix_shifts[:, :new_k].contiguous()
                    # (the groups were those of the longer rows: every slot counts as written until the next build)
                    self._shift_groups.fill_(-1)
        return False

    def _select_neighbor_list_method(self, N: int, B: int) -> str:
        """Name of the strategy, as the reference would report it; one kernel serves both."""
        if self.method is not None:
            return self.method
        return "cell_list" if N // max(B, 1) >= 2000 else "naive"
