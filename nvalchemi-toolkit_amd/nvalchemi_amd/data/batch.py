"""``Batch``: many systems concatenated, with the reference's layout and accessors.

Host-side mirror of nvalchemi/data/batch.py:182 for the part the MD path uses: three
storage groups (``atoms``: tensors concatenated on dim 0 with per-system segment lengths;
``edges``: likewise; ``system``: one row per system), lazily derived int32
``batch_idx``/``batch_ptr`` (nvalchemi/data/level_storage.py:122,1447-1463,
batch.py:283-297), ``edge_ptr`` (batch.py:299-325), attribute reads that search the
groups in order and raise ``AttributeError`` when absent (batch.py:1112-1128), attribute
writes routed by key name with unknown names going to the system group
(level_storage.py:175-198,2102-2107).
"""

from __future__ import annotations

from typing import Any, Iterator

import torch

from . import buffer_kernels
from .atomic_data import EDGE_KEYS, NODE_KEYS, SYSTEM_KEYS, AtomicData


_NEIGHBOR_MATRIX_KEYS = ("neighbor_matrix", "neighbor_matrix_shifts", "num_neighbors")
_BUFFER_DTYPES = (torch.bool, torch.float32, torch.float64, torch.int32, torch.int64)


def _bool_on(mask: torch.Tensor, device) -> torch.Tensor:
    """``mask`` itself when it already is a bool tensor on ``device`` (so that in-place updates
    reach the caller), else a converted copy."""
    return mask if mask.dtype == torch.bool and mask.device == torch.device(device) else mask.to(
        device=device, dtype=torch.bool)


class SegmentedGroup:
    """Tensors whose leading dimension is a concatenation of per-system segments."""

    def __init__(self, data: dict[str, torch.Tensor], segment_lengths, device,
                 batch_ptr_capacity: int | None = None) -> None:
        """``batch_ptr_capacity``: entries to give the boundary tensor, so that ``put`` can append
        segments (``len + len(source) + 2`` are needed); the tensors may then hold more rows than the
        segments use (nvalchemi/data/level_storage.py:1289-1340)."""
        self._tensors = dict(data)
        self.segment_lengths = torch.as_tensor(segment_lengths).to(device=device, dtype=torch.int32)
        self.device = torch.device(device)
        self._batch_idx: torch.Tensor | None = None
        # boundaries; may hold more than len(self) + 1 entries (headroom for put)
        self._batch_ptr: torch.Tensor | None = None
        self._lengths_host: list[int] | None = None
        # True when the tensors may hold more rows than the segments use (empty, put, defrag)
        self._over_allocated = False
        if batch_ptr_capacity is not None:
            n = int(self.segment_lengths.shape[0])
            ends = torch.cumsum(self.segment_lengths, 0)
            store = torch.zeros(max(int(batch_ptr_capacity), n + 1), dtype=torch.int32, device=self.device)
            store[1: n + 1] = ends
            if n:
                store[n + 1:] = ends[-1]
            self._batch_ptr = store
            self._over_allocated = True

    def __len__(self) -> int:
        return int(self.segment_lengths.shape[0])

    def num_elements(self) -> int:
        if not self._over_allocated:
            for t in self._tensors.values():
                return int(t.shape[0])
        return int(sum(self.lengths_list()))

    def capacity(self) -> int:
        """Rows the tensors can hold."""
        for t in self._tensors.values():
            return int(t.shape[0])
        return 0

    def _ptr_store(self) -> torch.Tensor:
        if self._batch_ptr is None:
            ptr = torch.zeros(len(self) + 1, dtype=torch.int32, device=self.device)
            ptr[1:] = torch.cumsum(self.segment_lengths, 0)
            self._batch_ptr = ptr
        return self._batch_ptr

    def _invalidate(self) -> None:
        self._batch_idx = self._lengths_host = None
        if hasattr(self, "_edge_ptr"):
            del self._edge_ptr

    def _tight(self) -> dict[str, torch.Tensor]:
        if not self._over_allocated:
            return self._tensors
        n = self.num_elements()
        return {k: v[:n] for k, v in self._tensors.items()}

    def lengths_list(self) -> list[int]:
        if self._lengths_host is None:
            self._lengths_host = self.segment_lengths.tolist()
        return self._lengths_host

    @property
    def batch_ptr(self) -> torch.Tensor:
        store = self._ptr_store()
        n = len(self) + 1
        return store if store.shape[0] == n else store[:n]

    @property
    def batch_idx(self) -> torch.Tensor:
        if self._batch_idx is None:
            self._batch_idx = torch.repeat_interleave(
                torch.arange(len(self), dtype=torch.int32, device=self.device),
                self.segment_lengths.to(torch.long),
                output_size=self.num_elements(),
            )
        return self._batch_idx

    def __getitem__(self, key: str) -> torch.Tensor:
        return self._tensors[key]

    def __setitem__(self, key: str, value: torch.Tensor) -> None:
        self._tensors[key] = value

    def __contains__(self, key: str) -> bool:
        return key in self._tensors

    def __delitem__(self, key: str) -> None:
        del self._tensors[key]

    def keys(self):
        return self._tensors.keys()

    def items(self):
        return self._tensors.items()

    def mapped(self, fn, device) -> "SegmentedGroup":
        """A group over ``fn`` of every tensor (a copy or a move), bookkeeping included."""
        out = SegmentedGroup({k: fn(v) for k, v in self._tensors.items()}, fn(self.segment_lengths), device)
        out._over_allocated = self._over_allocated
        if self._over_allocated and self._batch_ptr is not None:
            out._batch_ptr = fn(self._batch_ptr)
        return out

    def select(self, idx: list[int]) -> "SegmentedGroup":
        """The segments ``idx`` (any order, repeats allowed) as a new group: one gather per tensor
        through an element index built from the boundaries."""
        lengths_host = self.lengths_list()
        new_lengths = [lengths_host[i] for i in idx]
        total = sum(new_lengths)
        sel = torch.tensor(idx, dtype=torch.long, device=self.device)
        lens = self.segment_lengths[sel].to(torch.long)
        starts = self.batch_ptr[sel].to(torch.long)
        new_starts = torch.cumsum(lens, 0) - lens
        rows = torch.repeat_interleave(starts - new_starts, lens, output_size=total) \
            + torch.arange(total, dtype=torch.long, device=self.device)
        out = SegmentedGroup({k: v.index_select(0, rows) for k, v in self._tensors.items()},
                             torch.tensor(new_lengths, dtype=torch.int32), self.device)
        out._lengths_host = new_lengths
        return out

    def concatenate(self, other: "SegmentedGroup") -> None:
        """Append the segments of ``other`` in place; keys that only one side has are dropped
        (derived data such as a neighbor matrix cannot be carried over a change of the batch)."""
        common = [k for k in self._tensors if k in other._tensors]
        mine, theirs = self._tight(), other._tight()
        self._tensors = {k: torch.cat([mine[k], theirs[k].to(self.device)], 0) for k in common}
        self.segment_lengths = torch.cat([self.segment_lengths, other.segment_lengths.to(self.device)])
        self._over_allocated = False
        self._batch_ptr = None
        self._invalidate()

    def extend_for_appended_graphs(self, n: int) -> None:
        """``n`` more systems without elements."""
        self.segment_lengths = torch.cat([self.segment_lengths,
                                          torch.zeros(n, dtype=torch.int32, device=self.device)])
        self._batch_ptr = None
        self._invalidate()

    # ---- fixed-capacity use (nvalchemi/data/level_storage.py:1778-1960) -----------------------
    def compute_put_per_system_fit_mask(self, source: "SegmentedGroup", source_mask: torch.Tensor,
                                        dest_mask: torch.Tensor | None, fit_mask: torch.Tensor) -> None:
        """``fit_mask[i]`` = segment ``i`` of ``source`` is masked and would fit behind this group's
        segments; all False when the boundary tensor has no headroom for ``len(source)`` more
        segments.  ``dest_mask`` is ignored.  Nothing is copied."""
        n_seg = len(source)
        if source_mask.shape[0] != n_seg:
            raise ValueError(f"source_mask shape {source_mask.shape[0]} != len(source) {n_seg}")
        if fit_mask.shape[0] != n_seg:
            raise ValueError(f"fit_mask shape {fit_mask.shape[0]} != {n_seg}")
        store = self._ptr_store()
        if store.shape[0] < len(self) + n_seg + 2:
            fit_mask.zero_()
            return
        buffer_kernels.compute_put_fit_mask_segmented(source.batch_ptr, _bool_on(source_mask, self.device), store,
                                                      len(self), self.capacity(), fit_mask)

    def put(self, src: "SegmentedGroup", mask: torch.Tensor, *, copied_mask: torch.Tensor | None = None) -> None:
        """Copy the masked segments of ``src`` that fit behind this group's segments, for the keys
        both sides have; ``copied_mask`` (or ``src._copied_mask``) receives which segments moved.
        One host read afterwards, for the new segment count.  Without headroom in the boundary
        tensor nothing is copied.  The boundary tensor is cut to the new count.

        The reference moves the float32 keys only (level_storage.py:1879-1884) and leaves the
        others zero in the destination; here every key of a supported dtype moves, except the
        per-atom neighbor data (matrix, its shifts, counts), which names atoms by their index in
        the source batch and has to be rebuilt.  ``neighbor_list`` moves as it is: ``Batch.put``
        re-bases it."""
        if not self._tensors or not src._tensors:
            raise ValueError("put requires non-empty source and dest")
        common = [k for k in self._tensors if k in src._tensors]
        if not common:
            raise ValueError("put requires at least one common attribute")
        n_seg = len(src)
        if mask.shape[0] != n_seg:
            raise ValueError(f"mask shape {mask.shape[0]} != num segments {n_seg}")
        mask = _bool_on(mask, self.device)
        if copied_mask is not None:
            if copied_mask.shape[0] != n_seg:
                raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {n_seg}")
            out_mask = _bool_on(copied_mask, self.device)
        else:
            out_mask = torch.zeros(n_seg, device=self.device, dtype=torch.bool)
            src._copied_mask = out_mask
        store = self._ptr_store()
        n_dest = len(self)
        if store.shape[0] < n_dest + n_seg + 2:
            return
        src_ptr = src.batch_ptr
        new_num_dest = None
        for key in common:
            src_t, dest_t = src._tensors[key], self._tensors[key]
            if key in _NEIGHBOR_MATRIX_KEYS or src_t.dtype != dest_t.dtype or src_t.dtype not in _BUFFER_DTYPES:
                continue
            new_num_dest = buffer_kernels.put_masked_segmented(src_t, src_ptr, mask, dest_t, store, n_dest, out_mask)
        if new_num_dest is not None:
            new_n = int(new_num_dest.item())
            self._batch_ptr = store[: new_n + 1].clone()
            self.segment_lengths = self._batch_ptr[1:] - self._batch_ptr[:-1]
            self._over_allocated = True
            self._invalidate()

    def defrag(self, copied_mask: torch.Tensor | None = None) -> "SegmentedGroup":
        """Drop the segments whose ``copied_mask`` is True in place: the others move to the front,
        the rows behind them are zeroed, the tensors keep their shape."""
        if not self._tensors:
            return self
        n_seg = len(self)
        if copied_mask is None:
            copied_mask = getattr(self, "_copied_mask", None)
            if copied_mask is None:
                raise ValueError("defrag requires copied_mask or a prior put")
        copied_mask = _bool_on(copied_mask, self.device)
        if copied_mask.shape[0] != n_seg:
            raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {n_seg}")
        ptr = self.batch_ptr
        original = ptr.clone()
        num_kept = None
        for key, t in self._tensors.items():
            if num_kept is None:
                num_kept = buffer_kernels.defrag_segmented(t, ptr, copied_mask)
            else:
                buffer_kernels.defrag_segmented(t, original.clone(), copied_mask)
        n_kept = int(num_kept.item())
        self.segment_lengths = (ptr[1:] - ptr[:-1])[:n_kept].clone()
        self._over_allocated = True
        self._invalidate()
        if hasattr(self, "_copied_mask"):
            del self._copied_mask
        return self

    def zero(self) -> None:
        """No segments, all rows zero; tensors and boundary headroom are kept."""
        for t in self._tensors.values():
            t.zero_()
        self.segment_lengths = torch.empty(0, dtype=torch.int32, device=self.device)
        if self._batch_ptr is not None:
            self._batch_ptr = torch.zeros(self._batch_ptr.shape[0], dtype=torch.int32, device=self.device)
        self._over_allocated = True
        self._invalidate()


class UniformGroup:
    """Tensors with exactly one leading row per system."""

    def __init__(self, data: dict[str, torch.Tensor], n: int, device) -> None:
        self._tensors = dict(data)
        self._n = int(n)
        self.device = torch.device(device)
        # True when the rows in use are counted apart from the tensors' shape (empty, defrag):
        # then put adds to the count
        self._counted = False

    def __len__(self) -> int:
        return self._n

    def capacity(self) -> int:
        """Rows the tensors can hold."""
        for t in self._tensors.values():
            return int(t.shape[0])
        return self._n

    def _tight(self) -> dict[str, torch.Tensor]:
        return {k: v[: self._n] for k, v in self._tensors.items()} if self._counted else self._tensors

    def __getitem__(self, key):
        return self._tensors[key]

    def __setitem__(self, key, value):
        self._tensors[key] = value

    def __contains__(self, key):
        return key in self._tensors

    def __delitem__(self, key):
        del self._tensors[key]

    def keys(self):
        return self._tensors.keys()

    def items(self):
        return self._tensors.items()

    def mapped(self, fn, device) -> "UniformGroup":
        """A group over ``fn`` of every tensor (a copy or a move), bookkeeping included."""
        out = UniformGroup({k: fn(v) for k, v in self._tensors.items()}, self._n, device)
        out._counted = self._counted
        return out

    def select(self, idx: list[int]) -> "UniformGroup":
        sel = torch.tensor(idx, dtype=torch.long, device=self.device)
        return UniformGroup({k: v.index_select(0, sel) for k, v in self._tensors.items()}, len(idx), self.device)

    def concatenate(self, other: "UniformGroup") -> None:
        common = [k for k in self._tensors if k in other._tensors]
        mine, theirs = self._tight(), other._tight()
        self._tensors = {k: torch.cat([mine[k], theirs[k].to(self.device)], 0) for k in common}
        self._n += len(other)
        self._counted = False

    def extend_for_appended_graphs(self, n: int) -> None:
        """``n`` more systems with zero rows (the other batch has no such group)."""
        self._tensors = {k: torch.cat([v, torch.zeros((n,) + tuple(v.shape[1:]), dtype=v.dtype, device=v.device)], 0)
                         for k, v in self._tight().items()}
        self._n += n
        self._counted = False

    # ---- fixed-capacity use (nvalchemi/data/level_storage.py:1067-1228) -----------------------
    def _dest_mask(self, dest_mask: torch.Tensor | None) -> torch.Tensor:
        cap = self.capacity()
        if dest_mask is None:
            return torch.zeros(cap, device=self.device, dtype=torch.bool)
        if dest_mask.shape[0] != cap:
            raise ValueError(f"dest_mask shape {dest_mask.shape[0]} != dest capacity {cap}")
        return _bool_on(dest_mask, self.device)

    def compute_put_per_system_fit_mask(self, source: "UniformGroup", source_mask: torch.Tensor,
                                        dest_mask: torch.Tensor | None, fit_mask: torch.Tensor) -> None:
        """``fit_mask[i]`` = row ``i`` of ``source`` is masked and an empty slot is left for it
        (``dest_mask`` True = occupied; None = every slot empty).  Nothing is copied."""
        n_src = len(source)
        if source_mask.shape[0] != n_src:
            raise ValueError(f"source_mask shape {source_mask.shape[0]} != len(source) {n_src}")
        if fit_mask.shape[0] != n_src:
            raise ValueError(f"fit_mask shape {fit_mask.shape[0]} != {n_src}")
        buffer_kernels.compute_put_fit_mask_per_system(_bool_on(source_mask, self.device), self._dest_mask(dest_mask),
                                                       fit_mask)

    def put(self, src: "UniformGroup", mask: torch.Tensor, *, copied_mask: torch.Tensor | None = None,
            dest_mask: torch.Tensor | None = None) -> None:
        """Copy the masked rows of ``src`` into the empty slots, for the keys both sides have;
        ``dest_mask`` and ``copied_mask`` (or ``src._copied_mask``) are updated in place.

        Every key fills the same slots.  (The reference hands the mask that the first key's copy
        has already updated to the next key, level_storage.py:1170-1181, so that a second key's
        rows land behind the first key's.)"""
        if not self._tensors or not src._tensors:
            raise ValueError("put requires non-empty source and dest")
        common = [k for k in self._tensors if k in src._tensors]
        if not common:
            raise ValueError("put requires at least one common attribute")
        n_src = len(src)
        if mask.shape[0] != n_src:
            raise ValueError(f"mask shape {mask.shape[0]} != len(src) {n_src}")
        mask = _bool_on(mask, self.device)
        if copied_mask is not None:
            if copied_mask.shape[0] != n_src:
                raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {n_src}")
            out_mask = _bool_on(copied_mask, self.device)
        else:
            out_mask = torch.zeros(n_src, device=self.device, dtype=torch.bool)
            src._copied_mask = out_mask
        given = dest_mask
        dest_mask = self._dest_mask(dest_mask)
        before = dest_mask.clone()
        for key in common:
            # every key starts from the same occupancy: the kernel marks the slots it fills
            slots = before.clone()
            buffer_kernels.put_masked_per_system(src._tensors[key][:n_src], mask, self._tensors[key], slots, out_mask)
            dest_mask.copy_(slots)
        if given is not None and given is not dest_mask:
            given.copy_(dest_mask)
        if self._counted:
            self._n += int(out_mask.sum().item())

    def defrag(self, copied_mask: torch.Tensor | None = None) -> "UniformGroup":
        """Drop the rows whose ``copied_mask`` is True in place: the others move to the front, the
        rows behind them are zeroed, the tensors keep their shape."""
        if not self._tensors:
            return self
        n_src = len(self)
        if copied_mask is None:
            copied_mask = getattr(self, "_copied_mask", None)
            if copied_mask is None:
                raise ValueError("defrag requires copied_mask or a prior put")
        copied_mask = _bool_on(copied_mask, self.device)
        if copied_mask.shape[0] != n_src:
            raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {n_src}")
        for t in self._tensors.values():
            buffer_kernels.defrag_per_system(t[:n_src], copied_mask.clone())
        self._n = int((~copied_mask).sum().item())
        self._counted = True
        if hasattr(self, "_copied_mask"):
            del self._copied_mask
        return self

    def zero(self) -> None:
        for t in self._tensors.values():
            t.zero_()
        self._n = 0
        self._counted = True


class _Storage:
    def __init__(self, groups: dict[str, Any]) -> None:
        self.groups = groups

    def __len__(self) -> int:
        for name in ("system", "atoms", "edges"):
            g = self.groups.get(name)
            if g is not None:
                return len(g)
        return 0


_GROUP_ORDER = ("atoms", "edges", "system")
_RESERVED = {"_storage", "device", "_neighbor_list_cutoff", "_neighbor_row_order", "_neighbor_search_cutoff",
             "_copied_mask"}


class Batch:
    """Concatenated systems.  Build with :meth:`from_data_list`."""

    def __init__(self, storage: _Storage, device) -> None:
        object.__setattr__(self, "_storage", storage)
        object.__setattr__(self, "device", torch.device(device))

    # ---- construction ------------------------------------------------------------------------
    @classmethod
    def from_data_list(cls, data_list: list[AtomicData], device=None) -> "Batch":
        if not data_list:
            raise ValueError("from_data_list needs at least one AtomicData")
        dev = torch.device(device) if device is not None else data_list[0].positions.device
        per_level: dict[str, dict[str, list[torch.Tensor]]] = {"atoms": {}, "edges": {}, "system": {}}
        key_level: dict[str, str] = {}
        for d in data_list:
            for k in d.keys():
                key_level.setdefault(k, d.level_of(k))
        for k, lvl in key_level.items():
            if not all(k in d for d in data_list):
                continue  # keep only keys every sample has (the reference drops ragged keys too)
            per_level[lvl][k] = [getattr(d, k) for d in data_list]
        n_nodes = torch.tensor([d.num_nodes for d in data_list], dtype=torch.int32)
        groups: dict[str, Any] = {}
        atoms = {k: torch.cat(v, 0).to(dev) for k, v in per_level["atoms"].items()}
        groups["atoms"] = SegmentedGroup(atoms, n_nodes, dev)
        if per_level["edges"]:
            first = next(iter(per_level["edges"].values()))
            n_edges = torch.tensor([t.shape[0] for t in first], dtype=torch.int32)
            edges = {}
            offsets = torch.cumsum(n_nodes, 0) - n_nodes
            for k, v in per_level["edges"].items():
                if k == "neighbor_list":  # the only index key offset on batching (batch.py:60,137-138)
                    v = [t + int(o) for t, o in zip(v, offsets)]
                edges[k] = torch.cat(v, 0).to(dev)
            groups["edges"] = SegmentedGroup(edges, n_edges, dev)
        system = {k: torch.cat(v, 0).to(dev) for k, v in per_level["system"].items()}
        groups["system"] = UniformGroup(system, len(data_list), dev)
        return cls(_Storage(groups), dev)

    @classmethod
    def _construct(cls, device, groups: dict[str, Any]) -> "Batch":
        return cls(_Storage(groups), device)

    @classmethod
    def empty(cls, *, num_systems: int, num_nodes: int, num_edges: int, template: "AtomicData | Batch | None" = None,
              device="cpu") -> "Batch":
        """A batch of zero systems over zeroed storage for ``num_systems`` systems, ``num_nodes``
        atoms and ``num_edges`` edges in total, with the keys, trailing shapes and dtypes of
        ``template`` (default: positions, atomic numbers and an energy).  Fill it with :meth:`put`
        (nvalchemi/data/batch.py:569-687)."""
        if num_systems < 0 or num_nodes < 0 or num_edges < 0:
            raise ValueError("num_systems, num_nodes, and num_edges must be non-negative")
        dev = torch.device(device)
        if template is None:
            template = AtomicData(torch.zeros(1, 3), torch.zeros(1, dtype=torch.long), energy=torch.tensor([[0.0]]))
        ref = cls.from_data_list([template], device=dev) if isinstance(template, AtomicData) else template
        groups: dict[str, Any] = {}
        for name, group in ref._storage.groups.items():
            # (the per-atom neighbor data of the template is left out: put never carries it, and at
            # K entries per atom it would be most of the allocation)
            keys = [k for k in group.keys() if k not in _NEIGHBOR_MATRIX_KEYS]
            if not keys:
                continue
            rows = num_systems if name == "system" else num_nodes if name == "atoms" else num_edges
            data = {k: torch.zeros((rows,) + tuple(group[k].shape[1:]), device=dev, dtype=group[k].dtype) for k in keys}
            if name == "system":
                g = UniformGroup(data, 0, dev)
                g._counted = True
            else:
                g = SegmentedGroup(data, torch.empty(0, dtype=torch.int32), dev)
                g._batch_ptr = torch.zeros(max(num_systems + 2, 2), dtype=torch.int32, device=dev)
                g._over_allocated = True
            groups[name] = g
        return cls(_Storage(groups), dev)

    @classmethod
    def empty_like(cls, batch: "Batch", *, device=None) -> "Batch":
        """A batch of zero systems and zero capacity with the keys of ``batch``."""
        return cls.empty(num_systems=0, num_nodes=0, num_edges=0, template=batch,
                         device=device if device is not None else batch.device)

    def zero(self) -> None:
        """Back to zero systems; the storage is zeroed and kept (nvalchemi/data/batch.py:690-737)."""
        for group in self._storage.groups.values():
            group.zero()
        self._drop_neighbor_stamps()

    def _drop_neighbor_stamps(self) -> None:
        for stamp in ("_neighbor_row_order", "_neighbor_search_cutoff"):
            object.__setattr__(self, stamp, None)

    # ---- sizes and index tensors ---------------------------------------------------------------
    @property
    def _atoms_group(self) -> SegmentedGroup | None:
        return self._storage.groups.get("atoms")

    @property
    def _edges_group(self) -> SegmentedGroup | None:
        return self._storage.groups.get("edges")

    @property
    def _system_group(self) -> UniformGroup | None:
        return self._storage.groups.get("system")

    @property
    def num_graphs(self) -> int:
        return len(self._storage)

    batch_size = num_graphs

    @property
    def num_nodes(self) -> int:
        a = self._atoms_group
        return a.num_elements() if a is not None else 0

    @property
    def num_edges(self) -> int:
        e = self._edges_group
        return e.num_elements() if e is not None else 0

    @property
    def system_capacity(self) -> int:
        """Systems the storage can hold (for a batch from :meth:`empty`)."""
        g = self._system_group
        return g.capacity() if g is not None else 0

    @property
    def batch_idx(self) -> torch.Tensor:
        a = self._atoms_group
        if a is None:
            return torch.tensor([], dtype=torch.long, device=self.device)
        return a.batch_idx

    @property
    def batch_ptr(self) -> torch.Tensor:
        a = self._atoms_group
        if a is None:
            return torch.zeros(1, dtype=torch.int32, device=self.device)
        return a.batch_ptr

    @property
    def edge_ptr(self) -> torch.Tensor:
        """Per-atom CSR pointer ``(N+1)`` int32 into the COO edge list (zeros without edges)."""
        N = self.num_nodes
        e = self._edges_group
        if e is None or e.num_elements() == 0:
            return torch.zeros(N + 1, dtype=torch.int32, device=self.device)
        cached = getattr(e, "_edge_ptr", None)
        if cached is not None:
            return cached
        src = e["neighbor_list"][:, 0].to(torch.long)
        counts = torch.bincount(src, minlength=N)
        ptr = torch.zeros(N + 1, dtype=torch.int32, device=self.device)
        ptr[1:] = torch.cumsum(counts, 0)
        return ptr

    @property
    def num_nodes_list(self) -> list[int]:
        a = self._atoms_group
        return a.lengths_list() if a is not None else []

    @property
    def num_edges_list(self) -> list[int]:
        e = self._edges_group
        return e.lengths_list() if e is not None else []

    @property
    def num_nodes_per_graph(self) -> torch.Tensor:
        a = self._atoms_group
        if a is None:
            return torch.tensor([], dtype=torch.long, device=self.device)
        return a.segment_lengths

    @property
    def num_edges_per_graph(self) -> torch.Tensor:
        e = self._edges_group
        if e is None:
            return torch.tensor([], dtype=torch.long, device=self.device)
        return e.segment_lengths

    @property
    def max_num_nodes(self) -> int:
        nodes = self.num_nodes_list
        return max(nodes) if nodes else 0

    # ---- key access ----------------------------------------------------------------------------
    def _find(self, key: str):
        for name in _GROUP_ORDER:
            g = self._storage.groups.get(name)
            if g is not None and key in g:
                return g
        return None

    def __getattr__(self, name: str) -> Any:
        if name.startswith("__"):
            raise AttributeError(name)
        storage = self.__dict__.get("_storage")
        if storage is not None:
            g = self._find(name)
            if g is not None:
                return g[name]
        raise AttributeError(f"Batch has no key {name!r}")

    def __setattr__(self, name: str, value: Any) -> None:
        if name in _RESERVED or not isinstance(value, torch.Tensor):
            object.__setattr__(self, name, value)
            return
        self[name] = value

    def __getitem__(self, key):
        """A tensor by key name, or -- for an int, slice, list or tensor -- the selected systems
        (an ``AtomicData`` for an int, a ``Batch`` otherwise)."""
        if not isinstance(key, str):
            if isinstance(key, int):
                return self.get_data(key if key >= 0 else self.num_graphs + key)
            return self.index_select(key)
        g = self._find(key)
        if g is None:
            raise KeyError(key)
        return g[key]

    # ---- selection and growth (nvalchemi/data/batch.py:816-874, 987-1072, 1138-1178) -----------
    def _normalize_index(self, idx) -> list[int]:
        import numpy as np

        if isinstance(idx, bool):
            raise IndexError("Unsupported index type: bool")
        if isinstance(idx, int):
            result = [idx]
        elif isinstance(idx, slice):
            result = list(range(self.num_graphs)[idx])
        elif isinstance(idx, torch.Tensor):
            if idx.dtype == torch.bool:
                result = idx.flatten().nonzero(as_tuple=False).flatten().tolist()
            elif idx.dtype.is_floating_point:
                raise IndexError(f"Tensor index must be integer or bool, got {idx.dtype}")
            else:
                result = idx.flatten().tolist()
        elif isinstance(idx, np.ndarray):
            result = (idx.flatten().nonzero()[0] if idx.dtype == np.bool_ else idx.flatten()).tolist()
        elif isinstance(idx, (list, tuple, range)):
            result = list(idx)
        else:
            raise IndexError(f"Unsupported index type: {type(idx).__name__}")
        if not result:
            raise IndexError("Index is empty")
        n = self.num_graphs
        result = [n + i if i < 0 else i for i in result]
        if any(i < 0 or i >= n for i in result):
            raise IndexError(f"graph index out of range for a batch of {n}")
        return result

    def index_select(self, idx) -> "Batch":
        """The systems ``idx`` as a new batch, gathered from the concatenated tensors; the atom
        indices of ``neighbor_list`` are re-based.  Keys that hold global atom indices by value
        (a neighbor matrix) are carried as they are and must be rebuilt, as in the reference."""
        ids = self._normalize_index(idx)
        groups: dict[str, Any] = {}
        atoms = self._atoms_group
        offset_diff = None
        if atoms is not None:
            new_atoms = atoms.select(ids)
            sel = torch.tensor(ids, dtype=torch.long, device=self.device)
            offset_diff = atoms.batch_ptr[sel] - new_atoms.batch_ptr[:-1]
            groups["atoms"] = new_atoms
        edges = self._edges_group
        if edges is not None:
            new_edges = edges.select(ids)
            if "neighbor_list" in new_edges and offset_diff is not None:
                corr = offset_diff[new_edges.batch_idx.to(torch.long)]
                new_edges["neighbor_list"] = new_edges["neighbor_list"] - corr.unsqueeze(1).to(
                    new_edges["neighbor_list"].dtype)
            groups["edges"] = new_edges
        system = self._system_group
        if system is not None:
            groups["system"] = system.select(ids)
        return Batch(_Storage(groups), self.device)

    def trim(self, copied_mask: torch.Tensor | None = None) -> "Batch | None":
        """A new batch without the systems whose ``copied_mask`` is True; ``None`` if none is left."""
        if copied_mask is None:
            copied_mask = getattr(self, "_copied_mask", None)
            if copied_mask is None:
                raise ValueError("trim requires copied_mask or a prior put")
        keep = ~copied_mask.to(device=self.device, dtype=torch.bool)
        if not bool(keep.any()):
            return None
        return self.index_select(torch.where(keep)[0])

    # ---- fixed-capacity use (nvalchemi/data/batch.py:876-985) ------------------------------------
    def put(self, src_batch: "Batch", mask: torch.Tensor, *, copied_mask: torch.Tensor | None = None,
            dest_mask: torch.Tensor | None = None) -> None:
        """Copy the systems of ``src_batch`` with ``mask`` set into this batch's free storage: the
        systems that fit on every level (a free system slot, room for their atoms, room for their
        edges) are copied, the others are not.  ``copied_mask`` -- or, without it,
        ``src_batch._copied_mask`` -- receives which ones moved, for :meth:`defrag` or :meth:`trim`
        of the source.  ``dest_mask`` (one flag per system slot, True = occupied) is updated in
        place; None treats every slot as empty."""
        device = self.device
        n = src_batch.num_graphs
        if mask.shape[0] != n:
            raise ValueError(f"mask shape {mask.shape[0]} != num_graphs {n}")
        mask = _bool_on(mask, device)
        if copied_mask is not None:
            if copied_mask.shape[0] != n:
                raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {n}")
            copy_mask = _bool_on(copied_mask, device)
        else:
            copy_mask = torch.zeros(n, device=device, dtype=torch.bool)
            object.__setattr__(src_batch, "_copied_mask", copy_mask)
        levels = []
        for mine, theirs in ((self._system_group, src_batch._system_group),
                             (self._atoms_group, src_batch._atoms_group),
                             (self._edges_group, src_batch._edges_group)):
            if mine is not None and theirs is not None and len(mine.keys()) and len(theirs.keys()):
                levels.append((mine, theirs))
        fit_mask = torch.ones(n, device=device, dtype=torch.bool)
        for mine, theirs in levels:
            level_fit = torch.empty(n, device=device, dtype=torch.bool)
            mine.compute_put_per_system_fit_mask(theirs, mask, dest_mask if isinstance(mine, UniformGroup) else None,
                                                 level_fit)
            fit_mask.logical_and_(level_fit)
        copy_mask.copy_(fit_mask)
        if copied_mask is not None and copy_mask is not copied_mask:
            copied_mask.copy_(copy_mask)
        atoms, edges = self._atoms_group, self._edges_group
        n_before = len(atoms) if atoms is not None else 0
        for mine, theirs in levels:
            if isinstance(mine, UniformGroup):
                mine.put(theirs, copy_mask, copied_mask=copy_mask, dest_mask=dest_mask)
            else:
                mine.put(theirs, copy_mask, copied_mask=copy_mask)
        # the copied edges name atoms by their index in the source: move them to where the atoms went
        src_atoms, src_edges = src_batch._atoms_group, src_batch._edges_group
        if atoms is not None and src_atoms is not None and edges is not None and src_edges is not None \
                and "neighbor_list" in edges and "neighbor_list" in src_edges and len(atoms) > n_before \
                and len(edges) == len(atoms):
            moved = torch.where(copy_mask)[0]
            new_ids = torch.arange(n_before, n_before + moved.numel(), device=device)
            delta = atoms.batch_ptr[new_ids] - src_atoms.batch_ptr[moved]
            eptr = edges.batch_ptr
            lo, hi = int(eptr[n_before]), int(eptr[n_before + moved.numel()])
            if hi > lo:
                owner = edges.batch_idx[lo:hi].to(torch.long) - n_before
                nl = edges["neighbor_list"]
                nl[lo:hi] += delta[owner].unsqueeze(1).to(nl.dtype)
        self._drop_neighbor_stamps()

    def defrag(self, copied_mask: torch.Tensor | None = None) -> "Batch":
        """Drop the systems whose ``copied_mask`` is True (default: the mask the last :meth:`put`
        left on this batch) in place.  The kept systems move to the front of the storage, which
        keeps its size; rows behind them are zeroed."""
        if copied_mask is None:
            copied_mask = getattr(self, "_copied_mask", None)
            if copied_mask is None:
                raise ValueError("defrag requires copied_mask or a prior put")
        if copied_mask.shape[0] != self.num_graphs:
            raise ValueError(f"copied_mask shape {copied_mask.shape[0]} != {self.num_graphs}")
        atoms, edges = self._atoms_group, self._edges_group
        rebase = atoms is not None and edges is not None and "neighbor_list" in edges and len(atoms.keys()) > 0
        if rebase:
            kept = torch.where(~_bool_on(copied_mask, self.device))[0]
            old_starts = atoms.batch_ptr[kept].clone()
        for group in (self._system_group, atoms, edges):
            if group is not None:
                group.defrag(copied_mask=copied_mask)
        if rebase and kept.numel() and edges.num_elements():
            # the kept systems' atoms moved forward: so do the indices their edges hold
            delta = atoms.batch_ptr[: kept.numel()] - old_starts
            nl = edges["neighbor_list"]
            nl[: edges.num_elements()] += delta[edges.batch_idx.to(torch.long)].unsqueeze(1).to(nl.dtype)
        if "_copied_mask" in self.__dict__:
            object.__delattr__(self, "_copied_mask")
        self._drop_neighbor_stamps()
        return self

    def append_data(self, data_list: list[AtomicData]) -> None:
        if not data_list:
            raise ValueError("No data provided to append.")
        self.append(Batch.from_data_list(data_list, device=self.device))

    def append(self, other: "Batch") -> None:
        """Append the systems of ``other`` in place.  A group that ``other`` lacks is extended with
        empty segments (atoms, edges) or zero rows (system)."""
        if other is self or other._storage is self._storage:
            raise ValueError("Cannot append a Batch that shares storage with the receiver (would corrupt both).  "
                             "Use batch.append(batch.clone()) instead.")
        total_nodes = self.num_nodes
        n_other = other.num_graphs
        for name, group in self._storage.groups.items():
            other_group = other._storage.groups.get(name)
            if other_group is None:
                group.extend_for_appended_graphs(n_other)
                continue
            if name == "edges" and "neighbor_list" in other_group and "neighbor_list" in group:
                shifted = SegmentedGroup(dict(other_group.items()), other_group.segment_lengths, other_group.device)
                shifted["neighbor_list"] = other_group["neighbor_list"] + total_nodes
                other_group = shifted
            group.concatenate(other_group)
        self._drop_neighbor_stamps()

    def __setitem__(self, key: str, value: torch.Tensor) -> None:
        g = self._find(key)
        if g is None:
            level = "atoms" if key in NODE_KEYS else "edges" if key in EDGE_KEYS else "system"
            g = self._storage.groups.get(level)
            if g is None:
                if level == "system":
                    g = UniformGroup({}, self.num_graphs, self.device)
                else:
                    raise RuntimeError(f"cannot store {key!r}: batch has no {level} group")
                self._storage.groups[level] = g
        g[key] = value

    def __contains__(self, key: str) -> bool:
        return self._find(key) is not None

    def __delitem__(self, key: str) -> None:
        g = self._find(key)
        if g is None:
            raise KeyError(key)
        del g[key]

    def __len__(self) -> int:
        return self.num_graphs

    def keys(self) -> Iterator[str]:
        for name in _GROUP_ORDER:
            g = self._storage.groups.get(name)
            if g is not None:
                yield from g.keys()

    def model_dump(self, exclude_none: bool = True) -> dict[str, torch.Tensor]:
        return {k: self[k] for k in self.keys()}

    def __repr__(self) -> str:
        return f"Batch(num_graphs={self.num_graphs}, num_nodes={self.num_nodes}, keys={sorted(self.keys())})"

    # ---- movement ------------------------------------------------------------------------------
    def _mapped(self, fn, device) -> "Batch":
        groups = {name: g.mapped(fn, device) for name, g in self._storage.groups.items()}
        out = Batch(_Storage(groups), device)
        if "_neighbor_list_cutoff" in self.__dict__:
            out._neighbor_list_cutoff = self._neighbor_list_cutoff
        return out

    def to(self, device) -> "Batch":
        dev = torch.device(device)
        return self._mapped(lambda t: t.to(dev), dev)

    def clone(self) -> "Batch":
        return self._mapped(lambda t: t.clone(), self.device)

    def cpu(self) -> "Batch":
        return self.to("cpu")

    def get_data(self, idx: int) -> AtomicData:
        """One system back out of the batch; ``neighbor_list`` is re-based to the system's atoms."""
        ptr = self.batch_ptr.tolist()
        a0, a1 = ptr[idx], ptr[idx + 1]
        fields = {}
        for k, v in self._atoms_group.items():
            if k in ("neighbor_matrix", "neighbor_matrix_shifts", "num_neighbors"):
                continue
            fields[k] = v[a0:a1]
        edges = self._edges_group
        if edges is not None and len(edges.keys()):
            eptr = edges.batch_ptr.tolist()
            e0, e1 = eptr[idx], eptr[idx + 1]
            for k, v in edges.items():
                fields[k] = v[e0:e1] - a0 if k == "neighbor_list" else v[e0:e1]
        sysg = self._system_group
        if sysg is not None:
            for k, v in sysg.items():
                fields[k] = v[idx:idx + 1]
        pos = fields.pop("positions")
        z = fields.pop("atomic_numbers")
        return AtomicData(pos, z, **fields)

    def to_data_list(self) -> list[AtomicData]:
        return [self.get_data(i) for i in range(self.num_graphs)]
