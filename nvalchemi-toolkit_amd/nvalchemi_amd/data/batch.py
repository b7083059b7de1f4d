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

from .atomic_data import EDGE_KEYS, NODE_KEYS, SYSTEM_KEYS, AtomicData


class SegmentedGroup:
    """Tensors whose leading dimension is a concatenation of per-system segments."""

    def __init__(self, data: dict[str, torch.Tensor], segment_lengths: torch.Tensor, device) -> None:
        self._tensors = dict(data)
        self.segment_lengths = segment_lengths.to(device=device, dtype=torch.int32)
        self.device = torch.device(device)
        self._batch_idx: torch.Tensor | None = None
        self._batch_ptr: torch.Tensor | None = None
        self._lengths_host: list[int] | None = None

    def __len__(self) -> int:
        return int(self.segment_lengths.shape[0])

    def num_elements(self) -> int:
        for t in self._tensors.values():
            return int(t.shape[0])
        return int(sum(self.lengths_list()))

    def lengths_list(self) -> list[int]:
        if self._lengths_host is None:
            self._lengths_host = self.segment_lengths.tolist()
        return self._lengths_host

    @property
    def batch_ptr(self) -> torch.Tensor:
        if self._batch_ptr is None:
            ptr = torch.zeros(len(self) + 1, dtype=torch.int32, device=self.device)
            ptr[1:] = torch.cumsum(self.segment_lengths, 0)
            self._batch_ptr = ptr
        return self._batch_ptr

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
        self._tensors = {k: torch.cat([self._tensors[k], other._tensors[k].to(self.device)], 0) for k in common}
        self.segment_lengths = torch.cat([self.segment_lengths, other.segment_lengths.to(self.device)])
        self._batch_idx = self._batch_ptr = self._lengths_host = None
        if hasattr(self, "_edge_ptr"):
            del self._edge_ptr

    def extend_for_appended_graphs(self, n: int) -> None:
        """``n`` more systems without elements."""
        self.segment_lengths = torch.cat([self.segment_lengths,
                                          torch.zeros(n, dtype=torch.int32, device=self.device)])
        self._batch_idx = self._batch_ptr = self._lengths_host = None


class UniformGroup:
    """Tensors with exactly one leading row per system."""

    def __init__(self, data: dict[str, torch.Tensor], n: int, device) -> None:
        self._tensors = dict(data)
        self._n = int(n)
        self.device = torch.device(device)

    def __len__(self) -> int:
        return self._n

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

    def select(self, idx: list[int]) -> "UniformGroup":
        sel = torch.tensor(idx, dtype=torch.long, device=self.device)
        return UniformGroup({k: v.index_select(0, sel) for k, v in self._tensors.items()}, len(idx), self.device)

    def concatenate(self, other: "UniformGroup") -> None:
        common = [k for k in self._tensors if k in other._tensors]
        self._tensors = {k: torch.cat([self._tensors[k], other._tensors[k].to(self.device)], 0) for k in common}
        self._n += len(other)

    def extend_for_appended_graphs(self, n: int) -> None:
        """``n`` more systems with zero rows (the other batch has no such group)."""
        self._tensors = {k: torch.cat([v, torch.zeros((n,) + tuple(v.shape[1:]), dtype=v.dtype, device=v.device)], 0)
                         for k, v in self._tensors.items()}
        self._n += n


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
        for stamp in ("_neighbor_row_order", "_neighbor_search_cutoff"):
            object.__setattr__(self, stamp, None)

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
    def to(self, device) -> "Batch":
        dev = torch.device(device)
        groups: dict[str, Any] = {}
        for name, g in self._storage.groups.items():
            data = {k: v.to(dev) for k, v in g.items()}
            if isinstance(g, SegmentedGroup):
                groups[name] = SegmentedGroup(data, g.segment_lengths, dev)
            else:
                groups[name] = UniformGroup(data, len(g), dev)
        out = Batch(_Storage(groups), dev)
        if "_neighbor_list_cutoff" in self.__dict__:
            out._neighbor_list_cutoff = self._neighbor_list_cutoff
        return out

    def clone(self) -> "Batch":
        groups: dict[str, Any] = {}
        for name, g in self._storage.groups.items():
            data = {k: v.clone() for k, v in g.items()}
            if isinstance(g, SegmentedGroup):
                groups[name] = SegmentedGroup(data, g.segment_lengths.clone(), self.device)
            else:
                groups[name] = UniformGroup(data, len(g), self.device)
        out = Batch(_Storage(groups), self.device)
        if "_neighbor_list_cutoff" in self.__dict__:
            out._neighbor_list_cutoff = self._neighbor_list_cutoff
        return out

    def cpu(self) -> "Batch":
        return self.to("cpu")

    def get_data(self, idx: int) -> AtomicData:
        """One system back out of the batch (atoms and system keys)."""
        ptr = self.batch_ptr.tolist()
        a0, a1 = ptr[idx], ptr[idx + 1]
        fields = {}
        for k, v in self._atoms_group.items():
            if k in ("neighbor_matrix", "neighbor_matrix_shifts", "num_neighbors"):
                continue
            fields[k] = v[a0:a1]
        sysg = self._system_group
        if sysg is not None:
            for k, v in sysg.items():
                fields[k] = v[idx:idx + 1]
        pos = fields.pop("positions")
        z = fields.pop("atomic_numbers")
        return AtomicData(pos, z, **fields)
