"""Choosing which systems of a dataset share a batch, by size.

Mirror of nvalchemi/dynamics/sampler.py:36-641 (``SizeAwareSampler``): the object that
``FusedStage(..., sampler=...)`` asks for its first batch and for replacements of finished systems.
Host logic only; the same choices as the reference for the same dataset and arguments:

* samples are grouped in bins of ``num_atoms // bin_width``, in dataset order inside a bin
  (``shuffle=True`` permutes every bin with Python's ``random``, bins taken in the order their
  first sample appears);
* the first batch takes one fitting sample per bin per round, bins in ascending order, until the
  atom / edge / count limits stop a whole round (:261-369);
* budgeted replacements go through the bins from the largest down and take every sample that
  still fits the remaining atom and edge budget (:423-493);
* a slot replacement takes the first fitting sample from the slot's own bin downwards (:371-421),
  or -- for several slots at once -- the fitting sample of lowest dataset index (:549-618).

Every sample handed out gets a ``system_id`` (a running number) as a system-level key.
"""

from __future__ import annotations

import random
from typing import Any, Iterator

import torch

from ..data.atomic_data import AtomicData
from ..data.batch import Batch

__all__ = ["SizeAwareSampler"]

_BYTES_PER_ATOM = 300  # storage of an atom's state plus a model's hidden features, a generous guess


class SizeAwareSampler:
    """See the module text.  ``dataset`` needs ``__len__``, ``__getitem__(i) -> (AtomicData, info)``
    and ``get_metadata(i) -> (num_atoms, num_edges)``."""

    def __init__(self, dataset: Any, max_atoms: int | None = None, max_edges: int | None = None,
                 max_batch_size: int | None = None, bin_width: int = 1, shuffle: bool = False,
                 max_gpu_memory_fraction: float = 0.8) -> None:
        if max_atoms is None and max_batch_size is None:
            raise ValueError("At least one of max_atoms or max_batch_size must be set.")
        if max_batch_size is not None and max_batch_size < 1:
            raise ValueError(f"max_batch_size must be >= 1, got {max_batch_size}")
        if bin_width < 1:
            raise ValueError(f"bin_width must be >= 1, got {bin_width}")
        if not 0.0 < max_gpu_memory_fraction <= 1.0:
            raise ValueError(f"max_gpu_memory_fraction must be in (0.0, 1.0], got {max_gpu_memory_fraction}")
        for method, what in (("__len__", "__len__"), ("__getitem__", "__getitem__"),
                             ("get_metadata", "get_metadata(idx) -> (num_atoms, num_edges)")):
            if not hasattr(dataset, method):
                raise TypeError(f"dataset must implement {what}")
        self._dataset = dataset
        self._max_atoms = max_atoms
        self._max_edges = max_edges
        self._max_batch_size = max_batch_size
        self._bin_width = bin_width
        self._shuffle = shuffle
        self._max_gpu_memory_fraction = max_gpu_memory_fraction
        self._sample_meta: list[tuple[int, int]] = []
        self._bins: dict[int, list[int]] = {}  # bin -> sample indices in serving order
        self._consumed: set[int] = set()
        self._next_system_id = 0
        self._meta_on_device: torch.Tensor | None = None
        self._consumed_on_device: torch.Tensor | None = None
        for idx in range(len(dataset)):
            n_atoms, n_edges = dataset.get_metadata(idx)
            if max_atoms is not None and n_atoms > max_atoms:
                raise RuntimeError(f"Sample {idx} has {n_atoms} atoms, exceeding max_atoms={max_atoms}. "
                                   "This sample can never fit in any batch.")
            if max_edges is not None and n_edges > max_edges:
                raise RuntimeError(f"Sample {idx} has {n_edges} edges, exceeding max_edges={max_edges}. "
                                   "This sample can never fit in any batch.")
            self._sample_meta.append((n_atoms, n_edges))
            self._bins.setdefault(n_atoms // bin_width, []).append(idx)
        if shuffle:
            for members in self._bins.values():
                random.shuffle(members)

    # ---- limits ---------------------------------------------------------------------------------
    @property
    def max_atoms(self) -> int | None:
        return self._max_atoms

    @property
    def max_edges(self) -> int | None:
        return self._max_edges

    @property
    def max_batch_size(self) -> int | None:
        return self._max_batch_size

    def _estimate_max_atoms_from_gpu(self) -> int | None:
        """Atoms that fit the device's memory by a rough rule (``max_gpu_memory_fraction`` of it,
        less a fifth of it for the model and the runtime, at 300 bytes an atom); None without a
        device."""
        if not torch.cuda.is_available():
            return None
        total = torch.cuda.get_device_properties(torch.cuda.current_device()).total_memory
        for_data = max(int(total * self._max_gpu_memory_fraction) - int(total * 0.2), 0)
        return max(for_data // _BYTES_PER_ATOM, 1)

    # ---- handing out ----------------------------------------------------------------------------
    def _open(self, bin_key: int) -> list[int]:
        """The samples of a bin that are still to be handed out, in serving order."""
        return [i for i in self._bins.get(bin_key, ()) if i not in self._consumed]

    def _hand_out(self, idx: int) -> AtomicData:
        data, _ = self._dataset[idx]
        data.add_system_property("system_id", torch.tensor([[self._next_system_id]], dtype=torch.long))
        self._next_system_id += 1
        self._consumed.add(idx)
        if self._consumed_on_device is not None:
            self._consumed_on_device[idx] = True
        return data

    def build_initial_batch(self) -> Batch:
        """The first batch, with ``status`` zero for every system.  ``RuntimeError`` when no sample
        can be taken."""
        atom_limit = self._max_atoms
        by_memory = self._estimate_max_atoms_from_gpu()
        if by_memory is not None:
            atom_limit = by_memory if atom_limit is None else min(atom_limit, by_memory)
        count_limit = self._max_batch_size if self._max_batch_size is not None else float("inf")
        chosen: list[AtomicData] = []
        atoms = edges = 0
        rotation = sorted(self._bins)
        while rotation and len(chosen) < count_limit:
            still_open: list[int] = []
            took_one = False
            for bin_key in rotation:
                if len(chosen) >= count_limit:
                    break
                members = self._open(bin_key)
                if not members:
                    continue
                for idx in members:
                    n_atoms, n_edges = self._sample_meta[idx]
                    if atom_limit is not None and atoms + n_atoms > atom_limit:
                        continue
                    if self._max_edges is not None and edges + n_edges > self._max_edges:
                        continue
                    chosen.append(self._hand_out(idx))
                    atoms += n_atoms
                    edges += n_edges
                    took_one = True
                    break
                still_open.append(bin_key)
            if not took_one or len(chosen) >= count_limit:
                break
            rotation = still_open
        if not chosen:
            raise RuntimeError("Cannot build initial batch: no samples available or constraints too tight.")
        batch = Batch.from_data_list(chosen, device=chosen[0].device)
        batch["status"] = torch.zeros(batch.num_graphs, 1, dtype=torch.long, device=batch.device)
        return batch

    def request_replacement(self, num_atoms: int, num_edges: int) -> AtomicData | None:
        """A sample of at most ``num_atoms`` atoms and ``num_edges`` edges, looked for from the bin of
        ``num_atoms`` downwards; None when there is none."""
        for bin_key in range(num_atoms // self._bin_width, -1, -1):
            for idx in self._open(bin_key):
                n_atoms, n_edges = self._sample_meta[idx]
                if n_atoms <= num_atoms and n_edges <= num_edges:
                    return self._hand_out(idx)
        return None

    def request_replacements_budget(self, atom_budget: int | None = None, edge_budget: int | None = None,
                                    max_count: int | None = None) -> list[AtomicData]:
        """Samples that together stay within the budgets (None = no limit), largest bins first."""
        out: list[AtomicData] = []
        for bin_key in sorted(self._bins, reverse=True):
            for idx in self._open(bin_key):
                if max_count is not None and len(out) >= max_count:
                    return out
                n_atoms, n_edges = self._sample_meta[idx]
                if atom_budget is not None and n_atoms > atom_budget:
                    continue
                if edge_budget is not None and n_edges > edge_budget:
                    continue
                out.append(self._hand_out(idx))
                if atom_budget is not None:
                    atom_budget -= n_atoms
                if edge_budget is not None:
                    edge_budget -= n_edges
        return out

    def request_replacements(self, node_counts: torch.Tensor, edge_counts: torch.Tensor) -> list[AtomicData | None]:
        """One replacement per slot: for slot ``k`` the sample of lowest dataset index with at most
        ``node_counts[k]`` atoms and ``edge_counts[k]`` edges that no earlier slot took (None when
        there is none).  The fit test runs on the device of the counts, one host read per slot."""
        device = node_counts.device
        if self._meta_on_device is None or self._meta_on_device.device != device:
            self._meta_on_device = torch.tensor(self._sample_meta, dtype=torch.long, device=device).reshape(-1, 2)
            taken = torch.zeros(len(self._sample_meta), dtype=torch.bool, device=device)
            if self._consumed:
                taken[torch.tensor(sorted(self._consumed), dtype=torch.long, device=device)] = True
            self._consumed_on_device = taken
        meta = self._meta_on_device
        fits = (meta[:, 0].unsqueeze(0) <= node_counts.unsqueeze(1)) \
            & (meta[:, 1].unsqueeze(0) <= edge_counts.unsqueeze(1))
        out: list[AtomicData | None] = []
        for k in range(len(node_counts)):
            candidates = (fits[k] & ~self._consumed_on_device).nonzero(as_tuple=False)
            out.append(self._hand_out(int(candidates[0, 0].item())) if candidates.numel() else None)
        return out

    # ---- what is left ---------------------------------------------------------------------------
    @property
    def exhausted(self) -> bool:
        return len(self._consumed) >= len(self._sample_meta)

    def __iter__(self) -> Iterator[int]:
        """The indices still to be handed out, bins in ascending order."""
        for bin_key in sorted(self._bins):
            yield from self._open(bin_key)

    def __len__(self) -> int:
        return len(self._dataset) - len(self._consumed)
