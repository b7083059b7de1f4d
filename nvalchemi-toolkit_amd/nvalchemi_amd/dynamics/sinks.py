"""Places to put systems that leave a running batch.

Mirror of nvalchemi/dynamics/sinks.py: the ``DataSink`` interface (:43-198), ``GPUBuffer``
(:201-534), a fixed-capacity batch in device memory filled with the masked-copy kernels, and
``HostMemory`` (:537-670), a list of systems in host memory.  The reference's third sink writes
Zarr stores; the Zarr package is not part of this build's environment and that sink is not
provided.
"""

from __future__ import annotations

from abc import ABC, abstractmethod

import torch

from ..data.atomic_data import AtomicData
from ..data.batch import Batch, SegmentedGroup

__all__ = ["DataSink", "GPUBuffer", "HostMemory"]


class DataSink(ABC):
    """Storage for systems: ``write`` (optionally only the masked systems), ``read`` everything
    back as one batch, ``zero`` to clear, ``len`` and ``capacity`` in systems."""

    @abstractmethod
    def write(self, batch: Batch, mask: torch.Tensor | None = None) -> None:
        """Store the systems of ``batch`` (those with ``mask`` set, when given).  ``RuntimeError``
        when they do not fit."""

    @abstractmethod
    def read(self) -> Batch:
        """Everything stored, as one batch.  ``RuntimeError`` when nothing is stored."""

    @abstractmethod
    def zero(self) -> None:
        """Forget everything stored."""

    @abstractmethod
    def __len__(self) -> int:
        """Systems stored."""

    @property
    @abstractmethod
    def capacity(self) -> int:
        """Systems the sink can hold."""

    @property
    def is_full(self) -> bool:
        return len(self) >= self.capacity

    def drain(self) -> Batch:
        """``read`` followed by ``zero``."""
        batch = self.read()
        self.zero()
        return batch

    @property
    def local_rank(self) -> int:
        return 0

    @property
    def global_rank(self) -> int:
        return 0


def _checked_mask(batch: Batch, mask: torch.Tensor | None) -> torch.Tensor | None:
    if mask is None:
        return None
    mask = mask.to(device=batch.device, dtype=torch.bool)
    if mask.shape[0] != batch.num_graphs:
        raise ValueError(f"mask length {mask.shape[0]} != num_graphs {batch.num_graphs}")
    return mask


class GPUBuffer(DataSink):
    """A batch of fixed capacity in device memory: ``capacity`` systems of at most ``max_atoms``
    atoms and ``max_edges`` edges each.  Allocated on the first ``write``, with the keys and dtypes
    of the batch written; later writes copy into it without allocating storage."""

    def __init__(self, capacity: int, max_atoms: int, max_edges: int, device: torch.device | str = "cuda") -> None:
        if not torch.cuda.is_available():
            raise RuntimeError("GPUBuffer requires an available GPU device: "
                               f"found {torch.cuda.device_count()} device(s)")
        dev = torch.device(device)
        if dev.type != "cuda":
            raise RuntimeError(f"GPUBuffer requires a GPU device, got: '{dev.type}'")
        self._capacity = capacity
        self._max_atoms = max_atoms
        self._max_edges = max_edges
        self._device = dev
        self._buffer: Batch | None = None
        self._copied_mask: torch.Tensor | None = None  # which systems of the last write were placed
        self._dest_mask: torch.Tensor | None = None  # which system slots are occupied

    def _ensure_buffer(self, template: Batch) -> None:
        if self._buffer is not None:
            return
        self._buffer = Batch.empty(num_systems=self._capacity, num_nodes=self._capacity * self._max_atoms,
                                   num_edges=self._capacity * self._max_edges, template=template,
                                   device=self._device)
        self._dest_mask = torch.zeros(self._capacity, dtype=torch.bool, device=self._device)
        self._restore_batch_ptr_capacity()

    def _restore_batch_ptr_capacity(self, incoming: int = 0) -> None:
        """Give the boundary tensors of the buffer their headroom back (a put cuts them to the
        segments in use): ``capacity + 2`` entries, the prefix kept, and room for a source batch
        of ``incoming`` systems.  (A put wants headroom for every system of the source batch, masked
        or not; with ``capacity + 2`` entries alone, sinks.py:318-343, a masked write from a batch
        of more systems than the buffer has free slots would copy nothing and say nothing.)"""
        if self._buffer is None:
            return
        want = max(self._capacity + 2, len(self) + incoming + 2)
        for group in self._buffer._storage.groups.values():
            if not isinstance(group, SegmentedGroup):
                continue
            bp = group._ptr_store()
            if bp.shape[0] < want:
                grown = torch.zeros(want, dtype=bp.dtype, device=bp.device)
                grown[: bp.shape[0]] = bp
                group._batch_ptr = grown

    def write(self, batch: Batch, mask: torch.Tensor | None = None) -> None:
        num_total = batch.num_graphs or 0
        if num_total == 0:
            return
        mask = _checked_mask(batch, mask)
        if mask is None:
            mask = torch.ones(num_total, dtype=torch.bool, device=batch.device)
        self._ensure_buffer(template=batch)
        num_to_write = int(mask.sum().item())
        if num_to_write == 0:
            return
        current = len(self)
        if current + num_to_write > self._capacity:
            raise RuntimeError(f"Buffer is full. Cannot add {num_to_write} samples to buffer "
                               f"with {current}/{self._capacity} samples.")
        most_atoms = int(batch.num_nodes_per_graph[mask].max().item())
        if most_atoms > self._max_atoms:
            raise RuntimeError(f"Atom capacity exceeded: a system has {most_atoms} atoms "
                               f"but buffer max_atoms={self._max_atoms}")
        if self._max_edges > 0 and batch.num_edges > 0:
            most_edges = int(batch.num_edges_per_graph[mask].max().item())
            if most_edges > self._max_edges:
                raise RuntimeError(f"Edge capacity exceeded: a system has {most_edges} edges "
                                   f"but buffer max_edges={self._max_edges}")
        self._copied_mask = torch.zeros(num_total, dtype=torch.bool, device=self._device)
        self._restore_batch_ptr_capacity(incoming=num_total)
        self._buffer.put(batch, mask, copied_mask=self._copied_mask, dest_mask=self._dest_mask)
        self._restore_batch_ptr_capacity()
        placed = int(self._copied_mask.sum().item())
        if placed != num_to_write:
            raise RuntimeError(f"GPUBuffer placed {placed} of {num_to_write} systems")

    def read(self) -> Batch:
        """The stored systems as a batch with tight tensors.  (When the buffer is full the
        reference returns a clone of the whole padded buffer, sinks.py:455-457; the systems are the
        same.)"""
        if self._buffer is None or len(self) == 0:
            raise RuntimeError("Cannot read from empty buffer.")
        return self._buffer.index_select(torch.arange(len(self), dtype=torch.long, device=self._device))

    def zero(self) -> None:
        if self._dest_mask is not None:
            self._dest_mask.zero_()
        if self._buffer is not None:
            self._buffer.zero()

    def __len__(self) -> int:
        return 0 if self._buffer is None else self._buffer.num_graphs

    @property
    def capacity(self) -> int:
        return self._capacity

    @property
    def device(self) -> torch.device:
        return self._device


class HostMemory(DataSink):
    """Systems kept one by one in host memory, whatever device they come from."""

    def __init__(self, capacity: int) -> None:
        self._capacity = capacity
        self._data_list: list[AtomicData] = []
        self._device = torch.device("cpu")

    def write(self, batch: Batch, mask: torch.Tensor | None = None) -> None:
        num_total = batch.num_graphs or 0
        if num_total == 0:
            return
        mask = _checked_mask(batch, mask)
        if mask is not None:
            num_selected = int(mask.sum().item())
            if num_selected == 0:
                return
            if num_selected < num_total:
                batch = batch.index_select(torch.nonzero(mask, as_tuple=True)[0])
        data_list = batch.to("cpu").to_data_list()
        if len(self._data_list) + len(data_list) > self._capacity:
            raise RuntimeError(f"Buffer is full. Cannot add {len(data_list)} samples "
                               f"to buffer with {len(self._data_list)}/{self._capacity} samples.")
        # slices of one transferred batch: give every system storage of its own
        self._data_list.extend(d.clone() for d in data_list)

    def read(self) -> Batch:
        if not self._data_list:
            raise RuntimeError("Cannot read from empty buffer.")
        return Batch.from_data_list(self._data_list, device=self._device)

    def zero(self) -> None:
        self._data_list.clear()

    def __len__(self) -> int:
        return len(self._data_list)

    @property
    def capacity(self) -> int:
        return self._capacity
