"""``AtomicData``: one atomic system as plain tensors.

Host-side mirror of the fields the batched MD path reads from
nvalchemi/data/atomic_data.py:103 (schema), :352-387 (which keys live on atoms, edges and
the system), :482-510 (float fields follow ``positions.dtype``), :554-567 (velocities
default to zeros).  It is a plain container: no pydantic machinery, no serialisation.
"""

from __future__ import annotations

from typing import Any

import torch

# dim(0) == number of atoms
NODE_KEYS = frozenset({
    "atomic_masses", "positions", "forces", "charges", "node_embeddings", "atomic_numbers",
    "node_attrs", "atom_categories", "velocities", "momenta", "kinetic_energies",
    "neighbor_matrix", "neighbor_matrix_shifts", "num_neighbors",
})
# dim(0) == number of edges
EDGE_KEYS = frozenset({"shifts", "neighbor_list_shifts", "neighbor_list", "edge_embeddings"})
# one leading row per system
SYSTEM_KEYS = frozenset({
    "energy", "stress", "virial", "dipole", "charge", "graph_embeddings", "cell", "pbc", "spin",
})

# standard atomic weights (amu) for Z = 1..54; heavier elements need explicit masses
_ATOMIC_WEIGHTS = (
    0.0, 1.008, 4.002602, 6.94, 9.0121831, 10.81, 12.011, 14.007, 15.999, 18.998403163, 20.1797,
    22.98976928, 24.305, 26.9815385, 28.085, 30.973761998, 32.06, 35.45, 39.948, 39.0983, 40.078,
    44.955908, 47.867, 50.9415, 51.9961, 54.938044, 55.845, 58.933194, 58.6934, 63.546, 65.38,
    69.723, 72.630, 74.921595, 78.971, 79.904, 83.798, 85.4678, 87.62, 88.90584, 91.224, 92.90637,
    95.95, 97.0, 101.07, 102.90550, 106.42, 107.8682, 112.414, 114.818, 118.710, 121.760, 127.60,
    126.90447, 131.293,
)


def default_masses(atomic_numbers: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Standard atomic weight per atomic number (reference: atomic_data.py:86-100,512-530)."""
    z = atomic_numbers.to(torch.long)
    if z.numel() and (int(z.max()) >= len(_ATOMIC_WEIGHTS) or int(z.min()) < 0):
        raise ValueError("no default mass for Z > 54: pass atomic_masses explicitly")
    table = torch.tensor(_ATOMIC_WEIGHTS, dtype=dtype, device=atomic_numbers.device)
    return table[z]


class AtomicData:
    """A single system.  ``positions (n,3)`` and ``atomic_numbers (n)`` are required.

    System-level tensors carry a leading row of one: ``cell (1,3,3)``, ``pbc (1,3)``,
    ``energy (1,1)``.  A ``(3,3)`` cell or ``(3,)`` pbc is promoted.  Unknown keyword
    tensors are kept and classified by their leading dimension.
    """

    def __init__(self, positions: torch.Tensor, atomic_numbers: torch.Tensor, **fields: Any) -> None:
        positions = torch.as_tensor(positions)
        if positions.dim() != 2 or positions.shape[1] != 3:
            raise ValueError(f"positions must have shape (n, 3), got {tuple(positions.shape)}")
        if not positions.dtype.is_floating_point:
            raise TypeError("positions must be a floating-point tensor")
        atomic_numbers = torch.as_tensor(atomic_numbers)
        if atomic_numbers.dim() != 1 or atomic_numbers.shape[0] != positions.shape[0]:
            raise ValueError("atomic_numbers must have shape (n,)")
        if atomic_numbers.dtype.is_floating_point or atomic_numbers.dtype == torch.bool:
            raise TypeError("atomic_numbers must be an integer tensor")
        n = positions.shape[0]
        dtype = positions.dtype
        self._data: dict[str, torch.Tensor] = {"positions": positions, "atomic_numbers": atomic_numbers}
        self._levels: dict[str, str] = {}
        for key, value in fields.items():
            if value is None:
                continue
            value = torch.as_tensor(value)
            if key == "cell" and value.dim() == 2:
                value = value.unsqueeze(0)
            if key == "pbc":
                value = value.to(torch.bool)
                if value.dim() == 1:
                    value = value.unsqueeze(0)
            if key == "energy" and value.dim() < 2:
                value = value.reshape(1, 1)
            if value.dtype.is_floating_point:
                value = value.to(dtype)
            self._data[key] = value
        if "atomic_masses" not in self._data:
            self._data["atomic_masses"] = default_masses(atomic_numbers, dtype)
        if "velocities" not in self._data:
            self._data["velocities"] = torch.zeros_like(positions)
        for key in NODE_KEYS & self._data.keys():
            if self._data[key].shape[0] != n:
                raise ValueError(f"{key}: leading dimension must be the atom count {n}")
        if "cell" in self._data and tuple(self._data["cell"].shape) != (1, 3, 3):
            raise ValueError("cell must have shape (3,3) or (1,3,3)")
        if "pbc" in self._data and tuple(self._data["pbc"].shape) != (1, 3):
            raise ValueError("pbc must have shape (3,) or (1,3)")

    @property
    def num_nodes(self) -> int:
        return int(self._data["positions"].shape[0])

    def keys(self):
        return self._data.keys()

    def items(self):
        return self._data.items()

    def level_of(self, key: str) -> str:
        """``"atoms"``, ``"edges"`` or ``"system"`` (unknown keys: as declared by ``add_*_property``,
        else by leading dimension)."""
        if key in self._levels:
            return self._levels[key]
        if key in NODE_KEYS:
            return "atoms"
        if key in EDGE_KEYS:
            return "edges"
        if key in SYSTEM_KEYS:
            return "system"
        v = self._data[key]
        return "atoms" if v.dim() > 0 and v.shape[0] == self.num_nodes and self.num_nodes != 1 else "system"

    def __getattr__(self, name: str) -> torch.Tensor:
        data = self.__dict__.get("_data")
        if data is not None and name in data:
            return data[name]
        raise AttributeError(name)

    def __setattr__(self, name: str, value: Any) -> None:
        """A tensor assigned to a public name becomes a key of the system."""
        if name.startswith("_") or not isinstance(value, torch.Tensor):
            object.__setattr__(self, name, value)
        else:
            self._data[name] = value

    def __contains__(self, key: str) -> bool:
        return key in self._data

    @property
    def device(self) -> torch.device:
        return self._data["positions"].device

    def add_system_property(self, key: str, value: torch.Tensor) -> None:
        """``value`` (leading dimension one) as a system-level key, whatever its name
        (nvalchemi/data/atomic_data.py:667-670)."""
        self._data[key] = torch.as_tensor(value)
        self._levels[key] = "system"

    def add_node_property(self, key: str, value: torch.Tensor) -> None:
        self._data[key] = torch.as_tensor(value)
        self._levels[key] = "atoms"

    def add_edge_property(self, key: str, value: torch.Tensor) -> None:
        self._data[key] = torch.as_tensor(value)
        self._levels[key] = "edges"

    def to(self, device) -> "AtomicData":
        out = object.__new__(AtomicData)
        out._data = {k: v.to(device) for k, v in self._data.items()}
        out._levels = dict(self._levels)
        return out

    def clone(self) -> "AtomicData":
        out = object.__new__(AtomicData)
        out._data = {k: v.clone() for k, v in self._data.items()}
        out._levels = dict(self._levels)
        return out
