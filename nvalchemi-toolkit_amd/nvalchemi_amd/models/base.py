"""Model-side contract of the MD path: neighbor-list configuration and the mixin through
which dynamics talks to a model.

Mirror of nvalchemi/models/base.py:38-228 (``NeighborListFormat``, ``NeighborConfig``,
``ModelConfig``), :594-619 (``input_data``) and :699-733 (``make_neighbor_hooks``), field
for field for what the path reads.
"""

from __future__ import annotations

from enum import Enum
from typing import Any

from pydantic import BaseModel, ConfigDict, Field, model_validator


class NeighborListFormat(str, Enum):
    """``COO``: edge list ``(E,2)`` rows ``[source, target]``; ``MATRIX``: dense
    ``neighbor_matrix (N,K)`` + ``num_neighbors (N)``."""

    COO = "coo"
    MATRIX = "matrix"


class NeighborConfig(BaseModel):
    """``cutoff``, ``format`` (default COO), ``half_list`` (each pair with i<j once),
    ``skin`` (Verlet skin; 0 = rebuild every step)."""

    cutoff: float
    format: NeighborListFormat = NeighborListFormat.COO
    half_list: bool = False
    skin: float = 0.0


class ModelConfig(BaseModel):
    """Capabilities (frozen sets) and runtime switches (``active_outputs``) of a model."""

    outputs: frozenset[str] = Field(default_factory=lambda: frozenset({"energy"}))
    autograd_outputs: frozenset[str] = Field(default_factory=frozenset)
    autograd_inputs: frozenset[str] = Field(default_factory=lambda: frozenset({"positions"}))
    required_inputs: frozenset[str] = Field(default_factory=frozenset)
    optional_inputs: frozenset[str] = Field(default_factory=frozenset)
    supports_pbc: bool = False
    needs_pbc: bool = False
    neighbor_config: NeighborConfig | None = None
    active_outputs: set[str] | None = None
    gradient_keys: set[str] = Field(default_factory=set)

    model_config = ConfigDict(extra="forbid")

    @model_validator(mode="after")
    def _default_active_outputs(self) -> "ModelConfig":
        if self.active_outputs is None:
            object.__setattr__(self, "active_outputs", set(self.outputs))
        return self

    @property
    def needs_neighborlist(self) -> bool:
        return self.neighbor_config is not None


class BaseModelMixin:
    """What :class:`~nvalchemi_amd.dynamics.base.BaseDynamics` requires of a model: a
    ``model_config`` attribute and a call ``model(batch) -> OrderedDict`` of outputs."""

    model_config: ModelConfig

    def set_config(self, key: str, value: Any) -> None:
        setattr(self.model_config, key, value)

    def input_data(self) -> set[str]:
        """Required input keys: positions, atomic_numbers, the neighbor keys of the
        configured format, ``pbc`` if needed, plus ``required_inputs``."""
        base = {"positions", "atomic_numbers"}
        nc = self.model_config.neighbor_config
        if nc is not None:
            if nc.format == NeighborListFormat.COO:
                base.add("neighbor_list")
            elif nc.format == NeighborListFormat.MATRIX:
                base |= {"neighbor_matrix", "num_neighbors"}
        if self.model_config.needs_pbc:
            base.add("pbc")
        return base | set(self.model_config.required_inputs)

    def output_data(self) -> set[str]:
        return set(self.model_config.active_outputs) & set(self.model_config.outputs)

    def make_neighbor_hooks(self, max_neighbors: int | None = None,
                            neighbor_list_method: str | None = None) -> list:
        """One :class:`NeighborListHook` at ``BEFORE_COMPUTE`` for this model's neighbor
        configuration, or an empty list."""
        from ..dynamics.base import DynamicsStage
        from ..hooks import NeighborListHook

        nc = self.model_config.neighbor_config
        if nc is None:
            return []
        return [NeighborListHook(nc, skin=nc.skin, max_neighbors=max_neighbors,
                                 method=neighbor_list_method, stage=DynamicsStage.BEFORE_COMPUTE)]
