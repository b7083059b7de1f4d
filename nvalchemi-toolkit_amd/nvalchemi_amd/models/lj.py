"""``LennardJonesModelWrapper``: the LJ potential as a model for the dynamics engine.

Mirror of nvalchemi/models/lj.py:82-488: same constructor, the same ``ModelConfig``
(outputs energy/forces/stress, active energy+forces, MATRIX neighbor format), the same
``adapt_input`` errors (``KeyError`` for a missing input, ``TypeError`` for a non-batch),
outputs ``energy (B,1)`` / ``forces (N,3)`` / optional ``stress (B,3,3) = -W/|det cell|``.
The per-system energy (fp64 sum of float32 atomic energies) and the per-system virial come
out of the same kernel launch instead of separate scatter passes.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import Any

import torch
from torch import nn

from ..data import AtomicData, Batch
from ._ops.lj import lj_energy_forces_system_batch
from .base import BaseModelMixin, ModelConfig, NeighborConfig, NeighborListFormat

__all__ = ["LennardJonesModelWrapper"]


class LennardJonesModelWrapper(nn.Module, BaseModelMixin):
    """Lennard-Jones potential ``u(r) = 4 eps [(sigma/r)^12 - (sigma/r)^6]``, plain
    truncation at ``cutoff``.

    Parameters
    ----------
    epsilon, sigma, cutoff : float
        Well depth, zero-crossing distance, cutoff radius.
    switch_width : float
        Width of the C2-continuous switching region below ``cutoff``; ``0.0`` (default) is plain
        truncation.  The pair energy is multiplied by ``1 - t^3 (10 - 15 t + 6 t^2)`` with
        ``t = (r - (cutoff - switch_width)) / switch_width``.
    half_list : bool
        ``True`` if the neighbor matrix holds each pair once.
    """

    def __init__(self, epsilon: float, sigma: float, cutoff: float, switch_width: float = 0.0,
                 half_list: bool = False) -> None:
        super().__init__()
        if not 0.0 <= switch_width <= cutoff:
            raise ValueError(f"switch_width {switch_width} outside [0, cutoff]")
        self.epsilon = epsilon
        self.sigma = sigma
        self.cutoff = cutoff
        self.switch_width = switch_width
        self.half_list = half_list
        self.model_config = ModelConfig(
            outputs=frozenset({"energy", "forces", "stress"}),
            active_outputs={"energy", "forces"},
            autograd_outputs=frozenset(),
            autograd_inputs=frozenset({"positions"}),
            required_inputs=frozenset(),
            optional_inputs=frozenset(),
            supports_pbc=True,
            needs_pbc=False,
            neighbor_config=NeighborConfig(cutoff=self.cutoff, format=NeighborListFormat.MATRIX,
                                           half_list=self.half_list),
        )
        self._eye_cells: torch.Tensor | None = None
        # per-system energies of the last evaluation, kept between calls of the same batch size
        # (nvalchemi/models/lj.py:190-203); the pair kernel writes them, callers get a copy
        self._energies_buf: torch.Tensor | None = None

    def _ensure_compute_buffers(self, B: int, dtype: torch.dtype, device: torch.device) -> None:
        buf = self._energies_buf
        if buf is None or buf.shape[0] != B or buf.dtype != dtype or buf.device != torch.device(device):
            self._energies_buf = torch.zeros(B, dtype=dtype, device=device)

    #: ``forward(batch, out={"forces": ..., "energy": ...})`` writes into the given tensors
    #: (used by the dynamics engine to fill the batch without a copy pass)
    accepts_output_buffers = True

    @property
    def embedding_shapes(self) -> dict[str, tuple[int, ...]]:
        return {}

    def compute_embeddings(self, data, **kwargs):
        raise NotImplementedError("LennardJonesModelWrapper does not produce embeddings.")

    def export_model(self, path, as_state_dict: bool = False) -> None:
        raise NotImplementedError

    # ------------------------------------------------------------------
    def adapt_input(self, data: AtomicData | Batch, **kwargs: Any) -> dict[str, Any]:
        """Collect the kernel inputs from *data* (no gradients are enabled: forces are
        analytic)."""
        input_dict: dict[str, Any] = {}
        for key in self.input_data():
            value = getattr(data, key, None)
            if value is None:
                raise KeyError(f"'{key}' required but not found in input data.")
            input_dict[key] = value
        if not isinstance(data, Batch):
            raise TypeError("LennardJonesModelWrapper requires a Batch input; got "
                            f"{type(data).__name__}.  Use Batch.from_data_list([data]) to wrap it.")
        input_dict["batch_idx"] = data.batch_idx.to(torch.int32)
        input_dict["ptr"] = data.batch_ptr.to(torch.int32)
        input_dict["num_graphs"] = data.num_graphs
        input_dict["fill_value"] = data.num_nodes
        input_dict["cells"] = getattr(data, "cell", None)
        input_dict["neighbor_matrix_shifts"] = getattr(data, "neighbor_matrix_shifts", None)
        return input_dict

    def adapt_output(self, model_output: Any, data: AtomicData | Batch) -> OrderedDict:
        output: OrderedDict = OrderedDict()
        output["energy"] = model_output["energy"]
        if "forces" in self.model_config.active_outputs:
            output["forces"] = model_output["forces"]
        if "stress" in self.model_config.active_outputs:
            if "virial" in model_output:
                if not hasattr(data, "cell") or data.cell is None:
                    raise ValueError("stress output requires cell for volume computation")
                volume = torch.det(data.cell).abs().view(-1, 1, 1)
                output["stress"] = -model_output["virial"] / volume
            elif "stress" in model_output:
                output["stress"] = model_output["stress"]
            else:
                raise RuntimeError("'stress' is in active_outputs but missing from model output")
        return output

    def output_data(self) -> set[str]:
        keys = {"energy"}
        if "forces" in self.model_config.active_outputs:
            keys.add("forces")
        if "stress" in self.model_config.active_outputs:
            keys.add("stress")
        return keys

    @staticmethod
    def _row_order_of(data, N: int, device) -> torch.Tensor | None:
        """The cell order the neighbor hook left on the batch for systems too large to stage
        in LDS (it keeps the pair kernel's gathers in the caches), if it fits this batch."""
        order = getattr(data, "_neighbor_row_order", None)
        if (isinstance(order, torch.Tensor) and order.shape == (N,) and order.dtype == torch.int32
                and order.device == device and order.is_contiguous()):
            return order
        return None

    @staticmethod
    def _pair_tiles_of(data, positions: torch.Tensor, neighbor_matrix: torch.Tensor):
        """What the neighbor hook left for the pair kernel of large systems, if it was made from exactly these
        positions (same storage, no write since) together with exactly this matrix."""
        tiles = getattr(data, "_neighbor_pair_tiles", None)
        if (isinstance(tiles, tuple) and len(tiles) == 7 and tiles[4] == positions.data_ptr()
                and tiles[5] == positions._version and tiles[6] == neighbor_matrix.data_ptr()
                and tuple(tiles[0].shape) == tuple(neighbor_matrix.shape)):
            return tiles[:4]
        return None

    @staticmethod
    def _search_cutoff_of(data, neighbor_matrix: torch.Tensor) -> float:
        """The radius the neighbor matrix in hand was searched with, if the builder left it on the
        batch for exactly this tensor; 0.0 (unknown) otherwise."""
        stamp = getattr(data, "_neighbor_search_cutoff", None)
        if (isinstance(stamp, tuple) and len(stamp) == 3 and stamp[1] == neighbor_matrix.data_ptr()
                and stamp[2] == tuple(neighbor_matrix.shape)):
            return float(stamp[0])
        return 0.0

    # ------------------------------------------------------------------
    def forward(self, data: AtomicData | Batch, out: dict | None = None, **kwargs: Any) -> OrderedDict:
        """``OrderedDict`` with ``energy (B,1)``, ``forces (N,3)`` and optionally
        ``stress (B,3,3)``.  Results are fresh tensors unless ``out`` supplies float32
        contiguous ``forces (N,3)`` / ``energy (B,1)`` tensors to fill."""
        inp = self.adapt_input(data, **kwargs)
        positions = inp["positions"]
        B = inp["num_graphs"]
        cells = inp.get("cells")
        shifts = inp.get("neighbor_matrix_shifts")
        if cells is None:
            if (self._eye_cells is None or self._eye_cells.shape[0] != B
                    or self._eye_cells.device != positions.device):
                self._eye_cells = torch.eye(3, dtype=positions.dtype, device=positions.device) \
                    .unsqueeze(0).expand(B, 3, 3).contiguous()
            cells = self._eye_cells
            shifts = None
        else:
            cells = cells.contiguous()
        compute_stress = "stress" in self.model_config.active_outputs
        N = positions.shape[0]
        bufs = {}
        if out:
            f_out, e_out = out.get("forces"), out.get("energy")
            if (isinstance(f_out, torch.Tensor) and f_out.shape == (N, 3) and f_out.dtype == positions.dtype
                    and f_out.is_contiguous() and f_out.device == positions.device):
                bufs["forces"] = f_out
            if (isinstance(e_out, torch.Tensor) and e_out.numel() == B and e_out.dtype == positions.dtype
                    and e_out.is_contiguous() and e_out.device == positions.device):
                bufs["system_energies"] = e_out.view(B)
        own_energy = "system_energies" not in bufs
        if own_energy:
            self._ensure_compute_buffers(B, positions.dtype, positions.device)
            bufs["system_energies"] = self._energies_buf
        neighbor_matrix = inp["neighbor_matrix"].contiguous()
        _, forces, sys_e, virials = lj_energy_forces_system_batch(
            positions.contiguous(), cells, neighbor_matrix,
            None if shifts is None else shifts.contiguous(), inp["num_neighbors"].contiguous(),
            inp["batch_idx"].contiguous(), inp["fill_value"], self.epsilon, self.sigma, self.cutoff,
            self.switch_width, self.half_list, compute_virial=compute_stress, out=bufs,
            row_order=self._row_order_of(data, N, positions.device),
            neighbor_list_cutoff=self._search_cutoff_of(data, neighbor_matrix),
            pair_tiles=self._pair_tiles_of(data, inp["positions"], neighbor_matrix))
        if own_energy:
            sys_e = sys_e.clone()  # a fresh tensor for the caller, as in the reference (:482)
        model_output: dict[str, Any] = {"energy": sys_e.unsqueeze(-1), "forces": forces}
        if virials is not None:
            model_output["virial"] = virials.view(B, 3, 3)
        return self.adapt_output(model_output, data)
