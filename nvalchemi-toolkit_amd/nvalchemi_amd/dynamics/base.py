"""The dynamics step contract.

Mirror of nvalchemi/dynamics/base.py for the single-process path: ``DynamicsStage``
(:120-157), ``_ConvergenceCriterion`` (:180-349), ``ConvergenceHook`` (:2215-2501),
``BaseDynamics.step/compute/run`` (:1815-1955).  One step is

    BEFORE_STEP -> BEFORE_PRE_UPDATE -> pre_update -> AFTER_PRE_UPDATE -> BEFORE_COMPUTE ->
    compute (= model(batch), outputs copied into the batch's existing energy/forces/stress)
    -> AFTER_COMPUTE -> BEFORE_POST_UPDATE -> post_update -> AFTER_POST_UPDATE -> AFTER_STEP
    -> convergence check (-> ON_CONVERGE) -> step_count += 1

The first step integrates with whatever ``batch.forces`` holds: ``run`` does not prime
forces.  Systems with ``status >= exit_status`` keep positions, velocities and cell through
a step; integrators that set ``_honors_active_mask`` get the mask (``self._active_mask``)
and skip those systems inside their kernels, everything else is saved and restored around
the update as the reference does.
"""

from __future__ import annotations

from collections import OrderedDict
from enum import Enum
from typing import Any, Callable, Literal

import torch
from pydantic import BaseModel, ConfigDict

from .. import _lib
from ..hooks._context import DynamicsContext
from ..hooks._registry import HookRegistryMixin
from ..models.base import BaseModelMixin


class DynamicsStage(Enum):
    BEFORE_STEP = 0
    BEFORE_PRE_UPDATE = 1
    AFTER_PRE_UPDATE = 2
    BEFORE_COMPUTE = 3
    AFTER_COMPUTE = 4
    BEFORE_POST_UPDATE = 5
    AFTER_POST_UPDATE = 6
    AFTER_STEP = 7
    ON_CONVERGE = 8


class _ConvergenceCriterion(BaseModel):
    """One criterion on a batch key: optional reduction inside each entry (``reduce_op`` over
    ``reduce_dims``), node-level values reduced per graph with max, then ``<= threshold``."""

    model_config = ConfigDict(arbitrary_types_allowed=True)

    key: str
    threshold: float
    reduce_dims: int | list[int] = -1
    reduce_op: Literal["min", "max", "norm", "mean", "sum"] | None = None
    custom_op: Callable[[torch.Tensor], torch.Tensor] | None = None

    def _reduce_within_entry(self, target: torch.Tensor) -> torch.Tensor:
        if self.reduce_op is None:
            return target
        if self.reduce_op == "min":
            return torch.amin(target, self.reduce_dims)
        if self.reduce_op == "max":
            return torch.amax(target, self.reduce_dims)
        if self.reduce_op == "norm":
            return torch.linalg.vector_norm(target, dim=self.reduce_dims)
        if self.reduce_op == "mean":
            return torch.mean(target, dim=self.reduce_dims)
        if self.reduce_op == "sum":
            return torch.sum(target, dim=self.reduce_dims)
        raise ValueError(f"Unknown reduce_op: {self.reduce_op!r}")

    @staticmethod
    def _scatter_reduce_to_graph(values: torch.Tensor, batch_idx: torch.Tensor, num_graphs: int) -> torch.Tensor:
        out = torch.full((num_graphs,), float("-inf"), dtype=values.dtype, device=values.device)
        out.scatter_reduce_(0, batch_idx.to(torch.long), values, reduce="amax", include_self=False)
        return out

    def _is_force_norm(self, target: torch.Tensor, batch) -> bool:
        return (self.reduce_op == "norm" and self.reduce_dims in (-1, 1) and target.dim() == 2
                and target.shape[1] == 3 and target.dtype in (torch.float32, torch.float64) and target.is_cuda
                and target.shape[0] == batch.num_nodes and batch.num_nodes != batch.num_graphs)

    @staticmethod
    def _force_norm_max(target: torch.Tensor, batch) -> torch.Tensor:
        """Per-system max of the atomic force norms in one pass."""
        fmax = torch.empty(batch.num_graphs, dtype=target.dtype, device=target.device)
        _lib.segment_fmax(target.contiguous(), batch.batch_idx, fmax)
        return fmax

    def reduced_values(self, batch) -> torch.Tensor | None:
        """The per-system values that ``__call__`` compares with the threshold, where they come from a kernel of this
        library (the maximum force norm); ``None`` for every other criterion."""
        target = getattr(batch, self.key, None)
        if target is None:
            raise KeyError("Key for convergence check not found;"
                           f" expected={self.key!r}, available={list(batch.keys())}")
        if self.custom_op is None and self._is_force_norm(target, batch):
            return self._force_norm_max(target, batch)
        return None

    def __call__(self, batch) -> torch.Tensor:
        target = getattr(batch, self.key, None)
        if target is None:
            raise KeyError("Key for convergence check not found;"
                           f" expected={self.key!r}, available={list(batch.keys())}")
        if self.custom_op is not None:
            return self.custom_op(target)
        if self._is_force_norm(target, batch):
            return self._force_norm_max(target, batch) <= self.threshold
        target = self._reduce_within_entry(target)
        is_node_level = target.shape[0] == batch.num_nodes and batch.num_nodes != batch.num_graphs
        if is_node_level:
            if target.dim() > 1:
                target = target.view(target.shape[0], -1).amax(dim=-1)
            reduced = self._scatter_reduce_to_graph(target, batch.batch_idx, batch.num_graphs)
        else:
            reduced = target.squeeze(-1) if target.dim() == 2 else target
        return reduced <= self.threshold


class ConvergenceHook:
    """AND of one or more criteria; optionally migrates ``batch.status`` of converged systems
    from ``source_status`` to ``target_status``."""

    def __init__(self, criteria=None, source_status: int | None = None, target_status: int | None = None,
                 frequency: int = 1) -> None:
        self.frequency = frequency
        self.stage = DynamicsStage.AFTER_STEP
        self.source_status = source_status
        self.target_status = target_status
        if criteria is None:
            self.criteria = [_ConvergenceCriterion(key="forces", threshold=0.05, reduce_op="norm", reduce_dims=-1)]
        elif isinstance(criteria, _ConvergenceCriterion):
            self.criteria = [criteria]
        elif isinstance(criteria, dict):
            self.criteria = [_ConvergenceCriterion(**criteria)]
        elif isinstance(criteria, (list, tuple)):
            normalized = []
            for item in criteria:
                if isinstance(item, dict):
                    normalized.append(_ConvergenceCriterion(**item))
                elif isinstance(item, _ConvergenceCriterion):
                    normalized.append(item)
                else:
                    raise TypeError("Each criterion must be a dict or _ConvergenceCriterion, "
                                    f"got {type(item).__name__}")
            self.criteria = normalized
        else:
            raise TypeError("criteria must be a dict, _ConvergenceCriterion, or list thereof, "
                            f"got {type(criteria).__name__}")

    @classmethod
    def from_fmax(cls, threshold: float = 0.05, source_status: int | None = None,
                  target_status: int | None = None, frequency: int = 1) -> "ConvergenceHook":
        return cls.from_forces(threshold=threshold, frequency=frequency, source_status=source_status,
                               target_status=target_status)

    @classmethod
    def from_forces(cls, threshold: float, frequency: int = 1, source_status: int | None = None,
                    target_status: int | None = None) -> "ConvergenceHook":
        return cls(criteria=[{"key": "forces", "threshold": threshold, "reduce_op": "norm", "reduce_dims": -1}],
                   frequency=frequency, source_status=source_status, target_status=target_status)

    @property
    def num_criteria(self) -> int:
        return len(self.criteria)

    def converged_mask(self, batch) -> torch.Tensor:
        """Boolean ``(B,)`` mask (no host synchronisation)."""
        mask = self.criteria[0](batch)
        for c in self.criteria[1:]:
            mask = mask & c(batch)
        return mask

    def evaluate(self, batch) -> torch.Tensor | None:
        """Indices of systems that satisfy every criterion, or ``None``."""
        mask = self.converged_mask(batch)
        idx = torch.where(mask)[0]
        return idx if idx.numel() > 0 else None

    def __call__(self, ctx: DynamicsContext, stage: Enum) -> None:
        batch = ctx.batch
        status = getattr(batch, "status", None)
        migrates = self.source_status is not None and self.target_status is not None and status is not None
        if (migrates and len(self.criteria) == 1 and status.dtype == torch.int64 and status.is_cuda
                and status.is_contiguous() and status.numel() >= batch.num_graphs):
            # one criterion on the maximum force norm: comparison and migration in one launch
            values = self.criteria[0].reduced_values(batch)
            if values is not None:
                _lib.status_migrate(values, self.criteria[0].threshold, status.view(-1), self.source_status,
                                    self.target_status)
                return
        mask = self.converged_mask(batch)  # (a missing key is an error whether or not anything migrates)
        if self.source_status is None or self.target_status is None:
            return
        if not hasattr(batch, "status") or batch.status is None:
            return
        flat = batch.status.view(-1)
        migrate = mask & (flat[: mask.shape[0]] == self.source_status)
        flat[: mask.shape[0]] = torch.where(migrate, torch.full_like(flat[: mask.shape[0]], self.target_status),
                                            flat[: mask.shape[0]])


class BaseDynamics(HookRegistryMixin):
    """Coordinates a model with an integrator over a ``Batch``.

    Subclasses override ``pre_update`` / ``post_update`` (and ``_init_state`` for per-system
    state) and declare ``__needs_keys__`` / ``__provides_keys__``.
    """

    _stage_type = DynamicsStage
    __needs_keys__: set[str] = set()
    __provides_keys__: set[str] = set()
    _mutable_fields: tuple[str, ...] = ("positions", "velocities", "cell")
    _honors_active_mask: bool = False
    #: graph-level fields that travel with a system (nvalchemi/dynamics/base.py:1336-1362)
    _bookkeeping_keys: dict[str, Callable[[int, torch.device], torch.Tensor]] = {
        "status": lambda n, dev: torch.zeros(n, 1, dtype=torch.long, device=dev),
        "system_id": lambda n, dev: torch.full((n, 1), -1, dtype=torch.long, device=dev),
    }
    _OUTPUT_KEY_TO_BATCH_ATTR: dict[str, str] = {"energy": "energy", "forces": "forces", "stress": "stress"}

    def __init__(self, model: BaseModelMixin, hooks: list | None = None, convergence_hook: Any = None,
                 n_steps: int | None = None, exit_status: int = 1, **kwargs: Any) -> None:
        if not isinstance(model, BaseModelMixin):
            raise TypeError(f"Expected a `BaseModelMixin` instance, got {type(model).__name__}."
                            " Please wrap your model with a `BaseModelMixin` subclass.")
        self.model = model
        self.step_count = 0
        if isinstance(convergence_hook, dict):
            convergence_hook = ConvergenceHook(**convergence_hook)
        self.convergence_hook = convergence_hook
        self.n_steps = n_steps
        self.exit_status = exit_status
        self.model_config = model.model_config
        self.current_hook_stage: DynamicsStage | None = None
        self.sampler = kwargs.pop("sampler", None)
        sinks = kwargs.pop("sinks", None)
        self.sinks = list(sinks) if sinks is not None else []
        self.refill_frequency: int = kwargs.pop("refill_frequency", 1)
        self.done = False
        self.active_batch = None
        self.global_rank = 0
        device_type = kwargs.pop("device_type", None)
        self.device_type: str = device_type if device_type else ("cuda" if torch.cuda.is_available() else "cpu")
        self._stream: torch.cuda.Stream | None = None
        self._stream_ctx: Any = None
        self._init_hooks(hooks)
        self._last_converged: torch.Tensor | None = None
        self._last_outputs: OrderedDict | None = None
        self._active_mask: torch.Tensor | None = None

    # ---- a stream of its own (nvalchemi/dynamics/base.py:686-742) ----------------------------------
    @property
    def device(self) -> torch.device:
        return torch.device(f"cuda:{torch.cuda.current_device()}") if self.device_type == "cuda" and \
            torch.cuda.is_available() else torch.device("cpu")

    @property
    def stream(self) -> "torch.cuda.Stream | None":
        """The stream made by ``with dynamics:`` (None outside the block or without a GPU)."""
        return self._stream

    def __enter__(self):
        """``with dynamics:`` -- a new stream of default priority becomes the current one: every kernel
        of the steps inside the block goes to it.  The caller orders it against the work that made
        the batch, as with any stream."""
        if self.device_type == "cuda" and torch.cuda.is_available():
            self._stream = torch.cuda.Stream(device=self.device)
            self._stream_ctx = torch.cuda.stream(self._stream)
            self._stream_ctx.__enter__()
        return self

    def __exit__(self, exc_type, exc_val, exc_tb) -> None:
        if self._stream_ctx is not None:
            self._stream_ctx.__exit__(exc_type, exc_val, exc_tb)
        self._stream = None
        self._stream_ctx = None

    @classmethod
    def register_bookkeeping_key(cls, key: str, init_fn: Callable[[int, torch.device], torch.Tensor]) -> None:
        """Register a graph-level field (``init_fn(n, device) -> (n, 1)`` tensor) that a fused stage
        creates on the batch when it is absent."""
        cls._bookkeeping_keys = {**cls._bookkeeping_keys, key: init_fn}

    def __add__(self, other: "BaseDynamics") -> "FusedStage":
        """``dyn_a + dyn_b``: a :class:`FusedStage` with status codes 0 and 1
        (nvalchemi/dynamics/base.py:1210-1243)."""
        if not isinstance(other, BaseDynamics):
            raise TypeError("Both operands of + must be BaseDynamics instances. "
                            f"other is {type(other).__name__}, not BaseDynamics.")
        return FusedStage(sub_stages=[(0, self), (1, other)])

    # ---- hooks ---------------------------------------------------------------------------------
    def _call_hooks(self, stage: DynamicsStage, batch) -> None:
        self.current_hook_stage = stage
        super()._call_hooks(stage, batch)

    def _build_context(self, batch) -> DynamicsContext:
        mask = None
        if self._last_converged is not None:
            mask = torch.zeros(batch.num_graphs, dtype=torch.bool, device=batch.positions.device)
            mask[self._last_converged] = True
        return DynamicsContext(batch=batch, step_count=self.step_count, model=self.model,
                               converged_mask=mask, global_rank=self.global_rank, workflow=self)

    def _open_hooks(self) -> None:
        seen: set[int] = set()
        for hook in self.hooks:
            if id(hook) not in seen and hasattr(hook, "__enter__"):
                seen.add(id(hook))
                hook.__enter__()

    def _close_hooks(self) -> None:
        seen: set[int] = set()
        for hook in self.hooks:
            if id(hook) in seen:
                continue
            seen.add(id(hook))
            if hasattr(hook, "__exit__"):
                hook.__exit__(None, None, None)
            elif hasattr(hook, "close"):
                hook.close()

    # ---- state ---------------------------------------------------------------------------------
    def _init_state(self, batch) -> None:
        """Allocate per-system integrator state (``self._state``); default: none."""

    def _ensure_state_initialized(self, batch) -> None:
        if not getattr(self, "_state_ready", False):
            self._init_state(batch)
            self._state_ready = True

    def pre_update(self, batch) -> None:
        """First half of the integration step (no-op here)."""

    def post_update(self, batch) -> None:
        """Second half of the integration step (no-op here)."""

    # ---- model evaluation ----------------------------------------------------------------------
    def _check_convergence(self, batch) -> torch.Tensor | None:
        if self.convergence_hook is None:
            return None
        return self.convergence_hook.evaluate(batch)

    def _validate_model_outputs(self, outputs) -> None:
        for key in self.__needs_keys__:
            if outputs.get(key) is None:
                raise RuntimeError(f"{type(self).__name__} requires '{key}' from the model, but the model "
                                   f"returned only {list(outputs.keys())}.")

    def compute(self, batch) -> OrderedDict:
        """``model(batch)``, validated against ``__needs_keys__``; known outputs are copied
        into the batch tensors that already exist (``copy_(value.view(target.shape))``)."""
        self._last_outputs = None
        if getattr(self.model, "accepts_output_buffers", False):
            # the model writes straight into the batch's result tensors: no second pass over them
            buffers = {k: getattr(batch, attr, None) for k, attr in self._OUTPUT_KEY_TO_BATCH_ATTR.items()}
            outputs = self.model(batch, out=buffers)
        else:
            outputs = self.model(batch)
        self._validate_model_outputs(outputs)
        detached: OrderedDict = OrderedDict()
        for key, value in outputs.items():
            detached[key] = value.detach() if isinstance(value, torch.Tensor) else value
        del outputs
        for out_key, batch_attr in self._OUTPUT_KEY_TO_BATCH_ATTR.items():
            value = detached.get(out_key)
            if value is not None:
                target = getattr(batch, batch_attr, None)
                if target is not None and not (value.data_ptr() == target.data_ptr()
                                               and value.numel() == target.numel()):
                    target.copy_(value.view(target.shape))
        pos = getattr(batch, "positions", None)
        if isinstance(pos, torch.Tensor) and pos.requires_grad:
            pos.requires_grad_(False)
        self._last_outputs = detached
        return detached

    # ---- the step ------------------------------------------------------------------------------
    def step(self, batch):
        self._ensure_state_initialized(batch)
        self._call_hooks(DynamicsStage.BEFORE_STEP, batch)

        active_mask: torch.Tensor | None = None
        status = getattr(batch, "status", None)
        if status is not None:
            flat = status.squeeze(-1) if status.dim() == 2 else status
            active_mask = flat[: batch.num_graphs] < self.exit_status
        self._active_mask = active_mask

        saved: dict[str, torch.Tensor] = {}
        node_mask = sys_mask = None
        if active_mask is not None and not self._honors_active_mask:
            node_mask = torch.repeat_interleave(active_mask, batch.num_nodes_per_graph.to(torch.long),
                                                output_size=batch.num_nodes)
            sys_mask = ~active_mask
            for field in self._mutable_fields:
                val = getattr(batch, field, None)
                if val is None:
                    continue
                if val.shape[0] == batch.num_nodes:
                    saved[field] = val[~node_mask].clone()
                elif val.shape[0] == batch.num_graphs:
                    saved[field] = val[sys_mask].clone()

        self._call_hooks(DynamicsStage.BEFORE_PRE_UPDATE, batch)
        self.pre_update(batch)
        self._call_hooks(DynamicsStage.AFTER_PRE_UPDATE, batch)
        self._call_hooks(DynamicsStage.BEFORE_COMPUTE, batch)
        self.compute(batch)
        self._call_hooks(DynamicsStage.AFTER_COMPUTE, batch)
        self._call_hooks(DynamicsStage.BEFORE_POST_UPDATE, batch)
        self.post_update(batch)
        self._call_hooks(DynamicsStage.AFTER_POST_UPDATE, batch)
        if saved:
            with torch.no_grad():
                for field, sv in saved.items():
                    val = getattr(batch, field)
                    if val.shape[0] == batch.num_nodes:
                        val[~node_mask] = sv
                    else:
                        val[sys_mask] = sv

        self._call_hooks(DynamicsStage.AFTER_STEP, batch)
        converged = self._check_convergence(batch)
        self._last_converged = converged
        if converged is not None:
            self._call_hooks(DynamicsStage.ON_CONVERGE, batch)
        self.step_count += 1
        return batch, converged

    # ---- replacing finished systems (nvalchemi/dynamics/base.py:1628-1680, 1957-2083) ------------
    def _sync_state_to_batch(self, remaining_indices: torch.Tensor, n_new: int, template_batch) -> None:
        """Keep ``self._state`` aligned with a batch whose systems were replaced: the rows of the
        remaining systems in order, then fresh default rows (``_make_new_state``) for the new ones."""
        if not hasattr(self, "_state"):
            return
        remaining = self._state.index_select(remaining_indices) if remaining_indices.numel() > 0 else None
        fresh = self._make_new_state(n_new, template_batch) if n_new > 0 else None
        if remaining is not None and fresh is not None:
            remaining.append(fresh)
            self._state = remaining
        elif remaining is not None:
            self._state = remaining
        elif fresh is not None:
            self._state = fresh
        else:
            del self._state
            self._state_ready = False

    def _overflow_to_sinks(self, batch, mask: torch.Tensor | None = None) -> None:
        """Write ``batch`` (its masked systems) to the first sink that is not full
        (nvalchemi/dynamics/base.py:878-901)."""
        for sink in self.sinks:
            if not sink.is_full:
                sink.write(batch, mask=mask)
                return
        raise RuntimeError(f"All sinks are full. Cannot store {batch.num_graphs} overflow samples.")

    def refill_check(self, batch, exit_status: int):
        """Drop the systems with ``status >= exit_status`` (after writing them to the first sink with
        room, when sinks are configured) and append replacements from
        ``self.sampler`` (an object with ``max_atoms``, ``max_edges``, ``max_batch_size``,
        ``exhausted`` and ``request_replacements_budget(atom_budget=, edge_budget=, max_count=)``
        returning a list of ``AtomicData``).  Returns the batch itself when nothing graduated, a new
        batch otherwise, or ``None`` when no system is left (``self.done`` is set once the sampler
        is exhausted too).  Bookkeeping fields of the remaining systems are carried over, those of
        the new ones take their defaults; per-system integrator state follows."""
        if self.sampler is None:
            raise RuntimeError("refill_check requires a sampler to be configured.")
        status = batch.status
        if status.dim() == 2:
            status = status.squeeze(-1)
        graduated = status >= exit_status
        if not graduated.any():
            return batch
        remaining_indices = torch.where(~graduated)[0]
        if self.sinks:
            self._overflow_to_sinks(batch, mask=graduated)
        n_remaining = remaining_indices.numel()
        result = batch.index_select(remaining_indices) if n_remaining > 0 else None
        sampler = self.sampler
        remaining_atoms = int(batch.num_nodes_per_graph[remaining_indices].sum()) if n_remaining > 0 else 0
        atom_budget = sampler.max_atoms - remaining_atoms if sampler.max_atoms is not None else None
        edges_per_graph = batch.num_edges_per_graph
        remaining_edges = int(edges_per_graph[remaining_indices].sum()) \
            if n_remaining > 0 and edges_per_graph.numel() > 0 else 0
        edge_budget = sampler.max_edges - remaining_edges if sampler.max_edges is not None else None
        max_new = sampler.max_batch_size - n_remaining if sampler.max_batch_size is not None else None
        replacements = sampler.request_replacements_budget(atom_budget=atom_budget, edge_budget=edge_budget,
                                                           max_count=max_new)
        from ..data.batch import Batch

        if result is not None and replacements:
            result.append(Batch.from_data_list(replacements, device=batch.device))
        elif result is None and replacements:
            result = Batch.from_data_list(replacements, device=batch.device)
        if result is not None:
            n_total = result.num_graphs
            for key, default_fn in self._bookkeeping_keys.items():
                new_tensor = default_fn(n_total, result.device)
                vals = getattr(result, key, None)
                if vals is not None:
                    vals = vals.unsqueeze(-1) if vals.dim() == 1 else vals
                    if vals.shape != new_tensor.shape:
                        raise RuntimeError(f"Bookkeeping key '{key}' has shape {vals.shape} after refill, "
                                           f"expected {new_tensor.shape}.")
                    new_tensor.copy_(vals)
                old = getattr(batch, key, None)
                if old is not None and n_remaining > 0:
                    src = old[remaining_indices]
                    new_tensor[:n_remaining] = src.unsqueeze(-1) if src.dim() == 1 else src
                result[key] = new_tensor
            self._sync_state_to_batch(remaining_indices, len(replacements), result)
            return result
        if sampler.exhausted:
            self.done = True
        self._sync_state_to_batch(remaining_indices, 0, batch)
        return None

    # ---- updates of selected systems only (nvalchemi/dynamics/base.py:2085-2212) ---------------
    def _run_masked(self, batch, mask: torch.Tensor, do_pre: bool, do_post: bool) -> None:
        """``pre_update`` and/or ``post_update`` for the systems with ``mask`` set; the others keep
        their mutable fields.  Integrators whose kernels take the mask get it; for the rest the
        fields of the unselected systems are saved and restored, as in the reference."""
        self._ensure_state_initialized(batch)
        mask = mask.to(device=batch.device, dtype=torch.bool)
        previous = self._active_mask
        if self._honors_active_mask:
            self._active_mask = mask
            try:
                if do_pre:
                    self.pre_update(batch)
                if do_post:
                    self.post_update(batch)
            finally:
                self._active_mask = previous
            return
        node_mask = mask[batch.batch_idx.to(torch.long)]
        sys_mask = ~mask
        saved: dict[str, torch.Tensor] = {}
        for field in self._mutable_fields:
            val = getattr(batch, field, None)
            if val is None:
                continue
            if val.shape[0] == batch.num_nodes:
                saved[field] = val[~node_mask].clone()
            elif val.shape[0] == batch.num_graphs:
                saved[field] = val[sys_mask].clone()
        self._active_mask = None
        try:
            if do_pre:
                self.pre_update(batch)
            if do_post:
                self.post_update(batch)
        finally:
            self._active_mask = previous
        with torch.no_grad():
            for field, sv in saved.items():
                val = getattr(batch, field)
                if val.shape[0] == batch.num_nodes:
                    val[~node_mask] = sv
                else:
                    val[sys_mask] = sv

    def masked_update(self, batch, mask: torch.Tensor) -> None:
        """``pre_update`` then ``post_update`` for the systems selected by ``mask (B,) bool``."""
        self._run_masked(batch, mask, True, True)

    def _masked_pre_update(self, batch, mask: torch.Tensor) -> None:
        self._run_masked(batch, mask, True, False)

    def _masked_post_update(self, batch, mask: torch.Tensor) -> None:
        self._run_masked(batch, mask, False, True)

    # ---- steady-state steps replayed from a captured HIP graph ---------------------------------------
    #: ``run`` replays a captured step when nothing in the step needs the host (see ``_graph_eligible``);
    #: set to False on an instance or a subclass to always step eagerly
    graph_replay: bool = True
    #: eager steps taken with an unchanged batch before a capture is attempted (the first steps size
    #: workspaces and settle the neighbor hook's row width, which involves the host)
    _GRAPH_WARM_STEPS = 2

    def _graph_eligible(self, batch) -> bool:
        """A step can be captured once and replayed when every step enqueues the same kernels on the same
        buffers and no decision is taken on the host: no convergence criterion (its result ends the run), no
        sampler, the plain ``step`` of this class, and only hooks that run on every step and declare
        ``graph_safe`` (their work is kernels on persistent buffers: the neighbor hook after its first build)."""
        if not self.graph_replay or self.convergence_hook is not None or self.sampler is not None:
            return False
        if type(self).step is not BaseDynamics.step or not torch.cuda.is_available():
            return False
        pos = getattr(batch, "positions", None)
        if not isinstance(pos, torch.Tensor) or pos.device.type != "cuda":
            return False
        if getattr(batch, "status", None) is not None and not self._honors_active_mask:
            return False  # (the save / restore of inactive systems indexes with masks: a host synchronisation)
        for hook in self.hooks:
            if getattr(hook, "frequency", 1) != 1 or not getattr(hook, "graph_safe", False):
                return False
        return True

    def _graph_key(self, batch) -> tuple:
        """What a captured step is tied to: the batch's tensors (a replay writes to the addresses it was
        captured with), its sizes, and whatever the hooks say their buffers are."""
        key: list = [id(batch), batch.num_nodes, batch.num_graphs, torch.cuda.current_stream().cuda_stream]
        for name in ("positions", "velocities", "forces", "energy", "atomic_masses", "batch_idx", "cell", "status"):
            t = getattr(batch, name, None)
            key.append((t.data_ptr(), tuple(t.shape)) if isinstance(t, torch.Tensor) else None)
        for name in ("batch_idx", "cell"):  # (kernels keep tables derived from these: an in-place edit ends the replay)
            t = getattr(batch, name, None)
            key.append(t._version if isinstance(t, torch.Tensor) else None)
        for hook in self.hooks:
            fn = getattr(hook, "graph_key", None)
            key.append((id(hook), fn() if callable(fn) else None))
        return tuple(key)

    def _capture(self, batch, body, key):
        """``body()`` captured as a HIP graph on a side stream; None if it cannot be (something in it needs the
        host, or it replaced one of the buffers that ``key`` names)."""
        from .. import _lib

        graph = torch.cuda.CUDAGraph()
        current = torch.cuda.current_stream()
        side = torch.cuda.Stream(device=current.device)
        # the captured kernels use the workspaces of the stream the eager steps ran on: replays are
        # launched into that stream, in order with its other work
        _lib.workspaces.share(current.device, current.cuda_stream, side.cuda_stream)
        count, converged, mask = self.step_count, self._last_converged, self._active_mask
        side.wait_stream(current)
        try:
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    body()
        except Exception:  # something in the step needs the host after all: stay eager for this batch
            return None
        finally:
            current.wait_stream(side)
            _lib.workspaces.unshare(current.device, side.cuda_stream)
            # (the capture ran nothing)
            self.step_count, self._last_converged, self._active_mask = count, converged, mask
        if self._graph_key(batch) != key:  # the body replaced a buffer: what was captured is already stale
            return None
        return graph

    def _graph_step(self, batch) -> bool:
        """One step by graph replay.  False: not possible now (the caller takes the step eagerly)."""
        if not self._graph_eligible(batch):
            self._graph_state = None
            return False
        key = self._graph_key(batch)
        st = getattr(self, "_graph_state", None)
        if st is None or st["key"] != key:
            st = self._graph_state = {"key": key, "warm": 0, "graph": None, "failed": False}
        if st["failed"]:
            return False
        if st["graph"] is None:
            if st["warm"] < self._GRAPH_WARM_STEPS:
                st["warm"] += 1
                return False
            graph = self._capture(batch, lambda: self.step(batch), key)
            if graph is None:
                st["failed"] = True
                return False
            st["graph"] = graph
        st["graph"].replay()
        self._last_converged = None
        self.step_count += 1
        return True

    #: whole steps, at most, in a graph that joins ``post_update`` of a step with ``pre_update`` of the next
    _GRAPH_JOINED_STEPS = 4

    def _joined_steps_possible(self, batch) -> bool:
        """Several steps may be captured as one graph whose inner boundaries are one launch each
        (``post_then_pre_update``) when nothing can run between two steps: no hook on the four stages around the
        boundary, and no status mask (it is worked out from ``batch.status`` at the start of every step)."""
        if not callable(getattr(self, "post_then_pre_update", None)) or getattr(batch, "status", None) is not None:
            return False
        boundary = (DynamicsStage.AFTER_POST_UPDATE, DynamicsStage.AFTER_STEP, DynamicsStage.BEFORE_STEP,
                    DynamicsStage.BEFORE_PRE_UPDATE)
        for hook in self.hooks:
            runs_on_stage = getattr(hook, "_runs_on_stage", None)
            if runs_on_stage is not None:
                if any(runs_on_stage(stage) for stage in boundary):
                    return False
            elif hook.stage in boundary:
                return False
        return True

    def _joined_steps(self, batch, k: int) -> None:
        """``k`` steps as ``step`` takes them when the stages around the step boundary are empty, with the
        boundaries inside taken as one launch.  (Called under graph capture only.)"""
        self._active_mask = None
        self.pre_update(batch)
        for j in range(k):
            self._call_hooks(DynamicsStage.AFTER_PRE_UPDATE, batch)
            self._call_hooks(DynamicsStage.BEFORE_COMPUTE, batch)
            self.compute(batch)
            self._call_hooks(DynamicsStage.AFTER_COMPUTE, batch)
            self._call_hooks(DynamicsStage.BEFORE_POST_UPDATE, batch)
            if j == k - 1:
                self.post_update(batch)
            elif not self.post_then_pre_update(batch):
                raise RuntimeError("no joined form of post_update and pre_update for this batch")
            self.step_count += 1

    def _graph_steps(self, batch, remaining: int) -> int:
        """As many steps by graph replay as one replay takes: up to ``_GRAPH_JOINED_STEPS`` of those that remain where
        steps can be joined (one graph per number of steps, made when first needed), else one; 0: not possible now."""
        k = min(remaining, self._GRAPH_JOINED_STEPS)
        st = getattr(self, "_graph_state", None)
        if (k >= 2 and st is not None and st.get("graph") is not None and not st.get("joined_failed")
                and self._graph_eligible(batch) and st["key"] == self._graph_key(batch)
                and self._joined_steps_possible(batch)):
            joined = st.setdefault("joined", {})
            if k not in joined:
                graph = self._capture(batch, lambda: self._joined_steps(batch, k), st["key"])
                if graph is None:
                    st["joined_failed"] = True
                    return 1 if self._graph_step(batch) else 0
                joined[k] = graph
            joined[k].replay()
            self._last_converged = None
            self.step_count += k
            return k
        return 1 if self._graph_step(batch) else 0

    def run(self, batch, n_steps: int | None = None):
        resolved = n_steps if n_steps is not None else self.n_steps
        if resolved is None:
            raise ValueError("No step count provided. Either pass `n_steps` to run() or set it at "
                             f"construction time via `{type(self).__name__}(..., n_steps=N)`.")
        self._open_hooks()
        try:
            taken = 0
            while taken < resolved:
                replayed = self._graph_steps(batch, resolved - taken)
                if replayed:
                    taken += replayed
                    continue
                batch, converged = self.step(batch)
                taken += 1
                if self.sampler is None and converged is not None and converged.numel() == batch.num_graphs:
                    break
        finally:
            self._close_hooks()
        return batch

    def __repr__(self) -> str:
        return (f"{type(self).__name__}(model={type(self.model).__name__}, n_steps={self.n_steps}, "
                f"step_count={self.step_count}, convergence_hook={self.convergence_hook!r}, "
                f"hooks={len(self.hooks)})")


class FusedStage(BaseDynamics):
    """Several dynamics on one batch with one model evaluation per step: each sub-stage updates the
    systems whose ``batch.status`` equals its code, convergence (or a per-system step budget,
    ``n_steps`` of the sub-stage) moves a system on to the next code, ``exit_status`` (default: the
    number of sub-stages) means done.  Mirror of nvalchemi/dynamics/base.py:2504-3337 for a batch
    supplied by the caller; in-flight refill from a sampler and ``torch.compile`` of the step are
    not available here.

    One step (``_step_impl``, :2928-3079): BEFORE_STEP hooks; per sub-stage BEFORE_PRE_UPDATE and the
    masked ``pre_update``; BEFORE_COMPUTE hooks of this stage (the neighbor list at the new
    positions), one ``compute``, AFTER_COMPUTE; per sub-stage the masked ``post_update`` and
    AFTER_POST_UPDATE; AFTER_STEP hooks (the convergence hooks migrate statuses there); step-budget
    migration; ON_CONVERGE per sub-stage; counters.  Returns the indices of the systems that reached
    ``exit_status`` during the step, or ``None``.  As in the reference, a sub-stage's step budget is
    counted on the status after the migrations of the step (:3023-3028): the step in which a system
    arrives in a sub-stage already counts towards that sub-stage's ``n_steps``.
    """

    def __init__(self, sub_stages: list[tuple[int, BaseDynamics]], *, entry_status: int = 0, exit_status: int = -1,
                 compile_step: bool = False, compile_kwargs: dict[str, Any] | None = None,
                 init_fn: Callable | None = None, **kwargs: Any) -> None:
        if compile_step:
            raise NotImplementedError("FusedStage(compile_step=True): the step is not compiled in this build")
        if not sub_stages:
            raise ValueError("FusedStage needs at least one sub-stage")
        device_types = {dyn.device_type for _, dyn in sub_stages}
        if len(device_types) > 1:
            per_stage = {code: dyn.device_type for code, dyn in sub_stages}
            raise ValueError(f"All sub-stages in a FusedStage must share the same device_type, but got: {per_stage}. "
                             "A FusedStage runs on a single device.")
        kwargs.setdefault("device_type", next(iter(device_types)))
        super().__init__(model=sub_stages[0][1].model, **kwargs)
        self.sub_stages = list(sub_stages)
        self.__needs_keys__ = set().union(*(dyn.__needs_keys__ for _, dyn in sub_stages))
        self.__provides_keys__ = set().union(*(dyn.__provides_keys__ for _, dyn in sub_stages))
        self.entry_status = entry_status
        self.compile_kwargs = compile_kwargs if compile_kwargs is not None else {}
        self.compile_step = False
        self.exit_status = len(self.sub_stages) if exit_status == -1 else exit_status
        self.convergence_check_frequency = 1
        self.init_fn = init_fn
        self.fused_hooks: list = []
        # every sub-stage gets the convergence hook that moves its systems to the next code
        for i, (source_code, source) in enumerate(self.sub_stages):
            if i + 1 < len(self.sub_stages):
                target_code = self.sub_stages[i + 1][0]
            else:
                if source.convergence_hook is None:
                    continue
                target_code = self.exit_status
            source.hooks = [h for h in source.hooks
                            if not (isinstance(h, ConvergenceHook) and getattr(h, "source_status", None) == source_code
                                    and getattr(h, "target_status", None) == target_code)]
            criteria = source.convergence_hook.criteria if source.convergence_hook is not None else None
            source.register_hook(ConvergenceHook(criteria=criteria, source_status=source_code,
                                                 target_status=target_code))
        for code, dyn in self.sub_stages:
            if dyn.n_steps is not None:
                BaseDynamics.register_bookkeeping_key(
                    f"n_steps_counter_{code}", lambda n, dev: torch.zeros(n, 1, dtype=torch.long, device=dev))

    def __repr__(self) -> str:
        stages = ", ".join(f"{code}:{type(dyn).__name__}" for code, dyn in self.sub_stages)
        return (f"FusedStage(sub_stages=[{stages}], entry_status={self.entry_status}, "
                f"exit_status={self.exit_status}, compiled=False, step_count={self.step_count})")

    def __add__(self, other: BaseDynamics) -> "FusedStage":
        if not isinstance(other, BaseDynamics):
            raise TypeError("Cannot append stage: other must be a BaseDynamics instance. "
                            f"Got {type(other).__name__} instead.")
        return FusedStage(sub_stages=list(self.sub_stages) + [(len(self.sub_stages), other)],
                          entry_status=self.entry_status, compile_kwargs=self.compile_kwargs)

    # ---- hooks ---------------------------------------------------------------------------------
    def register_fused_hook(self, hook) -> None:
        """A hook that sees the whole batch at this stage's BEFORE_STEP / AFTER_STEP."""
        if not isinstance(hook.frequency, int) or hook.frequency < 1:
            raise ValueError(f"Hook {hook!r} has frequency={hook.frequency!r}. "
                             "frequency must be a positive integer (>= 1).")
        self.fused_hooks.append(hook)

    def _call_fused_hooks(self, stage: DynamicsStage, batch) -> None:
        ctx = self._build_context(batch)
        for hook in self.fused_hooks:
            runs_on_stage = getattr(hook, "_runs_on_stage", None)
            if runs_on_stage is not None:
                if not runs_on_stage(stage):
                    continue
            elif stage != hook.stage:
                continue
            if self.step_count % hook.frequency == 0:
                hook(ctx, stage)

    def __enter__(self):
        """The fused stage's stream is also the one its sub-stages report
        (nvalchemi/dynamics/base.py:2790-2840)."""
        super().__enter__()
        for _, dyn in self.sub_stages:
            dyn._stream = self._stream
        return self

    def __exit__(self, exc_type, exc_val, exc_tb) -> None:
        for _, dyn in self.sub_stages:
            dyn._stream = None
        super().__exit__(exc_type, exc_val, exc_tb)

    def _open_hooks(self) -> None:
        super()._open_hooks()
        seen: set[int] = set()
        for hook in self.fused_hooks:
            if id(hook) not in seen and hasattr(hook, "__enter__"):
                seen.add(id(hook))
                hook.__enter__()
        for _, dyn in self.sub_stages:
            dyn._open_hooks()

    def _close_hooks(self) -> None:
        super()._close_hooks()
        seen: set[int] = set()
        for hook in self.fused_hooks:
            if id(hook) in seen:
                continue
            seen.add(id(hook))
            if hasattr(hook, "__exit__"):
                hook.__exit__(None, None, None)
            elif hasattr(hook, "close"):
                hook.close()
        for _, dyn in self.sub_stages:
            dyn._close_hooks()

    def _sync_state_to_batch(self, remaining_indices: torch.Tensor, n_new: int, template_batch) -> None:
        for _, dyn in self.sub_stages:
            dyn._sync_state_to_batch(remaining_indices, n_new, template_batch)

    def refill_check(self, batch, exit_status: int):
        result = super().refill_check(batch, exit_status)
        self._last_converged = None
        for _, dyn in self.sub_stages:
            dyn._last_converged = None
        return result

    def _ensure_bookkeeping_fields(self, batch) -> None:
        for key, default_fn in self._bookkeeping_keys.items():
            if getattr(batch, key, None) is None:
                batch[key] = default_fn(batch.num_graphs, batch.device)

    # ---- the step ------------------------------------------------------------------------------
    @staticmethod
    def _flat_status(batch) -> torch.Tensor:
        status = batch.status
        return status.squeeze(-1) if status.dim() == 2 else status

    def _step_impl(self, batch):
        self._ensure_bookkeeping_fields(batch)
        self._call_fused_hooks(DynamicsStage.BEFORE_STEP, batch)
        self._call_hooks(DynamicsStage.BEFORE_STEP, batch)
        for _, dyn in self.sub_stages:
            dyn._call_hooks(DynamicsStage.BEFORE_STEP, batch)

        status = self._flat_status(batch)
        masks: list[torch.Tensor] = []
        for code, dyn in self.sub_stages:
            mask = status == code
            masks.append(mask)
            dyn._call_hooks(DynamicsStage.BEFORE_PRE_UPDATE, batch)
            if mask.any():
                dyn._masked_pre_update(batch, mask)

        self._call_hooks(DynamicsStage.BEFORE_COMPUTE, batch)
        outputs = self.compute(batch)
        for key, tensor in outputs.items():
            if key not in ("forces", "energy"):
                batch[key] = tensor
        self._call_hooks(DynamicsStage.AFTER_COMPUTE, batch)
        for _, dyn in self.sub_stages:
            dyn._call_hooks(DynamicsStage.AFTER_COMPUTE, batch)

        for (code, dyn), mask in zip(self.sub_stages, masks):
            if mask.any():
                dyn._masked_post_update(batch, mask)
            dyn._call_hooks(DynamicsStage.AFTER_POST_UPDATE, batch)

        before = self._flat_status(batch).clone()
        for _, dyn in self.sub_stages:
            dyn._call_hooks(DynamicsStage.AFTER_STEP, batch)
        self._call_hooks(DynamicsStage.AFTER_STEP, batch)
        self._call_fused_hooks(DynamicsStage.AFTER_STEP, batch)

        # per-system step budgets of the sub-stages
        for i, (code, dyn) in enumerate(self.sub_stages):
            if dyn.n_steps is None:
                continue
            key = f"n_steps_counter_{code}"
            if getattr(batch, key, None) is None:
                batch[key] = torch.zeros(batch.num_graphs, 1, dtype=torch.long, device=batch.device)
            counter = getattr(batch, key)
            active = self._flat_status(batch) == code
            counter[active] += 1
            next_code = self.sub_stages[i + 1][0] if i + 1 < len(self.sub_stages) else self.exit_status
            migrate = active & (counter.squeeze(-1) >= dyn.n_steps)
            if migrate.any():
                batch.status.view(-1)[migrate] = next_code
                counter[migrate] = 0

        for mask, (_, dyn) in zip(masks, self.sub_stages):
            converged = dyn._check_convergence(batch)
            dyn._last_converged = None
            if converged is None:
                continue
            here = torch.zeros(batch.num_graphs, dtype=torch.bool, device=batch.device)
            here[converged] = True
            here &= mask
            if not here.any():
                continue
            dyn._last_converged = torch.where(here)[0]
            dyn._call_hooks(DynamicsStage.ON_CONVERGE, batch)

        self.step_count += 1
        for _, dyn in self.sub_stages:
            dyn.step_count += 1
        after = self._flat_status(batch)
        graduated = (before < self.exit_status) & (after >= self.exit_status)
        return batch, (torch.where(graduated)[0] if graduated.any() else None)

    def step(self, batch):
        return self._step_impl(batch)

    def __call__(self, batch):
        return self.step(batch)

    @staticmethod
    def all_complete(batch, exit_status: int) -> bool:
        status = getattr(batch, "status", None)
        if status is None:
            return False
        if status.dim() == 2:
            status = status.squeeze(-1)
        return bool((status == exit_status).all())

    def run(self, batch=None, n_steps: int | None = None):
        """Evaluate the model once (the first step integrates with real forces), then step until
        every system has ``exit_status`` or ``n_steps`` steps are done.  With a sampler configured
        (``FusedStage(..., sampler=, refill_frequency=)``) and ``batch=None``, the first batch comes
        from ``sampler.build_initial_batch()`` and every ``refill_frequency`` steps finished systems
        are replaced (:meth:`refill_check`); the run ends, returning ``None``, when no system is
        left (nvalchemi/dynamics/base.py:3162-3265)."""
        if batch is None:
            if self.sampler is None:
                raise ValueError("No batch provided and no sampler configured.")
            batch = self.sampler.build_initial_batch()
            if self.init_fn is not None:
                self.init_fn(batch)
            self.active_batch = batch
        self._ensure_bookkeeping_fields(batch)
        resolved = n_steps if n_steps is not None else self.n_steps
        self._open_hooks()
        try:
            self._call_hooks(DynamicsStage.BEFORE_COMPUTE, batch)
            self.compute(batch)
            self._call_hooks(DynamicsStage.AFTER_COMPUTE, batch)
            step_num = 0
            while True:
                batch, _ = self.step(batch)
                if self.sampler is not None and (step_num + 1) % self.refill_frequency == 0:
                    result = self.refill_check(batch, self.exit_status)
                    if result is None:
                        self.active_batch = None
                        return None
                    # (newcomers are first integrated with the forces they arrive with, as in the
                    # reference: no evaluation is inserted here)
                    batch = result
                    self.active_batch = batch
                elif self.sampler is None and (step_num + 1) % self.convergence_check_frequency == 0 \
                        and self.all_complete(batch, self.exit_status):
                    break
                step_num += 1
                if resolved is not None and step_num >= resolved:
                    break
            return batch
        finally:
            self._close_hooks()
