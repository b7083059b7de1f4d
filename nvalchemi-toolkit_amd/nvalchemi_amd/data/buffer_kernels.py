"""Masked copy and in-place compaction of per-system rows and per-system segments.

Mirror of the public functions of nvalchemi/data/buffer_kernels.py (``put_masked_per_system``
:1171, ``compute_put_fit_mask_per_system`` :1139, ``defrag_per_system`` :1294,
``put_masked_segmented`` :1442, ``compute_put_fit_mask_segmented`` :558, ``defrag_segmented``
:1700) with the same arguments, in-place effects, return values and errors; the Warp launches
behind them are HIP kernels here (``csrc/buffers.hip``).  The custom ops keep the reference's
names under this package's namespace.

Layouts: *per-system* tensors have one row per system, ``(num_systems, ...)``; *segmented*
tensors are flat, ``(total_elems, ...)``, with system ``i`` owning rows
``batch_ptr[i]:batch_ptr[i+1]``.  Supported dtypes: bool, float32, float64, int32, int64.
No call synchronises with the host.
"""

from __future__ import annotations

import math

import torch

from nvalchemi_amd import _lib

__all__ = [
    "compute_put_fit_mask_per_system",
    "compute_put_fit_mask_segmented",
    "defrag_per_system",
    "defrag_segmented",
    "put_masked_per_system",
    "put_masked_segmented",
]


def _two_d(t: torch.Tensor) -> torch.Tensor:
    return t if t.dim() == 2 else t.view(t.shape[0], math.prod(t.shape[1:]))


# ---------------------------------------------------------------------------------------------
# per-system rows
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("nvalchemi_amd::put_masked_per_system",
                         mutates_args=("source", "source_mask", "dest", "dest_mask", "source_data_copied"))
def put_masked_per_system_impl(source: torch.Tensor, source_mask: torch.Tensor, dest: torch.Tensor,
                               dest_mask: torch.Tensor, source_data_copied: torch.Tensor) -> None:
    if source.shape[0] == 0:
        return
    _lib.put_masked_per_system(source, source_mask, dest, dest_mask, source_data_copied)


def put_masked_per_system(source: torch.Tensor, source_mask: torch.Tensor, dest: torch.Tensor,
                          dest_mask: torch.Tensor, source_data_copied: torch.Tensor) -> None:
    """Copy the rows with ``source_mask`` set into ``dest``, into consecutive slots from the first
    one whose ``dest_mask`` is False; only as many as ``dest`` has empty slots.  ``dest_mask`` is set
    for the written slots and ``source_data_copied`` for the rows that moved."""
    return put_masked_per_system_impl(_two_d(source), source_mask, _two_d(dest), dest_mask, source_data_copied)


@torch.library.custom_op("nvalchemi_amd::compute_put_fit_mask_per_system", mutates_args=("fit_mask",))
def compute_put_fit_mask_per_system_impl(source_mask: torch.Tensor, dest_mask: torch.Tensor,
                                         fit_mask: torch.Tensor) -> None:
    _lib.put_fit_mask_per_system(source_mask, dest_mask, fit_mask)


def compute_put_fit_mask_per_system(source_mask: torch.Tensor, dest_mask: torch.Tensor,
                                    fit_mask: torch.Tensor) -> None:
    """``fit_mask[i]`` = row ``i`` is masked and would be moved by :func:`put_masked_per_system`."""
    if source_mask.shape[0] == 0:
        return
    compute_put_fit_mask_per_system_impl(source_mask, dest_mask, fit_mask)


@torch.library.custom_op("nvalchemi_amd::defrag_per_system", mutates_args=("source", "source_data_copied"))
def defrag_per_system_impl(source: torch.Tensor, source_data_copied: torch.Tensor) -> None:
    if source.shape[0] == 0:
        return
    _lib.defrag_per_system(_two_d(source), source_data_copied)


def defrag_per_system(source: torch.Tensor, source_data_copied: torch.Tensor) -> None:
    """Move the rows whose ``source_data_copied`` is False to the front (order kept), zero the rest,
    and leave ``source_data_copied[i] = (i >= number kept)``."""
    return defrag_per_system_impl(source, source_data_copied)


# ---------------------------------------------------------------------------------------------
# segments
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("nvalchemi_amd::compute_put_fit_mask_segmented", mutates_args=("fit_mask",))
def compute_put_fit_mask_segmented_impl(source_batch_ptr: torch.Tensor, source_mask: torch.Tensor,
                                        dest_batch_ptr: torch.Tensor, num_dest_segments: int,
                                        dest_capacity: int, fit_mask: torch.Tensor) -> None:
    _lib.put_fit_mask_segmented(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments,
                                dest_capacity, fit_mask)


def compute_put_fit_mask_segmented(source_batch_ptr: torch.Tensor, source_mask: torch.Tensor,
                                   dest_batch_ptr: torch.Tensor, num_dest_segments: int, dest_capacity: int,
                                   fit_mask: torch.Tensor) -> None:
    """``fit_mask[i]`` = segment ``i`` is masked and, laid out behind the destination's last segment
    after the masked segments before it, ends within ``dest_capacity`` rows.  All False when
    ``dest_batch_ptr`` has fewer than ``num_dest_segments + num_systems + 2`` entries."""
    num_systems = source_batch_ptr.shape[0] - 1
    if num_systems == 0:
        return
    if dest_batch_ptr.shape[0] < num_dest_segments + num_systems + 2:
        fit_mask.zero_()
        return
    compute_put_fit_mask_segmented_impl(source_batch_ptr, source_mask, dest_batch_ptr, num_dest_segments,
                                        dest_capacity, fit_mask)


@torch.library.custom_op("nvalchemi_amd::put_masked_segmented",
                         mutates_args=("source", "source_batch_ptr", "source_mask", "dest", "dest_batch_ptr",
                                       "source_data_copied", "new_num_dest"))
def put_masked_segmented_impl(source: torch.Tensor, source_batch_ptr: torch.Tensor, source_mask: torch.Tensor,
                              dest: torch.Tensor, dest_batch_ptr: torch.Tensor, num_dest_segments: int,
                              source_data_copied: torch.Tensor, new_num_dest: torch.Tensor) -> None:
    if source_batch_ptr.shape[0] - 1 == 0:
        return
    _lib.put_masked_segmented(source, source_batch_ptr, source_mask, dest, dest_batch_ptr, num_dest_segments,
                              source_data_copied, new_num_dest)


def put_masked_segmented(source: torch.Tensor, source_batch_ptr: torch.Tensor, source_mask: torch.Tensor,
                         dest: torch.Tensor, dest_batch_ptr: torch.Tensor, num_dest_segments: int,
                         source_data_copied: torch.Tensor) -> torch.Tensor | None:
    """Copy the masked segments that fit into ``dest`` behind its last segment and append their ends
    to ``dest_batch_ptr``; returns the new number of destination segments as a ``(1,)`` int32
    tensor (``None`` for a source without systems)."""
    source, dest = _two_d(source), _two_d(dest)
    num_systems = source_batch_ptr.shape[0] - 1
    if num_systems == 0:
        return None
    need = num_dest_segments + num_systems + 2
    new_num_dest = torch.empty(1, device=source.device, dtype=torch.int32)
    if dest_batch_ptr.shape[0] < need:
        raise ValueError("dest_batch_ptr must have size >= num_dest_segments + num_systems + 2 "
                         f"({need}); got {dest_batch_ptr.shape[0]}")
    put_masked_segmented_impl(source, source_batch_ptr, source_mask, dest, dest_batch_ptr, num_dest_segments,
                              source_data_copied, new_num_dest)
    return new_num_dest


@torch.library.custom_op("nvalchemi_amd::defrag_segmented",
                         mutates_args=("source", "source_batch_ptr", "num_kept"))
def defrag_segmented_impl(source: torch.Tensor, source_batch_ptr: torch.Tensor,
                          source_data_copied: torch.Tensor, num_kept: torch.Tensor) -> None:
    ptr = source_batch_ptr if source_batch_ptr.dtype == torch.int32 else source_batch_ptr.to(torch.int32)
    _lib.defrag_segmented(source, ptr, source_data_copied, num_kept)
    if ptr is not source_batch_ptr:
        source_batch_ptr.copy_(ptr)


def defrag_segmented(source: torch.Tensor, source_batch_ptr: torch.Tensor,
                     source_data_copied: torch.Tensor) -> torch.Tensor:
    """Move the segments whose ``source_data_copied`` is False to the front (order kept), zero the
    rows behind them, rewrite ``source_batch_ptr`` (new boundaries, then the kept row count in every
    later entry) and return the number of kept segments as a ``(1,)`` int32 tensor."""
    source = _two_d(source)
    num_kept = torch.empty(1, device=source.device, dtype=torch.int32)
    defrag_segmented_impl(source, source_batch_ptr, source_data_copied, num_kept)
    return num_kept
