from ._context import DynamicsContext, HookContext
from ._registry import HookRegistryMixin
from .neighbor_list import NeighborListHook
from .periodic import WrapPeriodicHook, wrap_positions_into_cell

__all__ = ["DynamicsContext", "HookContext", "HookRegistryMixin", "NeighborListHook", "WrapPeriodicHook",
           "wrap_positions_into_cell"]
