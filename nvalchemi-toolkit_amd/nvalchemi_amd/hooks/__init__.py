from ._context import DynamicsContext, HookContext
from ._registry import HookRegistryMixin
from .neighbor_list import NeighborListHook

__all__ = ["DynamicsContext", "HookContext", "HookRegistryMixin", "NeighborListHook"]
