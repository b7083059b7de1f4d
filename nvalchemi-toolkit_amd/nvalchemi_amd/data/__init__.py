from .atomic_data import AtomicData
from .batch import Batch, SegmentedGroup, UniformGroup

__all__ = ["AtomicData", "Batch", "SegmentedGroup", "UniformGroup"]
