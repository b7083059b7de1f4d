from .base import BaseDynamics, ConvergenceHook, DynamicsStage, FusedStage
from .integrators.nve import NVE
from .integrators.nvt_langevin import NVTLangevin
from .integrators.nvt_nose_hoover import NVTNoseHoover
from .optimizers.fire import FIRE
from .optimizers.fire2 import FIRE2
from .sampler import SizeAwareSampler
from .sinks import DataSink, GPUBuffer, HostMemory

__all__ = ["BaseDynamics", "ConvergenceHook", "DynamicsStage", "FusedStage", "NVE", "NVTLangevin", "NVTNoseHoover", "FIRE", "FIRE2",
           "DataSink", "GPUBuffer", "HostMemory", "SizeAwareSampler"]
