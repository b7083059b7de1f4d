from .base import BaseDynamics, ConvergenceHook, DynamicsStage, FusedStage
from .integrators.nve import NVE
from .integrators.nvt_langevin import NVTLangevin
from .optimizers.fire import FIRE

__all__ = ["BaseDynamics", "ConvergenceHook", "DynamicsStage", "FusedStage", "NVE", "NVTLangevin", "FIRE"]
