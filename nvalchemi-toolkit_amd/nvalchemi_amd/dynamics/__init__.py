from .base import BaseDynamics, ConvergenceHook, DynamicsStage, FusedStage
from .integrators.nve import NVE
from .optimizers.fire import FIRE

__all__ = ["BaseDynamics", "ConvergenceHook", "DynamicsStage", "FusedStage", "NVE", "FIRE"]
