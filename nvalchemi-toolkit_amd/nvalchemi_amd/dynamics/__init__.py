from .base import BaseDynamics, ConvergenceHook, DynamicsStage
from .integrators.nve import NVE
from .optimizers.fire import FIRE

__all__ = ["BaseDynamics", "ConvergenceHook", "DynamicsStage", "NVE", "FIRE"]
