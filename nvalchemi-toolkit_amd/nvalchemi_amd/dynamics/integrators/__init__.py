from .nve import NVE
from .nvt_langevin import NVTLangevin
from .nvt_nose_hoover import NVTNoseHoover

__all__ = ["NVE", "NVTLangevin", "NVTNoseHoover"]
