from .nve import NVE
from .nvt_langevin import NVTLangevin

__all__ = ["NVE", "NVTLangevin"]
